"""The C-ABI library loads on a CPU-only host and exports every symbol the
public header declares (no compute calls here)."""
import ctypes
import os
import re

from flextrain_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared():
    names = set()
    inc = os.path.join(ROOT, "include")
    for fn in os.listdir(inc):
        if fn.endswith(".h"):
            text = open(os.path.join(inc, fn)).read()
            text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
            names |= set(re.findall(r"\b((?:fx_|create_|destroy_|get_stats|dispatch_|solve_|compute_buf)\w*)\s*\(", text))
    return names


def test_library_exports_every_declared_symbol():
    declared = _declared()
    assert declared, "no declarations found"
    handle = ctypes.CDLL(_lib.LIB_PATH)
    missing = [n for n in sorted(declared) if not hasattr(handle, n)]
    assert not missing, f"libflexhip.so lacks {missing}"


def test_python_binding_covers_the_header():
    declared = _declared()
    bound = set(_lib.exported_symbols())
    assert declared == bound, f"header-only: {declared - bound}; binding-only: {bound - declared}"
    _lib.lib()  # sets every argtypes/restype; raises if a symbol is missing


def test_version_string():
    assert _lib.lib().fx_version().decode().startswith("flexhip")


def test_fast_call_extension_loads_and_keeps_the_reference_conventions():
    """flextrain_amd._dispatch_fast (the METH_FASTCALL entry of
    helpers/matmul_dispatcher/src/dispatch_pyext.cpp:37-140): 24 positional arguments or TypeError,
    ValueError for a null context; bound to the dispatch_matmul of the loaded library."""
    import pytest

    from flextrain_amd import matmul_dispatcher as md

    fast = md._bind_fast()
    assert type(fast).__name__ == "builtin_function_or_method"
    with pytest.raises(TypeError):
        fast(1, 2, 3)
    with pytest.raises(TypeError):
        fast(*([0] * 25))
    null_ctx = [0, 0, 1, 1, 1, 0, 1, 0, 0, 1, 0, 0, 1, 0, 1, 0, 0, 2, 2, 2, 2, 0, 1.0, 0.0]
    with pytest.raises(ValueError):
        fast(*null_ctx)
    bad = list(null_ctx)
    bad[2] = "not a number"
    with pytest.raises(TypeError):
        fast(*bad)
    # a dimension that does not fit a C int is refused, not truncated; several bad arguments at
    # once report the first one (no conversion runs after an exception is set)
    big = list(null_ctx)
    big[0], big[2] = 1, 1 << 31
    with pytest.raises(OverflowError):
        fast(*big)
    big[3] = "x"
    with pytest.raises(OverflowError):
        fast(*big)
    two_bad = list(null_ctx)
    two_bad[2], two_bad[22] = "x", "y"
    with pytest.raises(TypeError):
        fast(*two_bad)
    # the module-level name of the reference's raw entry resolves to the same C function
    with pytest.raises(TypeError):
        md.matmul_fast(1)
    assert md.matmul_fast is fast


def test_dispatcher_constructs_without_the_fast_call_extension(monkeypatch):
    """The constructor does not need the C extension; only the first fast call does, and says so."""
    import pytest

    from flextrain_amd import matmul_dispatcher as md

    def missing():
        raise ImportError("no module named _dispatch_fast")

    monkeypatch.setattr(md, "_bind_fast", missing)
    disp = md.CublasLtDispatcher()
    assert disp.get_stats()["matmuls_called"] == 0
    with pytest.raises(ImportError, match="not built"):
        disp._fast(0)
