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
