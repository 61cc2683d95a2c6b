"""Dry run of bench.py on the CPU: ``python -m tests.hostsim.bench_dry_run`` (about five minutes).

bench.py runs unchanged, at its real shapes, on top of the package, whose library is replaced by one in which
every launch returns at once (workspace sizes, tile heights, the dispatcher's bookkeeping, pinned memory
and the save-level solver stay real) and whose "device" is host memory (tests/hostsim/mode.py).  Vendor GEMMs
are replaced by their result shapes.  What this checks is the script itself: that every leg's set-up, launch
sequence, row bookkeeping and the final JSON line run through without a Python error, so that a mistake in
the script does not first show on the GPU.  The figures it prints mean nothing."""
from __future__ import annotations

import contextlib
import ctypes
import io
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
REAL = ("_ws_bytes", "fx_version", "fx_host_alloc", "fx_host_free", "fx_stream_ring", "create_dispatcher", "destroy_dispatcher",
        "get_stats", "solve_scheduler", "compute_buf_size", "fx_grouped_rows_tile_height", "hostsim_")


def main(argv):
    os.environ["FLEXTRAIN_HOSTSIM"] = "1"
    for path in (ROOT, os.path.join(ROOT, "tests")):
        if path not in sys.path:
            sys.path.insert(0, path)
    import torch
    from hostsim import mode

    mode.ACTIVE = True
    mode.activate()
    from flextrain_amd import _lib

    real, stubs = _lib._lib, {}

    class LaunchesDoNothing:
        def __getattr__(self, name):
            fn = getattr(real, name, None)
            if fn is not None and any(k in name for k in REAL):
                return fn
            if name == "fx_probe_ws_bytes":                  # the probe kernels are not part of the simulated library
                return lambda: 1 << 20
            if name not in stubs:
                restype, argtypes = _lib._SIGNATURES[name]
                stubs[name] = ctypes.CFUNCTYPE(restype, *argtypes)(lambda *a: 0)     # a C function pointer, as the real entry is
            return stubs[name]

    _lib._lib = LaunchesDoNothing()
    mode._Event.elapsed_time = lambda self, other: 1.0

    def shape_only(*a, **k):
        if k.get("out") is not None:
            return k["out"]
        x, y = a[-2], a[-1]
        return torch.empty(*x.shape[:-1], y.shape[-1], dtype=x.dtype)

    torch.matmul = torch.mm = shape_only
    torch.Tensor.__matmul__ = lambda a, b: shape_only(a, b)
    torch.addmm = lambda c, a, b, **k: k.get("out", c)
    torch.Tensor.addmm_ = lambda self, a, b, **k: self

    import bench

    sys.argv = ["bench.py", "--steps", "2", "--warmup", "1", "--no-cpu"] + list(argv)
    t0 = time.time()
    out = io.StringIO()
    with contextlib.redirect_stdout(out):
        bench.main()
    result = json.loads(out.getvalue().strip().splitlines()[-1])
    failed = [r for r in result["ops"] if "error" in r and not r["op"].startswith("mfma_probe")]
    print(f"{len(result['ops'])} rows in {time.time() - t0:.0f} s; failed legs: {[r['op'] + ': ' + r['error'] for r in failed] or 'none'}")
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "roofline", "config", "summary"):
        assert key in result, key
    return 1 if failed else 0


if __name__ == "__main__":
    sys.exit(main(sys.argv[1:]))
