#!/usr/bin/env python3
"""Writes tests/golden/scheduler_cases.json: inputs and the outputs of the REAL reference
solver (helpers/transmission_scheduler/transmission_scheduler/transmission_scheduler.c),
compiled from the reference tree by ``make -C oracle`` into oracle/_ref/ — once as the
reference builds it (AVX2 path) and once with its scalar path selected.

Run in the development container only (needs /root/reference):
    make -C oracle && python tests/golden/make_scheduler_golden.py
The fixture holds data only: inputs, window widths, returned values and option vectors.
"""
import ctypes
import json
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
REF_DIR = os.path.join(HERE, "..", "..", "oracle", "_ref")


def _load(name):
    lib = ctypes.CDLL(os.path.join(REF_DIR, name))
    dp = ctypes.POINTER(ctypes.c_double)
    lib.solve_scheduler.argtypes = [ctypes.c_int] * 3 + [dp, dp, dp, ctypes.c_double, ctypes.c_int, ctypes.c_int,
                                                         ctypes.POINTER(ctypes.c_int)]
    lib.solve_scheduler.restype = ctypes.c_double
    lib.compute_buf_size.argtypes = [ctypes.c_int] * 3 + [dp, dp, ctypes.c_double, ctypes.c_int]
    lib.compute_buf_size.restype = ctypes.c_int
    return lib


def _ptr(a):
    return a.ctypes.data_as(ctypes.POINTER(ctypes.c_double))


def run(lib, compute, durations, sizes, deadline, time_scale, N, buf_size=None):
    compute = np.ascontiguousarray(compute, dtype=np.float64)
    durations = np.ascontiguousarray(durations, dtype=np.float64)
    sizes = np.ascontiguousarray(sizes, dtype=np.float64)
    T, k = durations.shape
    auto = lib.compute_buf_size(T, N, k, _ptr(compute), _ptr(durations), deadline, time_scale)
    if buf_size is None:
        buf_size = auto
    choices = np.full(T, -1, dtype=np.int32)
    val = lib.solve_scheduler(T, N, k, _ptr(compute), _ptr(durations), _ptr(sizes), deadline, time_scale, buf_size,
                              choices.ctypes.data_as(ctypes.POINTER(ctypes.c_int)))
    return auto, buf_size, val, choices.tolist()


def cases():
    out = []

    def add(name, compute, durations, sizes, N, deadline=None, time_scale=10, buf_size=None):
        compute, durations, sizes = (np.asarray(x, dtype=np.float64) for x in (compute, durations, sizes))
        if deadline is None:      # the wrapper's "safe" deadline
            deadline = float(np.sum(compute) + np.sum(np.max(durations, axis=1)) + 1000.0)
        out.append(dict(name=name, compute=compute.tolist(), durations=durations.tolist(), sizes=sizes.tolist(),
                        N=int(N), deadline=float(deadline), time_scale=int(time_scale), buf_size=buf_size))

    add("readme", [10.0] * 3, [[2.0, 5.0]] * 3, [[1.0, 3.0]] * 3, 2)
    T = 64
    add("tradeoff_64x4", np.ones(T) * 100.0, np.tile([200.0, 150.0, 100.0, 50.0], (T, 1)),
        np.tile([1000.0, 600.0, 300.0, 100.0], (T, 1)), 10)
    rng = np.random.default_rng(20240611)
    for idx in range(40):
        T = int(rng.integers(1, 48))
        k = int(rng.integers(1, 5))
        N = int(rng.integers(1, 12))
        compute = np.round(rng.uniform(2.0, 14.0, size=T), 3)
        durations = np.round(rng.uniform(0.01, 24.0, size=(T, k)), 3)
        sizes = np.round(durations * rng.uniform(0.5, 10.0, size=(T, k)), 3)
        if idx % 4 == 0:          # coarse values: many equal totals, exercises the tie-breaks
            sizes = rng.integers(1, 4, size=(T, k)).astype(np.float64)
            durations = rng.integers(1, 6, size=(T, k)).astype(np.float64) * 2.5
        if idx % 5 == 0:          # a hard global deadline
            add(f"rand{idx}_deadline", compute, durations, sizes, N, deadline=float(np.sum(compute)) * 0.9 + 5.0)
        else:
            add(f"rand{idx}", compute, durations, sizes, N)
    for idx, (T, k, N) in enumerate([(256, 4, 12), (256, 3, 4), (128, 4, 3)]):
        compute = np.round(rng.uniform(8.0, 12.0, size=T), 3)
        durations = np.round(rng.uniform(5.0, 15.0, size=(T, k)), 3)
        add(f"harness_like_{T}x{k}_N{N}", compute, durations, np.round(durations * 10.0, 2), N)
    # a window narrower than compute_buf_size asks for: states beyond it are dropped
    compute = np.round(rng.uniform(8.0, 12.0, size=96), 3)
    durations = np.round(rng.uniform(5.0, 15.0, size=(96, 3)), 3)
    add("narrow_window", compute, durations, np.round(durations * 7.0, 2), 6, buf_size=512)
    add("time_scale_3", compute[:20], durations[:20], np.round(durations[:20] * 7.0, 2), 4, time_scale=3)
    return out


def main():
    avx, scalar = _load("libts_ref.so"), _load("libts_ref_scalar.so")
    result = []
    for c in cases():
        a = run(avx, c["compute"], c["durations"], c["sizes"], c["deadline"], c["time_scale"], c["N"], c["buf_size"])
        s = run(scalar, c["compute"], c["durations"], c["sizes"], c["deadline"], c["time_scale"], c["N"], c["buf_size"])
        c = dict(c)
        c.update(auto_buf_size=a[0], buf_size=a[1], value=a[2], choices=a[3], value_scalar=s[2], choices_scalar=s[3])
        assert a[0] == s[0]
        result.append(c)
    path = os.path.join(HERE, "scheduler_cases.json")
    with open(path, "w") as f:
        json.dump(result, f)
    feasible = sum(1 for c in result if c["value"] != 0.0)
    agree = sum(1 for c in result if c["value"] == c["value_scalar"] and c["choices"] == c["choices_scalar"])
    print(f"{len(result)} cases ({feasible} feasible, {agree} with identical AVX2/scalar answers) -> {path}")


if __name__ == "__main__":
    main()
