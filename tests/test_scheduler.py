"""Save-level transmission scheduler: the product solver (``solve_scheduler`` /
``compute_buf_size`` of libflexhip.so, ``TransmissionScheduler.solve``) and the NumPy
oracle against (1) golden vectors written by the compiled reference
(tests/golden/scheduler_cases.json), (2) the README known answer, (3) exhaustive
enumeration on small problems, (4) the compiled reference itself when oracle/_ref is
present.  CPU only; integer option vectors must match exactly, values bit for bit."""
import ctypes
import json
import os

import numpy as np
import pytest

from flextrain_amd._lib import lib
from flextrain_amd.transmission_scheduler import TransmissionScheduler
from oracle import dp_solver as o_dp

HERE = os.path.dirname(os.path.abspath(__file__))
CASES = json.load(open(os.path.join(HERE, "golden", "scheduler_cases.json")))


def _product(c, buf_size=None):
    compute = np.ascontiguousarray(c["compute"], dtype=np.float64)
    durations = np.ascontiguousarray(c["durations"], dtype=np.float64)
    sizes = np.ascontiguousarray(c["sizes"], dtype=np.float64)
    T, k = durations.shape
    L = lib()
    auto = L.compute_buf_size(T, c["N"], k, compute.ctypes.data, durations.ctypes.data, c["deadline"], c["time_scale"])
    choices = np.full(T, -1, dtype=np.int32)
    val = L.solve_scheduler(T, c["N"], k, compute.ctypes.data, durations.ctypes.data, sizes.ctypes.data, c["deadline"],
                            c["time_scale"], c["buf_size"] if buf_size is None else buf_size, choices.ctypes.data)
    return auto, val, choices.tolist()


@pytest.mark.parametrize("c", CASES, ids=[c["name"] for c in CASES])
def test_product_matches_reference_golden(c):
    auto, val, choices = _product(c)
    assert auto == c["auto_buf_size"]
    assert val == c["value"] == c["value_scalar"]
    if val != 0.0:
        assert choices == c["choices"] == c["choices_scalar"]
    else:
        assert choices == [-1] * len(choices)       # untouched on failure


@pytest.mark.parametrize("c", CASES, ids=[c["name"] for c in CASES])
def test_oracle_matches_reference_golden(c):
    val, choices = o_dp.solve_scheduler(c["compute"], c["durations"], c["sizes"], c["deadline"], c["time_scale"], c["N"],
                                        buf_size=c["buf_size"])
    assert o_dp.compute_buf_size(c["compute"], c["durations"], c["deadline"], c["time_scale"], c["N"]) == c["auto_buf_size"]
    assert val == c["value"]
    if val != 0.0:
        assert choices.tolist() == c["choices"]


def test_readme_known_answer():
    # orig/transmission_scheduler_pkg/README.md:47-59
    ts = TransmissionScheduler()
    args = (np.array([10.0, 10.0, 10.0]), np.array([[2.0, 5.0]] * 3), np.array([[1.0, 3.0]] * 3))
    val, choices = ts.solve(*args, N=2)
    assert val == 9.0 and choices.tolist() == [1, 1, 1] and choices.dtype == np.int32
    oval, ochoices = o_dp.wrapper_solve(*args, N=2)
    assert oval == 9.0 and ochoices.tolist() == [1, 1, 1]


def test_exhaustive_small_problems():
    rng = np.random.default_rng(7)
    ts = TransmissionScheduler()
    feasible = 0
    for trial in range(120):
        T, k, N = int(rng.integers(1, 8)), int(rng.integers(1, 4)), int(rng.integers(1, 5))
        compute = np.round(rng.uniform(1.0, 6.0, size=T), 1)
        durations = np.round(rng.uniform(0.05, 9.0, size=(T, k)), 1)
        sizes = rng.integers(1, 6, size=(T, k)).astype(np.float64)
        deadline = float(compute.sum() + (durations.max() if trial % 3 else 0.5))
        best = o_dp.brute_force(compute, durations, sizes, deadline, 10, N)
        oval, ochoices = o_dp.solve_scheduler(compute, durations, sizes, deadline, 10, N)
        c = dict(compute=compute, durations=durations, sizes=sizes, deadline=deadline, time_scale=10, N=N, buf_size=2048)
        _, pval, pchoices = _product(c)
        if best is None:
            assert oval == 0.0 and ochoices is None and pval == 0.0
            continue
        feasible += 1
        assert oval == best == pval
        assert pchoices == ochoices.tolist()
        assert o_dp.simulate(pchoices, compute, durations, sizes, deadline, 10, N) == best
    assert feasible > 30


def test_wrapper_on_reference_demo_keeps_its_window_drops():
    # helpers/transmission_scheduler/simp_test.py: the reference's window (32768 ticks here) drops
    # states, so its answer (35200, golden) is below the unwindowed optimum (35700)
    T = 64
    args = (np.ones(T) * 100.0, np.tile([200.0, 150.0, 100.0, 50.0], (T, 1)), np.tile([1000.0, 600.0, 300.0, 100.0], (T, 1)))
    val, choices = TransmissionScheduler().solve(*args, N=10)
    c = next(c for c in CASES if c["name"] == "tradeoff_64x4")
    assert val == c["value"] == 35200.0 and choices.tolist() == c["choices"]
    deadline = float(args[0].sum() + args[1].max(axis=1).sum() + 1000.0)
    assert o_dp.solve_scheduler(*args, deadline, 10, 10)[0] == 35700.0


def test_wrapper_negative_sizes_and_infeasible():
    ts = TransmissionScheduler()
    rng = np.random.default_rng(3)
    compute = rng.uniform(8.0, 12.0, size=20)
    durations = rng.uniform(2.0, 9.0, size=(20, 3))
    sizes = -durations                                  # minimise total duration
    val, choices = ts.solve(compute, durations, sizes, N=3)
    oval, ochoices = o_dp.wrapper_solve(compute, durations, sizes, 3)
    assert val == oval and choices.tolist() == ochoices.tolist()
    np.testing.assert_allclose(val, sizes[np.arange(20), choices].sum(), rtol=1e-12)
    # N = 1: a task would have to finish before it arrives
    assert ts.solve(compute, durations, sizes, N=1) == (None, None)
    assert o_dp.wrapper_solve(compute, durations, sizes, 1) == (None, None)


def test_window_narrower_than_band_drops_states():
    c = next(c for c in CASES if c["name"] == "narrow_window")
    assert c["buf_size"] < c["auto_buf_size"]
    _, val, choices = _product(c)
    assert val == c["value"] and (val == 0.0 or choices == c["choices"])


REF = os.path.join(HERE, "..", "oracle", "_ref", "libts_ref.so")


@pytest.mark.skipif(not os.path.exists(REF), reason="compiled reference solver (oracle/_ref) not built")
def test_random_problems_against_compiled_reference():
    ref = ctypes.CDLL(REF)
    dp = ctypes.POINTER(ctypes.c_double)
    ref.solve_scheduler.argtypes = [ctypes.c_int] * 3 + [dp, dp, dp, ctypes.c_double, ctypes.c_int, ctypes.c_int,
                                                         ctypes.POINTER(ctypes.c_int)]
    ref.solve_scheduler.restype = ctypes.c_double
    rng = np.random.default_rng(99)
    checked = 0
    for trial in range(200):
        T, k, N = int(rng.integers(1, 200)), int(rng.integers(1, 5)), int(rng.integers(2, 14))
        compute = rng.uniform(4.0, 12.0, size=T)
        durations = rng.uniform(0.5, 18.0, size=(T, k))
        sizes = np.round(durations * rng.uniform(1.0, 5.0, size=(T, k)), 2)
        deadline = float(compute.sum() + durations.max(axis=1).sum() + 1000.0)
        c = dict(compute=compute, durations=durations, sizes=sizes, deadline=deadline, time_scale=10, N=N, buf_size=None)
        c["buf_size"] = lib().compute_buf_size(T, N, k, compute.ctypes.data, durations.ctypes.data, deadline, 10)
        _, val, choices = _product(c)
        rchoices = np.full(T, -1, dtype=np.int32)
        rval = ref.solve_scheduler(T, N, k, compute.ctypes.data_as(dp), durations.ctypes.data_as(dp),
                                   sizes.ctypes.data_as(dp), deadline, 10, c["buf_size"],
                                   rchoices.ctypes.data_as(ctypes.POINTER(ctypes.c_int)))
        assert val == rval, trial
        if rval != 0.0:
            assert choices == rchoices.tolist(), trial
            checked += 1
    assert checked > 50


@pytest.mark.parametrize("flags", [["-DFX_VECTOR_BUILDS="], ["-DFX_VECTOR_BUILDS=", "-mavx2"]], ids=["baseline", "avx2"])
def test_every_vector_build_of_the_inner_loops_gives_the_same_answer(flags, tmp_path):
    """The library picks a build of the two inner loops by the CPU it runs on; the other builds, compiled
    here as the only one, must return the same values and option vectors (ties included: integer sizes)."""
    import shutil
    import subprocess

    cxx = shutil.which("g++")
    if cxx is None:
        pytest.skip("no g++")
    if "-mavx2" in flags and "avx2" not in open("/proc/cpuinfo").read():
        pytest.skip("no AVX2 on this host")
    root = os.path.join(HERE, "..")
    so = str(tmp_path / "libsched_variant.so")
    subprocess.run([cxx, "-O3", "-std=c++17", "-fPIC", "-shared", "-D__HIP_PLATFORM_AMD__", "-I/opt/rocm/include",
                    "-I" + os.path.join(root, "include"), *flags,
                    os.path.join(root, "flextrain_amd", "csrc", "scheduler.cpp"), "-o", so], check=True)
    alt = ctypes.CDLL(so)
    alt.solve_scheduler.argtypes = [ctypes.c_int] * 3 + [ctypes.c_void_p] * 3 + [ctypes.c_double, ctypes.c_int, ctypes.c_int,
                                                                                 ctypes.c_void_p]
    alt.solve_scheduler.restype = ctypes.c_double
    rng = np.random.default_rng(41)
    feasible = 0
    for trial in range(150):
        T, k, N = int(rng.integers(1, 300)), int(rng.integers(1, 6)), int(rng.integers(2, 14))
        compute = rng.uniform(4.0, 12.0, size=T)
        durations = rng.uniform(0.5, 18.0, size=(T, k))
        sizes = rng.integers(1, 5, size=(T, k)).astype(np.float64) if trial % 2 else np.round(durations * 3.0, 2)
        deadline = float(compute.sum() + durations.max(axis=1).sum() + 1000.0)
        scale = 10 if trial % 5 else 100
        c = dict(compute=compute, durations=durations, sizes=sizes, deadline=deadline, time_scale=scale, N=N, buf_size=None)
        c["buf_size"] = lib().compute_buf_size(T, N, k, compute.ctypes.data, durations.ctypes.data, deadline, scale)
        if trial % 7 == 0:
            c["buf_size"] = 256                 # a window narrower than the band: states are dropped
        _, val, choices = _product(c)
        achoices = np.full(T, -1, dtype=np.int32)
        aval = alt.solve_scheduler(T, N, k, compute.ctypes.data, durations.ctypes.data, sizes.ctypes.data, deadline, scale,
                                   c["buf_size"], achoices.ctypes.data)
        assert val == aval, trial
        if val != 0.0:
            feasible += 1
            assert choices == achoices.tolist(), trial
    assert feasible > 50


def test_a_huge_window_costs_nothing():
    """The window width only bounds which states are kept: memory follows the band that the tasks can
    reach, so the largest window a caller can name gives the unwindowed answer at once."""
    c = dict(next(c for c in CASES if c["name"] == "tradeoff_64x4"))
    _, val, choices = _product(c, buf_size=(1 << 31) - 1)
    oval, ochoices = o_dp.solve_scheduler(c["compute"], c["durations"], c["sizes"], c["deadline"], c["time_scale"], c["N"])
    assert val == oval == 35700.0 and choices == ochoices.tolist()


@pytest.mark.skipif(not os.path.exists(REF), reason="compiled reference solver (oracle/_ref) not built")
def test_edge_problems_against_compiled_reference():
    """Windows of 1 to 4096 ticks (most far narrower than the band), 1 / 10 / 100 ticks per ms, zero compute
    times and durations, deadlines that cut the schedule short, integer values (ties): value and option
    vector as the compiled reference gives them, and untouched choices where it finds no schedule."""
    ref = ctypes.CDLL(REF)
    ref.solve_scheduler.argtypes = [ctypes.c_int] * 3 + [ctypes.c_void_p] * 3 + [ctypes.c_double, ctypes.c_int, ctypes.c_int,
                                                                                 ctypes.c_void_p]
    ref.solve_scheduler.restype = ctypes.c_double
    rng = np.random.default_rng(5)
    feasible = 0
    for trial in range(1500):
        T, k, N = int(rng.integers(1, 40)), int(rng.integers(1, 5)), int(rng.integers(1, 12))
        scale = int(rng.choice([1, 10, 100]))
        compute = rng.uniform(0.0, 12.0, T)
        durations = rng.uniform(0.0, 30.0, (T, k))
        sizes = rng.integers(1, 6, (T, k)).astype(np.float64) if trial % 2 else rng.uniform(0.5, 50, (T, k))
        deadline = float(compute.sum() + (durations.max(axis=1).sum() + 1000.0 if trial % 3 else rng.uniform(0, 20)))
        buf = int(rng.choice([1, 2, 3, 7, 64, 300, 2048, 4096]))
        c = dict(compute=compute, durations=durations, sizes=sizes, deadline=deadline, time_scale=scale, N=N, buf_size=buf)
        _, val, choices = _product(c)
        rchoices = np.full(T, -1, dtype=np.int32)
        rval = ref.solve_scheduler(T, N, k, compute.ctypes.data, durations.ctypes.data, sizes.ctypes.data, deadline, scale, buf,
                                   rchoices.ctypes.data)
        assert val == rval, trial
        assert choices == rchoices.tolist(), trial
        feasible += val != 0.0
    assert feasible > 50
