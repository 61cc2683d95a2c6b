"""Host-side pieces of bench.py that need no GPU: the traffic figure is recomputed from the committed
counter summary, a leg that raises is reported instead of ending the run, more than one GPU is refused."""
from __future__ import annotations

import os
import subprocess
import sys

import bench

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_traffic_comes_from_the_committed_counter_summary(tmp_path):
    got = bench._measured_traffic_bytes()
    algorithmic = 5 * 8192 * 14336 * 2
    assert got is not None and abs(got - algorithmic) / algorithmic < 1e-3      # nothing is re-read
    assert bench._measured_traffic_bytes(str(tmp_path / "absent.txt")) is None
    broken = tmp_path / "broken.txt"
    broken.write_text("copy_bytes_each_way: 536870912\ncopy_FETCH_SIZE_KiB: 0\n")
    assert bench._measured_traffic_bytes(str(broken)) is None
    # FETCH_SIZE counts half of what is fetched on this hardware: the calibration pass supplies the factor
    text = ("copy_bytes_each_way: 1048576\ncopy_FETCH_SIZE_KiB: 512.0\ncopy_WRITE_SIZE_KiB: 1024.0\n"
            "glu_bwd_FETCH_SIZE_KiB: 3.0\nglu_bwd_WRITE_SIZE_KiB: 2.0\n")
    ok = tmp_path / "ok.txt"
    ok.write_text(text)
    assert bench._measured_traffic_bytes(str(ok)) == (3 * 2 + 2) * 1024


def test_a_failing_leg_is_reported_and_ends_the_gpu_legs(monkeypatch):
    class _Cuda:
        @staticmethod
        def synchronize():
            pass

    class _Torch:
        cuda = _Cuda

    calls = []
    monkeypatch.setattr(bench, "run_rmsnorm", lambda *a: calls.append("c1") or [{"op": "c1.row", "unit": "GB/s"}])

    def boom(*a):
        calls.append("c4")
        raise RuntimeError("launch failed")

    monkeypatch.setattr(bench, "run_adamw", boom)
    monkeypatch.setattr(bench, "run_lm_head", lambda *a: calls.append("c3") or [])
    rows = bench.run_extra(_Torch, None, None, None, None, [])
    assert calls == ["c1", "c4"]                                     # nothing after the failure touches the GPU
    assert rows[0]["op"] == "c1.row" and rows[-1]["op"] == "c4.FAILED" and "launch failed" in rows[-1]["error"]
    calls.clear()
    rows = bench.run_extra(_Torch, None, None, None, None, ["c3"])   # --only selects legs
    assert calls == ["c3"] and rows == []


def test_more_than_one_gpu_is_refused():
    proc = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert proc.returncode == 2 and "one GPU only" in proc.stderr and proc.stdout == ""


def test_the_headline_path_runs_through_to_the_json_line():
    """bench.py itself, unchanged and at its real shapes, on a library whose launches return at once
    (tests/hostsim/bench_dry_run.py): the headline workload, one leg and the assembly of the final line
    raise no Python error.  The whole script takes five minutes that way and is run by hand."""
    from tests.hostsim.build import CLANG

    if not os.path.exists(CLANG):
        import pytest

        pytest.skip("the host simulation is compiled with " + CLANG)
    proc = subprocess.run([sys.executable, "-m", "tests.hostsim.bench_dry_run", "--only", "disp"], cwd=ROOT, capture_output=True,
                          text=True, timeout=900)
    assert proc.returncode == 0 and "failed legs: none" in proc.stdout, (proc.stdout[-500:], proc.stderr[-2000:])
