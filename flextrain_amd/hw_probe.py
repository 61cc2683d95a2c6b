"""Hardware probe for the save-level solver's inputs, calibrated for MI355X.

Mirror of flextrain/core/hw_probe.py:42-328 (``HardwareProbeResult``, ``probe_hardware``): the
solver needs the SUSTAINED GEMM rate, the concurrent host-link bandwidth per direction and the HBM
bandwidth.  What differs on this part, and why:

* The GEMM is this library's MFMA dispatcher (the kernels the layers really run), 8192^3 by
  default: a 4096^3 problem is 256 tiles, one per CU, and measures launch ramp rather than the
  steady state.  Operands are random: on MI355X the sustained clock, and with it the GEMM rate,
  depends on the data (constant operands run 30-40 % faster than random ones), so a probe on
  zeros would overstate what training sustains.
* The wall-clock-bounded two-half measurement is kept: the second half is the figure used, the
  first shows the drop from boost clocks.
* Host memory for the link test comes from the exact-size pinned allocator of this package.
"""
from __future__ import annotations

import time
from dataclasses import dataclass

import torch

from .save_level import HardwareCost


@dataclass(frozen=True)
class HardwareProbeResult:
    hw_cost: HardwareCost
    matmul_n: int
    matmul_per_call_ms: float
    matmul_total_seconds: float
    achieved_tflops_first_half: float
    achieved_tflops_second_half: float
    transfer_bytes: int
    transfer_per_call_ms: float
    mem_bw_gbps: float
    mem_bw_total_seconds: float


def _run_halves(launch, device, target_seconds: float, min_reps_per_half: int, burst: int):
    """Launch in bursts until each half's wall budget is spent; returns [(reps, seconds)] x 2."""
    out = []
    for _ in range(2):
        reps = 0
        torch.cuda.synchronize(device)
        t0 = time.perf_counter()
        while True:
            for _ in range(burst):
                launch()
            reps += burst
            torch.cuda.synchronize(device)
            dt = time.perf_counter() - t0
            if dt >= target_seconds / 2 and reps >= min_reps_per_half:
                break
        out.append((reps, dt))
    return out


def _bench_matmul_sustained(n, *, dtype, device, target_seconds, n_warmup, min_reps_per_half):
    from . import ops

    a = torch.randn(n, n, device=device).to(dtype)
    b = torch.randn(n, n, device=device).to(dtype)
    d = torch.empty(n, n, dtype=dtype, device=device)
    stream = torch.cuda.current_stream(device).cuda_stream
    disp = ops.dispatcher
    launch = lambda: disp.matmul_fast(stream, a, b, None, d)
    for _ in range(n_warmup):
        launch()
    (r1, t1), (r2, t2) = _run_halves(launch, device, target_seconds, min_reps_per_half, burst=10)
    flops = 2.0 * n * n * n
    return t2 / r2, flops * (r1 + r2) / (t1 + t2) / 1e12, flops * r1 / t1 / 1e12, flops * r2 / t2 / 1e12, t1 + t2


def _bench_mem_bandwidth_sustained(n, *, dtype, device, target_seconds, n_warmup, min_reps_per_half):
    """HBM read + write rate of a streaming pass over an n x n tensor (the gated-activation kernel
    of this library: two reads and one write per element)."""
    from . import ops

    x1 = torch.randn(n, n, device=device).to(dtype)
    x3 = torch.randn(n, n, device=device).to(dtype)
    out = torch.empty_like(x1)
    launch = lambda: ops.flextrain_swiglu_fwd(x1, x3, out=out)
    for _ in range(n_warmup):
        launch()
    (r1, t1), (r2, t2) = _run_halves(launch, device, target_seconds, min_reps_per_half, burst=10)
    nbytes = 3.0 * n * n * x1.element_size()
    return nbytes * r2 / t2 / 1e9, t1 + t2


def _bench_pcie_concurrent(nbytes, *, device, n_warmup, n_reps):
    """Both directions at once on two streams; returns (seconds per iteration, GB/s per direction)."""
    from .host_memory import LocalPinnedHostBackend

    be = LocalPinnedHostBackend()
    h_in = be.allocate_tensor((nbytes,), torch.uint8)
    h_out = be.allocate_tensor((nbytes,), torch.uint8)
    d_in = torch.empty(nbytes, dtype=torch.uint8, device=device)
    d_out = torch.empty(nbytes, dtype=torch.uint8, device=device)
    s_in, s_out = torch.cuda.Stream(device=device), torch.cuda.Stream(device=device)

    def once():
        with torch.cuda.stream(s_in):
            d_in.copy_(h_in, non_blocking=True)
        with torch.cuda.stream(s_out):
            h_out.copy_(d_out, non_blocking=True)
        torch.cuda.synchronize(device)

    for _ in range(n_warmup):
        once()
    t0 = time.perf_counter()
    for _ in range(n_reps):
        once()
    per_iter = (time.perf_counter() - t0) / n_reps
    be.release(h_in)
    be.release(h_out)
    return per_iter, nbytes / per_iter / 1e9


def probe_hardware(*, device="cuda:0", dtype=torch.bfloat16, matmul_n: int = 8192, mem_bw_n: int = 8192,
                   transfer_mib: int = 256, matmul_target_seconds: float = 7.0, mem_bw_target_seconds: float = 3.0,
                   n_matmul_warmup: int = 5, n_mem_bw_warmup: int = 5, min_matmul_reps_per_half: int = 50,
                   min_mem_bw_reps_per_half: int = 50, n_transfer_warmup: int = 2,
                   n_transfer_reps: int = 5) -> HardwareProbeResult:
    """Sustained GEMM TFLOP/s (second half of the window), HBM GB/s and concurrent host-link GB/s;
    ``hw_cost`` carries the two figures the save-level solver uses."""
    device = torch.device(device)
    per_call, _overall, tf1, tf2, mm_total = _bench_matmul_sustained(
        matmul_n, dtype=dtype, device=device, target_seconds=matmul_target_seconds, n_warmup=n_matmul_warmup,
        min_reps_per_half=min_matmul_reps_per_half)
    mem_gbps, mem_total = _bench_mem_bandwidth_sustained(
        mem_bw_n, dtype=dtype, device=device, target_seconds=mem_bw_target_seconds, n_warmup=n_mem_bw_warmup,
        min_reps_per_half=min_mem_bw_reps_per_half)
    nbytes = transfer_mib * (1 << 20)
    per_xfer, gbps = _bench_pcie_concurrent(nbytes, device=device, n_warmup=n_transfer_warmup, n_reps=n_transfer_reps)
    return HardwareProbeResult(hw_cost=HardwareCost(peak_tflops=tf2, pcie_bw_gbps=gbps), matmul_n=matmul_n,
                               matmul_per_call_ms=per_call * 1e3, matmul_total_seconds=mm_total,
                               achieved_tflops_first_half=tf1, achieved_tflops_second_half=tf2,
                               transfer_bytes=nbytes, transfer_per_call_ms=per_xfer * 1e3, mem_bw_gbps=mem_gbps,
                               mem_bw_total_seconds=mem_total)
