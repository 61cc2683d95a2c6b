#!/usr/bin/env python3
"""Throughput of the per-layer training compute path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-extra] [--no-cpu]

A "step" is one pass of the Llama-3.1-8B-shaped RoPE + SwiGLU forward+backward
workload (q [8192,32,128], k [8192,8,128], gate/up/dout [8192,14336], bf16,
synthetic N(0,1)) with every input already resident in HBM.  ``value`` is the
algorithmic HBM bytes of a step divided by its wall time on the GPU stream.
The dominant kernel (SwiGLU backward) is bracketed by HIP events on the launch
stream inside the timed region, which gives the average duration behind
``roofline``; the rows of the other kernels come from back-to-back launches
after the timed region (event records around every short launch would leave
the GPU idle for a visible share of the step).

After the timed region the other single-GPU configurations (RMSNorm, AdamW, ...)
are measured the same way and reported under ``ops``; they do not enter
``value``.  The CPU baseline times the CPU oracle of the same workload on a
bounded token sample on the host cores.

Prints exactly one JSON line on stdout.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0       # MI355X HBM3E, published
BF16_PEAK_TFLOPS = 2500.0    # MI355X dense bf16 MFMA, published

# HBM bytes per launch of the SwiGLU backward kernel at the benchmark shape come from the FETCH_SIZE
# and WRITE_SIZE hardware counters, each scaled by what it reads for a plain copy of known size.  The
# counter values live in this text summary (with the commands that produced them); the figure is
# recomputed from it on every run, and is null when the file is missing or does not parse.
TRAFFIC_PROFILE = os.path.join(ROOT, "profiles", "glu_bwd_hbm_traffic_pmc.txt")


def _measured_traffic_bytes(path=TRAFFIC_PROFILE):
    """`key: value` lines of the summary: KiB per dispatch of the calibration copy and of the kernel."""
    want = ("copy_bytes_each_way", "copy_FETCH_SIZE_KiB", "copy_WRITE_SIZE_KiB", "glu_bwd_FETCH_SIZE_KiB",
            "glu_bwd_WRITE_SIZE_KiB")
    vals = {}
    try:
        with open(path) as f:
            for line in f:
                key, _, rest = line.partition(":")
                if key.strip() in want:
                    vals[key.strip()] = float(rest.split()[0].replace(",", ""))
    except (OSError, ValueError, IndexError):
        return None
    if any(k not in vals for k in want) or vals["copy_FETCH_SIZE_KiB"] <= 0 or vals["copy_WRITE_SIZE_KiB"] <= 0:
        return None
    copy_kib = vals["copy_bytes_each_way"] / 1024.0
    read = vals["glu_bwd_FETCH_SIZE_KiB"] * (copy_kib / vals["copy_FETCH_SIZE_KiB"])
    written = vals["glu_bwd_WRITE_SIZE_KiB"] * (copy_kib / vals["copy_WRITE_SIZE_KiB"])
    return int(round((read + written) * 1024.0))

METRIC = "per-op HBM GB/s (% of 8 TB/s) + lm_head/MoE GEMM TFLOPS (% bf16 MFMA peak)"


def _parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--no-extra", action="store_true", help="skip the non-headline configurations")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    ap.add_argument("--only", default="", help="comma-separated subset of the non-headline configurations "
                                               "(c1, c3, c4, c5, moe_ref, ffn, attn, act, disp, probe, a15) to run, e.g. for a profiler pass")
    return ap.parse_args()


class Timed:
    """Accumulates HIP-event durations per named kernel on one stream."""

    def __init__(self, torch, stream):
        self.torch, self.stream = torch, stream
        self.pairs = {}

    def __call__(self, name, fn):
        a = self.torch.cuda.Event(enable_timing=True)
        b = self.torch.cuda.Event(enable_timing=True)
        a.record(self.stream)
        fn()
        b.record(self.stream)
        self.pairs.setdefault(name, []).append((a, b))

    def mean_ms(self, name):
        ev = self.pairs[name]
        return sum(a.elapsed_time(b) for a, b in ev) / len(ev)

    def clear(self):
        self.pairs = {}


def _op_entry(name, work, unit, ms):
    """work: algorithmic bytes (unit GB/s) or FLOPs (unit TFLOP/s) per launch."""
    if unit == "GB/s":
        ach, peak = work / (ms * 1e-3) / 1e9, HBM_PEAK_GBPS
    else:
        ach, peak = work / (ms * 1e-3) / 1e12, BF16_PEAK_TFLOPS
    return {"op": name, "algorithmic": work, "ms": round(ms, 5), "achieved": round(ach, 2),
            "unit": unit, "frac": round(ach / peak, 4)}


def _time_launches(torch, stream, fns, warmup=5, reps=20, settle_ms=40.0, window_ms=20.0):
    """Mean milliseconds per launch; ``fns`` is a list of equivalent closures over
    distinct buffer sets, called round-robin so small working sets cannot sit in
    the 256 MB last-level cache between launches.

    Coming from idle, the GPU runs MFMA-heavy kernels at boost clocks for the first few
    milliseconds, then drops below its sustained clocks and recovers over roughly 25 ms (one
    8192 x 4096 x 4096 GEMM: 222 us, then up to 281 us, then 214 us from the hundredth call on).
    The timed window therefore starts after at least ``settle_ms`` of the same work and covers at
    least ``window_ms``: the figure is the sustained one."""
    n = len(fns)
    with torch.cuda.stream(stream):
        a = torch.cuda.Event(enable_timing=True)
        b = torch.cuda.Event(enable_timing=True)
        a.record(stream)
        for i in range(max(warmup, 1)):
            fns[i % n]()
        b.record(stream)
        torch.cuda.synchronize()
        est = max(a.elapsed_time(b) / max(warmup, 1), 1e-3)
        done = max(warmup, 1)
        extra = min(2000, int(max(0.0, settle_ms - est * done) / est))
        for i in range(extra):
            fns[(done + i) % n]()
        done += extra
        reps = max(reps, min(2000, int(window_ms / est) + 1))
        a.record(stream)
        for i in range(reps):
            fns[(done + i) % n]()
        b.record(stream)
        torch.cuda.synchronize()
    return a.elapsed_time(b) / reps


def _progress(text):
    """One line on stderr per leg, flushed before the leg touches the GPU: what a run that dies leaves behind."""
    print(f"[bench {time.strftime('%H:%M:%S')}] {text}", file=sys.stderr, flush=True)


def run_extra(torch, ops, dev, stream, rn, only):
    """The legs beside the headline workload.  A leg that raises is recorded as a row with its error
    and ends the GPU legs (a failed launch leaves the context unusable); the rows measured so far and
    the headline figure are still reported."""
    want = lambda tag: not only or tag in only
    legs = (("c1", lambda: run_rmsnorm(torch, ops, dev, stream, rn)),
            ("c4", lambda: run_adamw(torch, ops, dev, stream) + run_streamed_adamw(torch, dev)),
            ("c3", lambda: run_lm_head(torch, dev, stream, rn)),
            ("c5", lambda: run_moe(torch, dev, stream, rn)),
            ("moe_ref", lambda: _moe_reference_microbench(torch, dev, stream, rn)),
            ("ffn", lambda: run_ffn_dense(torch, dev, stream, rn)),
            ("attn", lambda: run_attention_proj(torch, dev, stream, rn)),
            ("act", lambda: run_activation_slots(torch, dev)),
            ("disp", lambda: run_dispatch_overhead(torch, dev, stream)),
            ("probe", lambda: run_hw_probe(torch, dev)))
    rows = []
    for tag, leg in legs:
        if not want(tag):
            continue
        _progress(f"leg {tag}")
        try:
            rows += leg()
            torch.cuda.synchronize()
        except Exception as exc:  # noqa: BLE001 - reported in the output line, not swallowed
            _progress(f"leg {tag} FAILED: {type(exc).__name__}: {exc}")
            rows.append({"op": f"{tag}.FAILED", "unit": "", "error": f"{type(exc).__name__}: {exc}"[:400]})
            break
    return rows


def run_dispatch_overhead(torch, dev, stream):
    """Host time per dispatcher call on a GEMM too small to matter (64^3): the validating ``matmul``
    (ctypes), the class's ``matmul_fast`` (tensor introspection + the C fast-call entry) and the raw
    24-argument C entry on pre-extracted values; the library's own time per call (cache look-up and
    kernel launch, from get_stats) is common to all three."""
    from flextrain_amd import matmul_dispatcher as md

    A = torch.ones(64, 64, dtype=torch.bfloat16, device=dev)
    D = torch.empty_like(A)
    disp = md.CublasLtDispatcher()
    sp = stream.cuda_stream
    disp.matmul(sp, A, A, D=D)
    torch.cuda.synchronize()
    n = 2000

    def per_call(fn):
        best = 1e9
        for _ in range(3):
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(n):
                fn()
            best = min(best, (time.perf_counter() - t0) / n)
            torch.cuda.synchronize()
        return best * 1e6

    raw = [disp._ctx_int, sp, 64, 64, 64, A.data_ptr(), 64, 0, A.data_ptr(), 64, 0, 0, 64, D.data_ptr(), 64,
           disp.ws_ptr, disp.workspace_size, 2, 2, 2, 2, 0, 1.0, 0.0]
    fast = md._bind_fast()
    us_raw = per_call(lambda: fast(*raw))
    # the library's own time per call (cache look-up + kernel launch, from its statistics) over the SAME calls as a
    # mean of the raw entry's host time: their difference is what the extension adds
    st0 = disp.get_stats()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(n):
        fast(*raw)
    us_raw_mean = (time.perf_counter() - t0) / n * 1e6
    torch.cuda.synchronize()
    st1 = disp.get_stats()
    cpp_us = ((st1["avg_cpp_total_us"] * st1["matmuls_called"] - st0["avg_cpp_total_us"] * st0["matmuls_called"])
              / max(1, st1["matmuls_called"] - st0["matmuls_called"]))
    # the library's own split of that time (get_stats: key construction, cache look-up, and the enqueue =
    # current-device query + kernel launch call), over a window of calls of its own
    import ctypes

    def raw_stats():
        buf = (ctypes.c_uint64 * 7)()
        disp._lib.get_stats(disp.ctx, buf)
        return list(buf)

    r0 = raw_stats()
    for _ in range(n):
        fast(*raw)
    torch.cuda.synchronize()
    r1 = raw_stats()
    calls = max(1, r1[1] - r0[1])
    total_us, key_us, lookup_us, enqueue_us = ((r1[i] - r0[i]) / calls / 1e3 for i in (3, 4, 5, 6))
    us_fast = per_call(lambda: disp.matmul_fast(sp, A, A, D=D))
    us_full = per_call(lambda: disp.matmul(sp, A, A, D=D))
    return [{"op": "disp.host time per dispatcher call (64^3 GEMM, 2000 calls back to back)", "algorithmic": None,
             "unit": "us", "frac": None, "ms": None, "achieved": None,
             "matmul_ctypes_us": round(us_full, 2), "matmul_fast_method_us": round(us_fast, 2),
             "raw_fast_call_entry_us": round(us_raw, 2), "library_time_per_call_us": round(cpp_us, 2),
             "raw_fast_call_entry_mean_us": round(us_raw_mean, 2),
             "library_split_us": {"key": round(key_us, 3), "cache_lookup": round(lookup_us, 3),
                                  "enqueue (device query + launch call)": round(enqueue_us, 3),
                                  "other (argument checks, clock reads, error query)": round(max(0.0, total_us - key_us - lookup_us - enqueue_us), 3)},
             "raw_entry_overhead_over_library_us": round(max(0.0, us_raw_mean - cpp_us), 2)}]


def run_rmsnorm(torch, ops, dev, stream, rn):
    rows = []
    # ---- configs[0]: RMSNorm fwd+bwd, x [2048,4096] bf16; 24 buffer sets = 1.6 GB
    T, D, NSETS = 2048, 4096, 24
    w = rn(D, std=0.02, mean=1.0).to(dev)
    sets = []
    for _ in range(NSETS):
        x = rn(T, D).to(dev)
        sets.append(dict(x=x, dy=torch.randn_like(x), y=torch.empty_like(x), dx=torch.empty_like(x),
                         rstd=torch.empty(T, 1, dtype=torch.float32, device=dev)))
    dw = torch.zeros(D, dtype=torch.float32, device=dev)
    fwd = [lambda s=s: ops.flextrain_rmsnorm_fwd(s["x"], w, output=s["y"], rstd=s["rstd"]) for s in sets]
    ms = _time_launches(torch, stream, fwd, warmup=NSETS, reps=4 * NSETS)
    rows.append(_op_entry("c1.rmsnorm_fwd", 2 * T * D * 2 + D * 2 + T * 4, "GB/s", ms))
    bwd = [lambda s=s: ops.flextrain_rmsnorm_bwd(s["dy"], s["x"], w, s["rstd"], dX=s["dx"], dW=dw) for s in sets]
    for s in sets:
        s["dx"].zero_()
    ms = _time_launches(torch, stream, bwd, warmup=NSETS, reps=4 * NSETS)
    # dX given => accumulate: reads dy, x, dx_old, writes dx (4 row tensors)
    rows.append(_op_entry("c1.rmsnorm_bwd(dX+=,dW+=)", 4 * T * D * 2 + D * 2 + T * 4 + 2 * D * 4, "GB/s", ms))
    bwd_e = [lambda s=s: ops.flextrain_rmsnorm_bwd(s["dy"], s["x"], w, s["rstd"], dX=s["dx"], dW=dw,
                                                   recompute_output=True, recomputed_output_tensor=s["y"])
             for s in sets]
    ms = _time_launches(torch, stream, bwd_e, warmup=NSETS, reps=4 * NSETS)
    rows.append(_op_entry("c1.rmsnorm_bwd(dX+=,dW+=,y)", 5 * T * D * 2 + D * 2 + T * 4 + 2 * D * 4, "GB/s", ms))
    # yardstick at this size (16.8 MB per tensor): an elementwise kernel with one read and one write stream, and
    # the same with three reads and one write (the traffic of the backward), through the same rotating sets
    with torch.cuda.stream(stream):
        ms = _time_launches(torch, stream, [lambda s=s: torch.mul(s["x"], 2.0, out=s["y"]) for s in sets], warmup=NSETS, reps=4 * NSETS)
        rows.append(_op_entry("c1.yardstick: y = 2x over one [2048,4096] tensor (torch elementwise kernel, comparison)",
                              2 * T * D * 2, "GB/s", ms))
        ms = _time_launches(torch, stream, [lambda s=s: torch.addcmul(s["dx"], s["x"], s["dy"], out=s["dx"]) for s in sets],
                            warmup=NSETS, reps=4 * NSETS)
        rows.append(_op_entry("c1.yardstick: dx += x * dy over [2048,4096] tensors (torch elementwise kernel, comparison)",
                              4 * T * D * 2, "GB/s", ms))
    del sets, fwd, bwd, bwd_e
    torch.cuda.empty_cache()
    # ---- the same kernels at the token count of the headline workload's layer input x 4 (32768 rows, 268 MB per
    # tensor): configs[0] is 16 MB per tensor and therefore bound by launch and latency, not by HBM
    T2 = 32768
    big = [dict(x=rn(T2, D).to(dev), dy=rn(T2, D).to(dev), y=torch.empty(T2, D, dtype=torch.bfloat16, device=dev),
                dx=torch.zeros(T2, D, dtype=torch.bfloat16, device=dev), rstd=torch.empty(T2, 1, dtype=torch.float32, device=dev))
           for _ in range(3)]
    fwd = [lambda s=s: ops.flextrain_rmsnorm_fwd(s["x"], w, output=s["y"], rstd=s["rstd"]) for s in big]
    ms = _time_launches(torch, stream, fwd, warmup=3, reps=12)
    rows.append(_op_entry("c1x16.rmsnorm_fwd at 32768 tokens", 2 * T2 * D * 2 + D * 2 + T2 * 4, "GB/s", ms))
    bwd = [lambda s=s: ops.flextrain_rmsnorm_bwd(s["dy"], s["x"], w, s["rstd"], dX=s["dx"], dW=dw) for s in big]
    ms = _time_launches(torch, stream, bwd, warmup=3, reps=12)
    rows.append(_op_entry("c1x16.rmsnorm_bwd(dX+=,dW+=) at 32768 tokens", 4 * T2 * D * 2 + D * 2 + T2 * 4 + 2 * D * 4, "GB/s", ms))
    del big, fwd, bwd
    torch.cuda.empty_cache()
    return rows


def run_adamw(torch, ops, dev, stream):
    """configs[3] kernel: AdamW on one 218,112,000-parameter chunk resident in HBM."""
    rows = []
    n = 218_112_000
    p = (torch.randn(n, device=dev) * 0.02)
    m = torch.zeros(n, device=dev)
    v = torch.zeros(n, device=dev)
    gr = (torch.randn(n, device=dev) * 1e-3).to(torch.bfloat16)
    pb = torch.empty(n, dtype=torch.bfloat16, device=dev)
    hp = dict(lr=3e-5, beta1=0.9, beta2=0.95, eps=1e-8, weight_decay=0.1)
    step = [0]

    def adam(copy):
        step[0] += 1
        ops.flextrain_adamw_step(p, gr, m, v, step=step[0], params_bf16_out=pb if copy else None, **hp)

    ms = _time_launches(torch, stream, [lambda: adam(True)], warmup=3, reps=10)
    rows.append(_op_entry("c4.adamw(fp32 p/m/v, bf16 g, bf16 copy-out)", 28 * n, "GB/s", ms))
    ms = _time_launches(torch, stream, [lambda: adam(False)], warmup=3, reps=10)
    rows.append(_op_entry("c4.adamw(fp32 p/m/v, bf16 g)", 26 * n, "GB/s", ms))
    del p, m, v, gr, pb
    torch.cuda.empty_cache()
    return rows


def run_mfma_probe(torch, dev, stream):
    """What the matrix pipes sustain on this machine with nothing else going on: bf16 MFMAs only,
    operands in registers.  Constant data reaches the published peak; random data makes the power
    management lower the clock, and that rate is the practical ceiling for a GEMM on real data."""
    import ctypes

    from flextrain_amd._lib import lib

    L = lib()
    ws = torch.empty(int(L.fx_probe_ws_bytes()), dtype=torch.uint8, device=dev)
    out = {}
    for name, rnd in (("constant_operands", 0), ("random_operands", 1)):
        flop = ctypes.c_double()
        iters = 120000      # ~30-40 ms: long enough for the clock to settle under load

        def launch():
            L.fx_probe_mfma_rate(rnd, iters, ws.data_ptr(), ws.numel(), ctypes.byref(flop), stream.cuda_stream)

        ms = _time_launches(torch, stream, [launch], warmup=1, reps=3)
        clocks = ws[:16].view(torch.int64).cpu()
        ghz = float(clocks[0]) / max(1.0, float(clocks[1])) * 0.1      # wall clock ticks at 100 MHz
        out[name] = {"tflops": round(flop.value / (ms * 1e-3) / 1e12, 1), "shader_clock_ghz": round(ghz, 3),
                     "ms": round(ms, 3)}
    return out


def run_streamed_adamw(torch, dev):
    """configs[3] as the engine runs it: the chunk's fp32 master weights, bf16 grads and
    fp32 moments live in pinned host memory and stream through device staging slots.
    The host link is the roof here, not HBM: reported as bytes moved per direction."""
    from flextrain_amd.host_memory import LocalPinnedHostBackend
    from flextrain_amd.optim import adamw_stream_workspace, flextrain_adamw_step_streamed
    from flextrain_amd.streams import StreamBundle

    n = 218_112_000
    be = LocalPinnedHostBackend()
    sb = StreamBundle.create(dev)
    host = dict(p=be.allocate_tensor((n,), torch.float32), g=be.allocate_tensor((n,), torch.bfloat16),
                m=be.allocate_tensor((n,), torch.float32), v=be.allocate_tensor((n,), torch.float32),
                pc=be.allocate_tensor((n,), torch.bfloat16))
    host["p"].normal_(0, 0.02)
    host["g"].normal_(0, 1e-3)
    sub, slots = 4 * 1024 * 1024, 3
    ws = adamw_stream_workspace(sub, slots, torch.float32, torch.bfloat16, torch.float32, True, dev)
    hp = dict(lr=3e-5, beta1=0.9, beta2=0.95, eps=1e-8, weight_decay=0.1)

    def run(step):
        flextrain_adamw_step_streamed(host["p"], host["g"], host["m"], host["v"], streams=sb, step=step,
                                      params_bf16_out=host["pc"], workspace=ws, sub_elems=sub, n_slots=slots, **hp)

    run(1)
    sb.synchronize_all()
    times = []
    for step in range(2, 5):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        run(step)
        sb.synchronize_all()
        times.append(time.perf_counter() - t0)
    ms = sorted(times)[len(times) // 2] * 1e3
    h2d, d2h = 14 * n, 14 * n
    # one-direction copies of the same bytes alone, for the overlap figure
    dbuf = torch.empty(h2d, dtype=torch.uint8, device=dev)
    hbuf = be.allocate_tensor((h2d,), torch.uint8)
    alone = {}
    for name, (dst, src) in (("h2d", (dbuf, hbuf)), ("d2h", (hbuf, dbuf))):
        dst.copy_(src, non_blocking=True)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        dst.copy_(src, non_blocking=True)
        torch.cuda.synchronize()
        alone[name] = (time.perf_counter() - t0) * 1e3
    # what the link gives when both directions carry one plain copy of the same bytes at once: the ceiling of
    # any overlapped schedule (a direction alone is faster than either direction of a concurrent pair)
    dbuf2 = torch.empty(h2d, dtype=torch.uint8, device=dev)
    hbuf2 = be.allocate_tensor((h2d,), torch.uint8)
    both = []
    for _ in range(3):
        sb.synchronize_all()
        t0 = time.perf_counter()
        with torch.cuda.stream(sb.inbound):
            dbuf.copy_(hbuf, non_blocking=True)
        with torch.cuda.stream(sb.outbound):
            hbuf2.copy_(dbuf2, non_blocking=True)
        sb.synchronize_all()
        both.append((time.perf_counter() - t0) * 1e3)
    both_ms = sorted(both)[1]
    be.release(hbuf2)
    del dbuf2
    row = {"op": "c4.adamw streamed from pinned host (fp32 p/m/v, bf16 g, bf16 copy-out; 3 slots x 4Mi elements)",
           "algorithmic": h2d + d2h, "ms": round(ms, 3), "achieved": round((h2d + d2h) / (ms * 1e-3) / 1e9, 2),
           "unit": "GB/s (host link, both directions summed)", "frac": None,
           "h2d_GBps": round(h2d / (ms * 1e-3) / 1e9, 2), "d2h_GBps": round(d2h / (ms * 1e-3) / 1e9, 2),
           "copy_alone_ms": {k: round(v, 3) for k, v in alone.items()},
           "overlap_efficiency": round(max(alone.values()) / ms, 4),
           "plain_copies_both_directions_at_once_ms": round(both_ms, 3),
           "frac_of_concurrent_link_ceiling": round(both_ms / ms, 4)}
    for t in host.values():
        be.release(t)
    be.release(hbuf)
    return [row]


def run_lm_head(torch, dev, stream, rn):
    """configs[2]: chunked linear cross-entropy fwd+bwd, hidden [8192,4096], lm_head
    [128256,4096] (stored (V, d); the head sees the transposed view), chunk 1024."""
    from flextrain_amd.head import LMHead, LMHeadConfig
    from flextrain_amd.loss import TokenContext
    from flextrain_amd.matmul_dispatcher import CublasLtDispatcher

    T, d, V, chunk = 8192, 4096, 128256, 1024
    x0 = rn(T, d).to(dev)
    w = (torch.randn(V, d, device=dev) * 0.02).to(torch.bfloat16)
    w_norm = torch.ones(d, dtype=torch.float32, device=dev)
    labels = torch.randint(0, V, (T,), device=dev)
    labels[torch.rand(T, device=dev) < 0.1] = -100
    g_store = torch.zeros(V, d, dtype=torch.float32, device=dev)
    g_norm = torch.zeros(d, dtype=torch.float32, device=dev)
    head = None
    grads = {"g_head_proj": g_store.t(), "g_final_norm": g_norm}
    scale = 1.0 / int((labels != -100).sum())
    x = x0.clone()

    def run():
        x.copy_(x0)
        head.forward_backward(x, TokenContext(labels=labels), None, {"w_final_norm": w_norm, "w_head_proj": w.t()},
                              grads, None, loss_scale=scale)

    rows = []
    chunk_bytes = chunk * V * 2
    g_bf16 = torch.zeros(V, d, dtype=torch.bfloat16, device=dev)

    def head_row(name, fuse, g_head):
        nonlocal head
        head = LMHead(LMHeadConfig(d_model=d, vocab_size=V, head_chunk_size=chunk, fuse_chunks=fuse))
        grads["g_head_proj"] = g_head.t()
        ms = _time_launches(torch, stream, [run], warmup=1, reps=3)
        row = _op_entry(name, 6 * T * d * V, "TFLOP/s", ms)
        groups = fuse if fuse is not None else max(1, min(T // chunk, head.cfg.logits_buffer_bytes // chunk_bytes))
        row["logits_buffer_MB"] = round(groups * chunk_bytes / 1e6)
        row["head_gradient"] = str(g_head.dtype).replace("torch.", "")
        rows.append(row)

    # The reference's own schedule and gradient type first (one 1024-token logits buffer; torch.addmm
    # into a compute-dtype accumulator, flextrain/nn/head.py:82-84, :324-331: the head's default here
    # too), then the same with the fp32 accumulator this package also takes, then the opt-in 8-chunk
    # GEMM groups (a 2.1 GB logits buffer).
    head_row("c3.lm_head fwd+bwd (chunk 1024, one GEMM group per chunk and bf16 dW += as the reference)", 1, g_bf16)
    head_row("c3.lm_head fwd+bwd (chunk 1024, one GEMM group per chunk, fp32 dW +=)", 1, g_store)
    head_row("c3.lm_head fwd+bwd (chunk 1024 x 8 per GEMM group: opt-in, fp32 dW +=)", 8, g_store)
    # the three GEMMs of one micro-chunk, timed alone
    disp = CublasLtDispatcher()
    sp = stream.cuda_stream
    h = rn(chunk, d).to(dev)
    logits = torch.empty(chunk, V, dtype=torch.bfloat16, device=dev)
    dxh = torch.empty(chunk, d, dtype=torch.bfloat16, device=dev)
    gt = g_store
    ms = _time_launches(torch, stream, [lambda: disp.matmul_fast(sp, h, w.t(), D=logits)], warmup=2, reps=10)
    rows.append(_op_entry("c3.logits gemm [1024,4096]x[4096,128256]", 2 * chunk * d * V, "TFLOP/s", ms))
    logits.normal_()
    ms = _time_launches(torch, stream, [lambda: disp.matmul_fast(sp, logits.t(), h, C=gt, D=gt, alpha=scale, beta=1.0)],
                        warmup=2, reps=10)
    rows.append(_op_entry("c3.dW gemm [128256,1024]x[1024,4096] (+= fp32)", 2 * chunk * d * V, "TFLOP/s", ms))
    ms = _time_launches(torch, stream, [lambda: disp.matmul_fast(sp, logits.t(), h, C=g_bf16, D=g_bf16, alpha=scale, beta=1.0)],
                        warmup=2, reps=10)
    rows.append(_op_entry("c3.dW gemm [128256,1024]x[1024,4096] (+= bf16)", 2 * chunk * d * V, "TFLOP/s", ms))
    ms = _time_launches(torch, stream, [lambda: disp.matmul_fast(sp, logits, w, D=dxh)], warmup=2, reps=10)
    rows.append(_op_entry("c3.dX gemm [1024,128256]x[128256,4096]", 2 * chunk * d * V, "TFLOP/s", ms))
    # For comparison only (not a product path): the vendor BLAS, which the reference's cuBLASLt
    # dispatcher would map to on this hardware, on the same operands in the same run.
    with torch.cuda.stream(stream):
        ms = _time_launches(torch, stream, [lambda: torch.matmul(h, w.t(), out=logits)], warmup=2, reps=10)
        rows.append(_op_entry("c3.logits gemm, vendor BLAS through torch.matmul (comparison)", 2 * chunk * d * V, "TFLOP/s", ms))
        logits.normal_()
        ms = _time_launches(torch, stream, [lambda: torch.matmul(logits, w, out=dxh)], warmup=2, reps=10)
        rows.append(_op_entry("c3.dX gemm, vendor BLAS through torch.matmul (comparison)", 2 * chunk * d * V, "TFLOP/s", ms))
    from flextrain_amd import ops
    lab = labels[:chunk].contiguous()
    loss = torch.empty(chunk, dtype=torch.float32, device=dev)
    ms = _time_launches(torch, stream, [lambda: ops.flextrain_softmax_cross_entropy(logits, lab, L=loss)], warmup=2, reps=10)
    # two reads and one write of the logits chunk (the row does not stay in registers at V = 128256)
    row = _op_entry("c3.softmax_ce [1024,128256] in place", 3 * chunk * V * 2, "GB/s", ms)
    # the same launch priced by the least any implementation must move (one read, one write of the chunk)
    minimal = _op_entry("", 2 * chunk * V * 2, "GB/s", ms)
    row["bytes_counted"] = "two reads + one write of the logits chunk (what this kernel requests)"
    row["achieved_by_minimal_bytes"] = minimal["achieved"]
    row["frac_by_minimal_bytes"] = minimal["frac"]
    rows.append(row)
    del w, g_store, g_bf16, logits, x, x0
    torch.cuda.empty_cache()
    return rows


def run_hw_probe(torch, dev):
    """The inputs of the save-level solver as the library's probe measures them on this box
    (sustained GEMM rate on random operands, HBM streaming rate, concurrent host-link rate)."""
    from flextrain_amd.hw_probe import probe_hardware

    r = probe_hardware(device=dev, matmul_target_seconds=3.0, mem_bw_target_seconds=1.0)
    return [{"op": "probe.save-level solver inputs (8192^3 bf16 GEMM, two-half sustained window)", "algorithmic": None,
             "ms": round(r.matmul_per_call_ms, 4), "achieved": round(r.achieved_tflops_second_half, 1), "unit": "TFLOP/s",
             "frac": round(r.achieved_tflops_second_half / BF16_PEAK_TFLOPS, 4),
             "tflops_first_half": round(r.achieved_tflops_first_half, 1), "hbm_stream_GBps": round(r.mem_bw_gbps, 1),
             "host_link_GBps_each_direction_concurrent": round(r.hw_cost.pcie_bw_gbps, 2)}]


def run_activation_slots(torch, dev):
    """Activation-slot streaming of one Llama-3.1-8B-shaped decoder layer at save level 3 (every
    saved tensor of 8192 tokens): send_home from the HBM ring into a pinned home slot, fetch_home
    back, and both at once on the outbound / inbound streams.  The host link is the roof."""
    from flextrain_amd.activation_schema import ActivationField, ActivationSchema, ActivationSlot, fetch_home, send_home
    from flextrain_amd.host_memory import LocalPinnedHostBackend
    from flextrain_amd.streams import StreamBundle

    bf, f32 = torch.bfloat16, torch.float32
    dims = {"d": 4096, "kv": 1024, "H": 32, "F": 14336}
    F = ActivationField
    schema = ActivationSchema((
        F("x_inp", lambda T, m: (T, m["d"]), bf, 0), F("attn_norm_rstd", lambda T, m: (T, 1), f32, 0),
        F("xk", lambda T, m: (T, m["kv"]), bf, 0), F("xv", lambda T, m: (T, m["kv"]), bf, 0),
        F("attn_result", lambda T, m: (T, m["d"]), bf, 1), F("softmax_lse", lambda T, m: (m["H"], T), f32, 1, token_axis=1),
        F("xq", lambda T, m: (T, m["d"]), bf, 2), F("xo", lambda T, m: (T, m["d"]), bf, 2),
        F("ffn_norm_rstd", lambda T, m: (T, 1), f32, 0),
        F("x1", lambda T, m: (T, m["F"]), bf, 3), F("x3", lambda T, m: (T, m["F"]), bf, 3)), max_tier=3)
    T, level = 8192, 3
    be = LocalPinnedHostBackend()
    sb = StreamBundle.create(dev)
    nbytes = schema.offloaded_bytes_at_level(T, dims, level)
    ring = torch.empty(2 * schema.device_size_bytes(T, dims), dtype=torch.uint8, device=dev)
    half = ring.numel() // 2
    dev_slots = [ActivationSlot.from_buffer(schema, level, T, dims, ring[i * half:(i + 1) * half], include_nonpersistent=True)[0]
                 for i in range(2)]
    home_bufs = [be.allocate_tensor((schema.home_size_bytes(T, dims, level),), torch.uint8) for _ in range(2)]
    homes = [ActivationSlot.from_buffer(schema, level, T, dims, b)[0] for b in home_bufs]

    def timed(fn):
        fn()
        sb.synchronize_all()
        ts = []
        for _ in range(3):
            t0 = time.perf_counter()
            fn()
            sb.synchronize_all()
            ts.append(time.perf_counter() - t0)
        return sorted(ts)[1] * 1e3

    def out():
        with torch.cuda.stream(sb.outbound):
            send_home(homes[0], dev_slots[0], level)

    def back():
        with torch.cuda.stream(sb.inbound):
            fetch_home(dev_slots[1], homes[1], level)

    def both():
        out()
        back()

    ms_out, ms_in, ms_both = timed(out), timed(back), timed(both)
    row = {"op": "act.activation slot of one decoder layer, 8192 tokens, save level 3 (11 fields, one library call per slot)",
           "algorithmic": nbytes, "unit": "GB/s (host link)", "frac": None,
           "send_home_ms": round(ms_out, 3), "send_home_GBps": round(nbytes / ms_out / 1e6, 2),
           "fetch_home_ms": round(ms_in, 3), "fetch_home_GBps": round(nbytes / ms_in / 1e6, 2),
           "both_directions_ms": round(ms_both, 3), "both_directions_GBps_each": round(nbytes / ms_both / 1e6, 2),
           "ms": round(ms_both, 3), "achieved": round(2 * nbytes / ms_both / 1e6, 2)}
    for b in home_bufs:
        be.release(b)
    return [row]


def run_ffn_dense(torch, dev, stream, rn):
    """Llama-3.1-8B-shaped dense gated FFN block (the GEMMs around the SwiGLU kernels of the headline
    workload): T = 8192 tokens, d = 4096, F = 14336, bf16 weights and gradients."""
    import types

    from flextrain_amd.ffn_dense import SwiGLUConfig, SwiGLUFFN

    T, d, F = 8192, 4096, 14336
    bf = torch.bfloat16
    h, resid, dy = rn(T, d).to(dev), rn(T, d).to(dev), rn(T, d).to(dev)
    W = {"w_1": (torch.randn(d, F, device=dev) * 0.02).to(bf), "w_3": (torch.randn(d, F, device=dev) * 0.02).to(bf),
         "w_2": (torch.randn(F, d, device=dev) * 0.02).to(bf)}
    G = {"g_" + k[-1]: torch.zeros_like(v) for k, v in W.items()}
    slot = types.SimpleNamespace(x1=torch.empty(T, F, dtype=bf, device=dev), x3=torch.empty(T, F, dtype=bf, device=dev), aux={})
    act_buf = torch.empty(T, F, dtype=bf, device=dev)
    ctx = types.SimpleNamespace(scratch=lambda shape, dtype: act_buf)
    out = torch.empty(T, d, dtype=bf, device=dev)
    blk = SwiGLUFFN(SwiGLUConfig(d_model=d, expert_dim=F))

    def fwd():
        blk.fwd(h, W, resid, out, slot, ctx)

    def bwd():
        blk.bwd(dy, W, G, slot)
        blk.bwd_accumulate_w1_w3_grads(h, G, slot)

    unit = 2 * T * d * F
    ms_f = _time_launches(torch, stream, [fwd], warmup=2, reps=5)
    ms_b = _time_launches(torch, stream, [bwd], warmup=2, reps=5)
    # single GEMMs of the block, and the vendor BLAS on the same operands for comparison
    from flextrain_amd import ops
    sp = stream.cuda_stream
    x1 = slot.x1
    extra_rows = []
    ms = _time_launches(torch, stream, [lambda: ops.dispatcher.matmul_fast(sp, h, W["w_1"], D=x1)], warmup=2, reps=10)
    extra_rows.append(_op_entry("ffn.gate gemm [8192,4096]x[4096,14336] (weights (d,F) as the reference stores them)", unit, "TFLOP/s", ms))
    ms = _time_launches(torch, stream, [lambda: ops.dispatcher.matmul_fast(sp, act_buf, W["w_2"], D=out)], warmup=2, reps=10)
    extra_rows.append(_op_entry("ffn.down gemm [8192,14336]x[14336,4096]", unit, "TFLOP/s", ms))
    with torch.cuda.stream(stream):
        ms = _time_launches(torch, stream, [lambda: torch.matmul(h, W["w_1"], out=x1)], warmup=2, reps=10)
        extra_rows.append(_op_entry("ffn.gate gemm, vendor BLAS through torch.matmul (comparison)", unit, "TFLOP/s", ms))
        ms = _time_launches(torch, stream, [lambda: torch.matmul(act_buf, W["w_2"], out=out)], warmup=2, reps=10)
        extra_rows.append(_op_entry("ffn.down gemm, vendor BLAS through torch.matmul (comparison)", unit, "TFLOP/s", ms))
    return extra_rows + [_op_entry("ffn.dense block fwd (3 GEMMs + SwiGLU, residual in the down-projection epilogue)", 3 * unit, "TFLOP/s", ms_f),
            _op_entry("ffn.dense block bwd (6 GEMMs + SwiGLU bwd)", 6 * unit, "TFLOP/s", ms_b),
            _op_entry("ffn.dense block fwd+bwd", 9 * unit, "TFLOP/s", ms_f + ms_b)]


def run_attention_proj(torch, dev, stream, rn):
    """Llama-3.1-8B-shaped attention block without its core (the projections around the RoPE kernel of
    the headline workload): T = 8192 tokens, d = 4096, 32 query heads, 8 key/value heads of 128."""
    import types

    from flextrain_amd.attention_proj import GQAAttentionProjections, GQAProjectionConfig

    T = 8192
    cfg = GQAProjectionConfig(d_model=4096, n_heads=32, n_kv_heads=8, head_dim=128, rope_theta=500000.0)
    bf = torch.bfloat16
    x, resid, dy = rn(T, cfg.d_model).to(dev), rn(T, cfg.d_model).to(dev), rn(T, cfg.d_model).to(dev)
    pos = torch.arange(T, dtype=torch.int32, device=dev).view(T, 1)
    shapes = {"q": (cfg.d_model, cfg.attn_dim), "k": (cfg.d_model, cfg.kv_dim), "v": (cfg.d_model, cfg.kv_dim),
              "o": (cfg.attn_dim, cfg.d_model)}
    W = {"w_" + k: (torch.randn(*sh, device=dev) * 0.02).to(bf) for k, sh in shapes.items()}
    G = {"g_" + k: torch.zeros(*sh, dtype=bf, device=dev) for k, sh in shapes.items()}
    slot = types.SimpleNamespace(
        xq=torch.empty(T, cfg.n_heads, cfg.head_dim, dtype=bf, device=dev), xk=torch.empty(T, cfg.n_kv_heads, cfg.head_dim, dtype=bf, device=dev),
        xv=torch.empty(T, cfg.n_kv_heads, cfg.head_dim, dtype=bf, device=dev), attn_result=rn(T, cfg.n_heads, cfg.head_dim).to(dev),
        xo=torch.empty(T, cfg.d_model, dtype=bf, device=dev), aux={})
    dq, dk, dv = rn(T, cfg.n_heads, cfg.head_dim).to(dev), rn(T, cfg.n_kv_heads, cfg.head_dim).to(dev), rn(T, cfg.n_kv_heads, cfg.head_dim).to(dev)
    blk = GQAAttentionProjections(cfg)

    def fwd():
        blk.fwd_qkv(x, pos, W, slot)
        blk.fwd_o(resid, W, slot)

    def bwd():
        blk.bwd_o(dy, W, G, slot)
        blk.bwd_qkv(dq, dk, dv, pos, W, G, slot)
        blk.bwd_accumulate_qkv_grads(x, G, slot)

    fl = blk.projection_flops(T)
    ms_f = _time_launches(torch, stream, [fwd], warmup=2, reps=5)
    ms_b = _time_launches(torch, stream, [bwd], warmup=2, reps=5)
    return [_op_entry("attn.projections fwd (Q/K/V GEMMs + RoPE, O-projection with the residual in its epilogue)", fl, "TFLOP/s", ms_f),
            _op_entry("attn.projections bwd (8 GEMMs + RoPE bwd)", 2 * fl, "TFLOP/s", ms_b),
            _op_entry("attn.projections fwd+bwd", 3 * fl, "TFLOP/s", ms_f + ms_b)]


def run_moe(torch, dev, stream, rn):
    """configs[4]: Qwen3-30B-A3B-shaped routed-SwiGLU block fwd+bwd."""
    import types

    from flextrain_amd import full_moe
    from flextrain_amd.moe_backend import FlextrainMoEExpertCompute
    from flextrain_amd.ops.grouped import flextrain_grouped_gemm_rows, flextrain_grouped_gemm_wgrad

    T, d, E, K, F = 8192, 2048, 128, 8, 768
    TK = T * K
    bf = torch.bfloat16
    x, dy = rn(T, d).to(dev), rn(T, d).to(dev)
    weights = dict(w_router=rn(d, E, std=0.02).to(dev),
                   w_up=(torch.randn(E, 2 * F, d, device=dev) * 0.02).to(bf),
                   w_down=(torch.randn(E, d, F, device=dev) * 0.02).to(bf))
    grads = dict(g_router=torch.zeros(d, E, dtype=bf, device=dev), g_up=torch.zeros(E, 2 * F, d, dtype=bf, device=dev),
                 g_down=torch.zeros(E, d, F, dtype=bf, device=dev))
    slot = types.SimpleNamespace(
        x_router=torch.empty(T, E, dtype=bf, device=dev), chosen_experts=torch.empty(T, K, dtype=torch.int32, device=dev),
        router_weights=torch.empty(T, K, dtype=bf, device=dev), index_mapping=torch.empty(T, K, dtype=torch.int32, device=dev),
        expert_counts=torch.empty(E, dtype=torch.int32, device=dev),
        scattered_router_weights=torch.empty(TK, 1, dtype=bf, device=dev), x_up=torch.empty(TK, 2 * F, dtype=bf, device=dev),
        aux={})
    backend = FlextrainMoEExpertCompute()
    pool = {}

    def scratch(shape, dtype):   # a fixed scratch pool, as the engine's LayerContext provides
        key = (tuple(shape), dtype, sum(1 for k in pool if k[:2] == (tuple(shape), dtype) and pool[k][1]))
        if key not in pool:
            pool[key] = [torch.empty(shape, dtype=dtype, device=dev), False]
        pool[key][1] = True
        return pool[key][0]

    out = torch.empty(T, d, dtype=bf, device=dev)
    extra = {}
    common = dict(slot=slot, chunk_extra=extra, layer_id=0, primary_stream=stream, secondary_stream=None,
                  scratch_fn=scratch, expert_compute=backend)

    def release():
        for v in pool.values():
            v[1] = False

    def fwd():
        release()
        full_moe.routed_swiglu_moe_fwd(x, weights, out_tensor=out, residual=x, top_k=K, num_experts=E,
                                       routing_mode="topk_then_softmax", **common)

    def bwd(secondary=None):
        release()
        full_moe.routed_swiglu_moe_bwd(dy, weights, grads, slot, extra, 0, ffn_norm_output=x, top_k=K, num_experts=E,
                                       routing_mode="topk_then_softmax", load_balance_coef=0.0,
                                       total_tokens_per_step=None, primary_stream=stream, secondary_stream=secondary,
                                       scratch_fn=scratch, expert_compute=backend)

    rows = []
    fl_fwd = 6 * TK * d * F + 2 * T * d * E
    fl_bwd = 12 * TK * d * F + 4 * T * d * E
    ms_f = _time_launches(torch, stream, [fwd], warmup=2, reps=5)
    rows.append(_op_entry("c5.moe block fwd (route+sort+scatter+experts+gather)", fl_fwd, "TFLOP/s", ms_f))
    ms_b = _time_launches(torch, stream, [bwd], warmup=2, reps=5)
    rows.append(_op_entry("c5.moe block bwd", fl_bwd, "TFLOP/s", ms_b))
    rows.append(_op_entry("c5.moe block fwd+bwd", fl_fwd + fl_bwd, "TFLOP/s", ms_f + ms_b))
    # the grouped GEMMs alone, on the routing the block just produced
    counts = slot.expert_counts
    sx = torch.randn(TK, d, device=dev).to(bf)
    pre = slot.x_up
    act = torch.randn(TK, F, device=dev).to(bf)
    ms = _time_launches(torch, stream, [lambda: flextrain_grouped_gemm_rows(sx, weights["w_up"].transpose(1, 2), counts, pre)],
                        warmup=2, reps=10)
    def floor(row, flop, nbytes):
        # the least time the launch can take: its MFMA work at the published peak, or its HBM bytes
        # (operands and results once, accumulated gradients read and written) at 8 TB/s
        row["floor_ms"] = round(max(flop / (BF16_PEAK_TFLOPS * 1e12), nbytes / (HBM_PEAK_GBPS * 1e9)) * 1e3, 4)
        row["floor_bound"] = "mfma" if flop / (BF16_PEAK_TFLOPS * 1e12) >= nbytes / (HBM_PEAK_GBPS * 1e9) else "hbm"
        row["hbm_bytes"] = nbytes
        return row

    rows.append(floor(_op_entry("c5.grouped up-proj [65536,2048]x128x[2048,1536]", 2 * TK * d * 2 * F, "TFLOP/s", ms),
                      2 * TK * d * 2 * F, 2 * (TK * d + E * 2 * F * d + TK * 2 * F)))
    ms = _time_launches(torch, stream, [lambda: flextrain_grouped_gemm_rows(act, weights["w_down"].transpose(1, 2), counts, sx)],
                        warmup=2, reps=10)
    rows.append(floor(_op_entry("c5.grouped down-proj [65536,768]x128x[768,2048]", 2 * TK * d * F, "TFLOP/s", ms),
                      2 * TK * d * F, 2 * (TK * F + E * F * d + TK * d)))
    ms = _time_launches(torch, stream, [lambda: flextrain_grouped_gemm_wgrad(pre, sx, grads["g_up"], counts)], warmup=2, reps=10)
    rows.append(floor(_op_entry("c5.grouped wgrad g_up [1536,T_e]x[T_e,2048] x128 (+= bf16)", 2 * TK * d * 2 * F, "TFLOP/s", ms),
                      2 * TK * d * 2 * F, 2 * (TK * 2 * F + TK * d + 2 * E * 2 * F * d)))
    del sx, act, x, dy, out, weights, grads, slot
    pool.clear()
    torch.cuda.empty_cache()
    return rows


def _moe_reference_microbench(torch, dev, stream, rn):
    """The shape and scope of the reference's own MoE micro-benchmark
    (external_moe_impl/bench/bench_moe.py:4-13): d 2048, F 512, 256 experts, top-8, 16 K tokens;
    routed-MLP scope = scatter -> experts -> weighted gather (no router GEMM, no residual) forward,
    dy -> dx, g_up, g_down backward."""
    import types

    from flextrain_amd.moe_backend import FlextrainMoEExpertCompute
    from flextrain_amd.ops.moe import flextrain_fused_topk_softmax

    T, d, E, K, F = 16384, 2048, 256, 8, 512
    TK = T * K
    bf = torch.bfloat16
    x, dy = rn(T, d).to(dev), rn(T, d).to(dev)
    weights = dict(w_up=(torch.randn(E, 2 * F, d, device=dev) * 0.02).to(bf), w_down=(torch.randn(E, d, F, device=dev) * 0.02).to(bf))
    grads = dict(g_up=torch.zeros(E, 2 * F, d, dtype=bf, device=dev), g_down=torch.zeros(E, d, F, dtype=bf, device=dev))
    slot = types.SimpleNamespace(
        index_mapping=torch.empty(T, K, dtype=torch.int32, device=dev), expert_counts=torch.empty(E, dtype=torch.int32, device=dev),
        scattered_router_weights=torch.empty(TK, 1, dtype=bf, device=dev), x_up=torch.empty(TK, 2 * F, dtype=bf, device=dev), aux={})
    logits = torch.randn(T, E, device=dev).to(bf)
    ids = torch.empty(T, K, dtype=torch.int32, device=dev)
    probs = torch.empty(T, K, dtype=bf, device=dev)
    flextrain_fused_topk_softmax(logits, top_k=K, topk_ids_out=ids, topk_weights_out=probs, mode="topk_then_softmax")
    backend = FlextrainMoEExpertCompute()
    bufs = {}

    def scratch(shape, dtype):
        key = (tuple(shape), dtype, sum(1 for k in bufs if k[:2] == (tuple(shape), dtype) and bufs[k][1]))
        if key not in bufs:
            bufs[key] = [torch.empty(shape, dtype=dtype, device=dev), False]
        bufs[key][1] = True
        return bufs[key][0]

    def release():
        for v in bufs.values():
            v[1] = False

    out, dx, extra = torch.empty(T, d, dtype=bf, device=dev), torch.empty(T, d, dtype=bf, device=dev), {}
    common = dict(slot=slot, chunk_extra=extra, layer_id=0, primary_stream=stream, secondary_stream=None, scratch_fn=scratch)

    def fwd():
        release()
        backend.fwd(x, probs, ids, weights, out=out, residual=None, **common)

    def bwd():
        release()
        backend.bwd(dy, x, weights, grads, dx=dx, **common)
        slot.aux.pop("moe_dprobs", None)

    ms_f = _time_launches(torch, stream, [fwd], warmup=2, reps=5)
    ms_b = _time_launches(torch, stream, [bwd], warmup=2, reps=5)
    name = "moe_ref.routed MLP, the reference's micro-benchmark shape (16384 tokens, d 2048, F 512, 256 experts, top-8)"
    return [_op_entry(name + " fwd", 6 * TK * d * F, "TFLOP/s", ms_f), _op_entry(name + " bwd", 12 * TK * d * F, "TFLOP/s", ms_b),
            _op_entry(name + " fwd+bwd", 18 * TK * d * F, "TFLOP/s", ms_f + ms_b)]


def _cpu_model():
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.lower().startswith("model name"):
                    return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def _cpu_time(fn, budget_s, max_runs=50):
    """Median wall time of fn() over as many runs as fit budget_s (at least one, after one warm-up
    when a run is short)."""
    t0 = time.perf_counter()
    fn()
    first = time.perf_counter() - t0
    if first > budget_s / 2:
        return first, 1
    times = []
    t_begin = time.perf_counter()
    while len(times) < 3 or (time.perf_counter() - t_begin < budget_s and len(times) < max_runs):
        t1 = time.perf_counter()
        fn()
        times.append(time.perf_counter() - t1)
    times.sort()
    return times[len(times) // 2], len(times)


def run_cpu_baselines(torch, only):
    """The CPU oracle (the eager PyTorch formulas the reference keeps as its own checks, restated under
    oracle/) timed on this machine's host cores on a bounded sample of each configuration other than
    the headline one; work is scaled to the sample."""
    from oracle import adamw as o_adam
    from oracle import linear_ce as o_ce
    from oracle import moe as o_moe
    from oracle import rmsnorm as o_norm

    want = lambda tag: not only or tag in only
    cores = os.cpu_count() or 1
    torch.set_num_threads(cores)
    model = _cpu_model()
    bf = torch.bfloat16
    g = torch.Generator().manual_seed(1000)
    rows = []

    def row(name, work, unit, sec, runs, sample):
        r = _op_entry(name, work, unit, sec * 1e3)
        r.update({"cores": torch.get_num_threads(), "cpu_model": model, "kind": "port",
                  "sample": f"{sample}; median of {runs} run(s), {sec * 1e3:.1f} ms each"})
        return r

    if want("c1"):
        T, D = 2048, 4096
        x = torch.randn(T, D, generator=g).to(bf)
        w = (1 + 0.02 * torch.randn(D, generator=g)).to(bf)
        dy = torch.randn(T, D, generator=g).to(bf)

        def c1():
            _, rstd = o_norm.rmsnorm_fwd(x, w)
            o_norm.rmsnorm_bwd(dy, x, w, rstd)

        sec, runs = _cpu_time(c1, 3.0)
        rows.append(row("c1.cpu_baseline rmsnorm fwd+bwd", (2 + 3) * T * D * 2 + 2 * D * 2 + 2 * T * 4 + D * 4, "GB/s", sec, runs,
                        "CPU oracle on the whole configuration ([2048,4096])"))
    if want("c3"):
        Ts, d, V = 1024, 4096, 128256
        x = torch.randn(Ts, d, generator=g).to(bf)
        wh = (torch.randn(d, V, generator=g) * 0.02).to(bf)
        wn = torch.ones(d)
        lab = torch.randint(0, V, (Ts,), generator=g)
        lab[torch.rand(Ts, generator=g) < 0.1] = -100
        sec, runs = _cpu_time(lambda: o_ce.head_forward_backward(x, wn, wh, lab, chunk=1024, loss_scale=1.0 / Ts), 0.0)
        rows.append(row("c3.cpu_baseline linear cross-entropy fwd+bwd", 6 * Ts * d * V, "TFLOP/s", sec, runs,
                        "CPU oracle on one 1024-token chunk of the 8192 tokens (fp32 GEMMs over the whole vocabulary)"))
        del wh, x
    if want("c4"):
        n = 218_112_000 // 16
        p = torch.randn(n, generator=g) * 0.02
        gr = (torch.randn(n, generator=g) * 1e-3).to(bf)
        m, v = torch.zeros(n), torch.zeros(n)
        step = [0]

        def c4():
            step[0] += 1
            o_adam.adamw_step(p, gr, m, v, lr=3e-5, beta1=0.9, beta2=0.95, eps=1e-8, weight_decay=0.1, step=step[0])

        sec, runs = _cpu_time(c4, 3.0)
        rows.append(row("c4.cpu_baseline adamw step + bf16 copy-out", 28 * n, "GB/s", sec, runs,
                        "CPU oracle on 1/16 of the chunk (13,632,000 parameters)"))
    if want("c5"):
        T, d, E, K, F = 512, 2048, 8, 8, 768
        x = torch.randn(T, d, generator=g).to(bf)
        dy = torch.randn(T, d, generator=g).to(bf)
        wr = (torch.randn(d, E, generator=g) * 0.02).to(bf)
        wu = (torch.randn(E, 2 * F, d, generator=g) * 0.02).to(bf)
        wd = (torch.randn(E, d, F, generator=g) * 0.02).to(bf)

        def c5():
            logits = (x.float() @ wr.float()).to(bf)
            o_moe.routed_block_fwd_bwd(x, logits, wr, wu, wd, x, dy, K)

        sec, runs = _cpu_time(c5, 3.0)
        rows.append(row("c5.cpu_baseline moe block fwd+bwd", 18 * T * K * d * F + 6 * T * d * E, "TFLOP/s", sec, runs,
                        "CPU oracle on 1/16 of the block: 512 tokens, 8 experts, top-8 (512 rows per expert as in the "
                        "full block)"))
    if want("a15"):
        rows += run_dp_solver(model)
    return rows


def run_dp_solver(cpu_model):
    """The save-level solver (host code) beside the reference's own C solver, compiled from the
    reference's source under oracle/_ref: one planning problem of 32 layers x 8 chunks, 4 options per
    task, 8 activation slots, 0.1 ms ticks.  Both must return the same option vector."""
    import ctypes

    import numpy as np

    from flextrain_amd._lib import lib

    T, k, N, scale = 256, 4, 8, 10
    rng = np.random.default_rng(15)
    compute = rng.uniform(3.0, 9.0, T)
    durations = np.ascontiguousarray(np.sort(rng.uniform(0.5, 12.0, (T, k)), axis=1))
    sizes = np.ascontiguousarray(np.sort(rng.uniform(1.0, 100.0, (T, k)), axis=1))
    deadline = float(compute.sum() + durations.max(axis=1).sum() + 1000.0)

    def bind(so):
        so.solve_scheduler.restype = ctypes.c_double
        so.solve_scheduler.argtypes = [ctypes.c_int] * 3 + [ctypes.c_void_p] * 3 + [ctypes.c_double, ctypes.c_int,
                                                                                     ctypes.c_int, ctypes.c_void_p]
        so.compute_buf_size.restype = ctypes.c_int
        so.compute_buf_size.argtypes = [ctypes.c_int] * 3 + [ctypes.c_void_p] * 2 + [ctypes.c_double, ctypes.c_int]
        return so

    def solve_with(so):
        buf = so.compute_buf_size(T, N, k, compute.ctypes.data, durations.ctypes.data, deadline, scale)
        choices = np.zeros(T, dtype=np.int32)
        value = [0.0]

        def once():
            value[0] = so.solve_scheduler(T, N, k, compute.ctypes.data, durations.ctypes.data, sizes.ctypes.data,
                                          deadline, scale, buf, choices.ctypes.data)

        sec, runs = _cpu_time(once, 0.5, max_runs=2000)
        return sec, runs, value[0], choices

    shape = f"T {T} tasks x {k} options, {N} slots, {scale} ticks/ms"
    sec, runs, value, choices = solve_with(lib())
    rows = [{"op": f"a15.save-level solver, host C++ ({shape})", "algorithmic": None, "ms": round(sec * 1e3, 5),
             "achieved": round(1.0 / sec, 1), "unit": "solves/s", "frac": None, "cores": 1, "cpu_model": cpu_model,
             "sample": f"median of {runs} solves"}]
    ref_path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "oracle", "_ref", "libts_ref.so")
    if os.path.exists(ref_path):
        rsec, rruns, rvalue, rchoices = solve_with(bind(ctypes.CDLL(ref_path)))
        rows.append({"op": f"a15.cpu_baseline save-level solver, the reference's C source compiled ({shape})",
                     "algorithmic": None, "ms": round(rsec * 1e3, 5), "achieved": round(1.0 / rsec, 1), "unit": "solves/s",
                     "frac": None, "cores": 1, "cpu_model": cpu_model, "kind": "reference",
                     "same_answer": bool(value == rvalue and np.array_equal(choices, rchoices)),
                     "sample": f"median of {rruns} solves; the product solver takes {sec / rsec:.2f} of its time"})
    return rows


def main():
    args = _parse()
    if args.gpus != 1:
        print(f"bench.py measures one GPU only (got --gpus {args.gpus}); "
              "this path has no multi-GPU leg.", file=sys.stderr)
        sys.exit(2)

    import torch

    import __graft_entry__
    __graft_entry__.ensure_built()   # uses the library that is built; builds only when there is none

    from flextrain_amd import ops
    from flextrain_amd._lib import lib

    lib()  # fail loudly before any timing if the native library is missing
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    # Every launch of this script, torch's and the library's, goes to ONE stream, made current here for
    # the whole run: inputs are produced on the stream that the timed launches consume them on, so no
    # launch can overtake the kernel that writes its operands (routing tables, labels, weights).
    stream = torch.cuda.Stream(device=dev)
    torch.cuda.set_stream(stream)
    timed = Timed(torch, stream)
    _progress("headline workload: inputs")

    # ------------------------------------------------------------------ inputs
    T, HQ, HK, HD, F = 8192, 32, 8, 128, 14336
    g = torch.Generator().manual_seed(1001)

    def rn(*shape, dtype=torch.bfloat16, std=1.0, mean=0.0):
        return (torch.randn(*shape, generator=g, dtype=torch.float32) * std + mean).to(dtype)

    # q/k total 84 MB and would sit in the 256 MB last-level cache from one launch to the next: the
    # step rotates through ROPE_SETS buffer sets (503 MB) so that both RoPE launches read from HBM
    ROPE_SETS = 6
    q0, k0 = rn(T, HQ, HD).to(dev), rn(T, HK, HD).to(dev)
    qs = [q0] + [q0.clone() for _ in range(ROPE_SETS - 1)]
    ks = [k0] + [k0.clone() for _ in range(ROPE_SETS - 1)]
    pos = torch.arange(T, dtype=torch.int32).view(T, 1).to(dev)
    inv_freq = ops.build_rope_inv_freq(HD, 500000.0).to(dev)
    gate, up, dout = rn(T, F).to(dev), rn(T, F).to(dev), rn(T, F).to(dev)
    out, dgate, dup = torch.empty_like(gate), torch.empty_like(gate), torch.empty_like(gate)

    rope_bytes = 2 * T * (HQ + HK) * HD * 2          # read + write, q and k
    n = T * F
    swiglu_fwd_bytes, swiglu_bwd_bytes = 3 * n * 2, 5 * n * 2
    step_bytes = 2 * rope_bytes + swiglu_fwd_bytes + swiglu_bwd_bytes

    step_no = [0]

    def step(rec):
        i = step_no[0] % ROPE_SETS
        j = (step_no[0] + ROPE_SETS // 2) % ROPE_SETS      # the backward rotates a set last touched 3 steps ago
        step_no[0] += 1
        # Only the dominant kernel is bracketed by events inside the timed region (two event records around
        # a 30-200 us launch leave the GPU idle for several microseconds each); the other three kernels get
        # their rows from back-to-back launches after the timed region.
        ops.flextrain_rope_fwd([qs[i], ks[i]], pos, inv_freq)
        ops.flextrain_swiglu_fwd(gate, up, out=out)
        rec("swiglu_bwd", lambda: ops.flextrain_swiglu_bwd(gate, up, dout, dx1=dgate, dx3=dup))
        ops.flextrain_rope_bwd([qs[j], ks[j]], pos, inv_freq)

    # One plain pass of known size (reads and writes 536,870,912 bytes each, as an elementwise NOT so that
    # the launch has a kernel name of its own in a trace): the yardstick that hardware counter runs of
    # this script scale FETCH_SIZE / WRITE_SIZE by.  Larger than the 256 MB last-level cache and issued
    # after the warm-up steps have streamed gigabytes through it, so that its source is read from HBM
    # (a copy of a buffer that was just written is served from that cache and reads ~0).
    calib_src = torch.zeros(512 << 20, dtype=torch.uint8, device=dev)
    calib_dst = torch.empty_like(calib_src)
    untimed = lambda name, fn: fn()
    _progress("headline workload: warm-up, calibration pass, timed steps")
    with torch.cuda.stream(stream):
        for _ in range(args.warmup):
            step(untimed)
        torch.bitwise_not(calib_src, out=calib_dst)
        torch.cuda.synchronize()
        del calib_src, calib_dst
        t0 = time.perf_counter()
        for _ in range(args.steps):
            step(timed)
        torch.cuda.synchronize()
        wall = time.perf_counter() - t0

    ms_per_step = wall * 1e3 / args.steps
    value = step_bytes / (ms_per_step * 1e-3) / 1e9
    work = {"rope_fwd": rope_bytes, "rope_bwd": rope_bytes, "swiglu_fwd": swiglu_fwd_bytes,
            "swiglu_bwd": swiglu_bwd_bytes}
    dom_ms = timed.mean_ms("swiglu_bwd")
    # three rotating buffer sets (2.1 GB): a single 705 MB set would be served in part by the 256 MB last-level cache
    fwd_sets = [(gate, up, out)] + [(torch.randn_like(gate), torch.randn_like(up), torch.empty_like(out)) for _ in range(2)]
    ms_swiglu_fwd = _time_launches(torch, stream, [lambda a=a, b=b, o=o: ops.flextrain_swiglu_fwd(a, b, out=o) for a, b, o in fwd_sets],
                                   warmup=6, reps=48)
    del fwd_sets
    kernel_ms = {"rope_fwd": None, "rope_bwd": None, "swiglu_fwd": ms_swiglu_fwd, "swiglu_bwd": dom_ms}
    op_rows = [_op_entry(f"c2.{name}", work[name], "GB/s", kernel_ms[name] or 1.0) for name in work]
    dom_gbps = swiglu_bwd_bytes / (dom_ms * 1e-3) / 1e9
    roofline = {"kernel": "glu_bwd_kernel<bf16, silu>", "bound": "hbm", "achieved": round(dom_gbps, 1),
                "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": round(dom_gbps / HBM_PEAK_GBPS, 4),
                "traffic": _measured_traffic_bytes(), "algorithmic_bytes": swiglu_bwd_bytes, "avg_ms": round(dom_ms, 5)}
    # RoPE rows: timed over >= 100 back-to-back launches that rotate through the buffer sets (every launch
    # reads from HBM).  Then the same launches on ONE buffer set: the cache-resident case (in a layer q
    # and k come straight out of the projection GEMM).
    for row in op_rows:
        if row["op"] in ("c2.rope_fwd", "c2.rope_bwd"):
            fn = ops.flextrain_rope_fwd if row["op"].endswith("fwd") else ops.flextrain_rope_bwd
            cold = [lambda fn=fn, i=i: fn([qs[i], ks[i]], pos, inv_freq) for i in range(ROPE_SETS)]
            ms = _time_launches(torch, stream, cold, warmup=2 * ROPE_SETS, reps=100)
            row.update(_op_entry(row["op"], rope_bytes, "GB/s", ms))
            row["buffer_sets"] = ROPE_SETS
    for name, fn in (("rope_fwd", ops.flextrain_rope_fwd), ("rope_bwd", ops.flextrain_rope_bwd)):
        ms = _time_launches(torch, stream, [lambda fn=fn: fn([qs[0], ks[0]], pos, inv_freq)], warmup=10, reps=100)
        row = _op_entry(f"c2.{name}, one buffer set re-used (last-level-cache resident; not an HBM figure)", rope_bytes,
                        "GB/s", ms)
        op_rows.append(row)
    del qs, ks, q0, k0, gate, up, dout, out, dgate, dup

    # ------------------------------------------------- other configurations
    mfma_probe = None
    if not args.no_extra:
        op_rows += run_extra(torch, ops, dev, stream, rn, [t.strip() for t in args.only.split(",") if t.strip()])
        if not any("error" in r for r in op_rows):
            _progress("mfma probe")
            try:
                mfma_probe = run_mfma_probe(torch, dev, stream)
            except Exception as exc:  # noqa: BLE001 - the probe is an annotation: its failure must not cost the rows
                _progress(f"mfma probe FAILED: {type(exc).__name__}: {exc}")
                op_rows.append({"op": "mfma_probe.FAILED", "unit": "", "error": f"{type(exc).__name__}: {exc}"})
            sustained = (mfma_probe or {}).get("random_operands", {}).get("tflops", 0.0)
            for row in op_rows:
                if row["unit"] == "TFLOP/s" and sustained > 0:
                    row["frac_of_sustained_mfma_random_operands"] = round(row["achieved"] / sustained, 4)
    _progress("cpu baselines")

    # -------------------------------------------------------- CPU baseline
    cpu = None
    if not args.no_cpu and not args.no_extra:
        try:
            op_rows += run_cpu_baselines(torch, [t.strip() for t in args.only.split(",") if t.strip()])
        except Exception as exc:  # noqa: BLE001 - reported in the line; the measured GPU rows are kept
            _progress(f"cpu baselines FAILED: {type(exc).__name__}: {exc}")
            op_rows.append({"op": "cpu_baselines.FAILED", "unit": "", "error": f"{type(exc).__name__}: {exc}"})
    if not args.no_cpu:
        from oracle import glu as o_glu
        from oracle import rope as o_rope

        cores = os.cpu_count() or 1
        torch.set_num_threads(cores)
        Ts = 1024  # bounded sample: the first 1024 of the 8192 tokens
        gs = torch.Generator().manual_seed(1001)
        cq = torch.randn(Ts, HQ, HD, generator=gs).to(torch.bfloat16)
        ck = torch.randn(Ts, HK, HD, generator=gs).to(torch.bfloat16)
        cg, cu, cd = (torch.randn(Ts, F, generator=gs).to(torch.bfloat16) for _ in range(3))
        cpos = torch.arange(Ts, dtype=torch.int32).view(Ts, 1)
        cinv = o_rope.vanilla_inv_freq(HD, 500000.0)

        def cpu_step():
            o_rope.rope(cq, cpos, cinv), o_rope.rope(ck, cpos, cinv)
            o_glu.swiglu_fwd(cg, cu)
            o_glu.swiglu_bwd(cg, cu, cd)
            o_rope.rope(cq, cpos, cinv, backward=True), o_rope.rope(ck, cpos, cinv, backward=True)

        cpu_step()
        times = []
        t_begin = time.perf_counter()
        while len(times) < 3 or (time.perf_counter() - t_begin < 12.0 and len(times) < 400):  # about 12 s of CPU work
            t1 = time.perf_counter()
            cpu_step()
            times.append(time.perf_counter() - t1)
        times.sort()
        med = times[len(times) // 2]
        cpu = {"value": round(step_bytes * (Ts / T) / med / 1e9, 3), "unit": "GB/s",
               "cores": torch.get_num_threads(), "kind": "port", "cpu_model": _cpu_model(),
               "sample": f"CPU oracle (PyTorch fp32 formulas) on the first {Ts} of {T} tokens of the same "
                         f"workload, median of {len(times)} runs, {med * 1e3:.1f} ms each"}

    # The MFMA-bound half of the metric: the LM-head logits GEMM of one 1024-token chunk as the kernel
    # record (flop per launch over its event-timed launch duration), with the whole C3 step and the MoE
    # block beside it.
    by_name = {r["op"]: r for r in op_rows}
    roofline_mfma = None
    lg = by_name.get("c3.logits gemm [1024,4096]x[4096,128256]")
    if lg is not None:
        roofline_mfma = {"kernel": "gemm_kernel<bf16, bf16, 256x256x64, 8 waves, A K-contiguous, B K-contiguous> (LM-head logits, "
                                   "one 1024-token chunk)",
                         "bound": "mfma", "achieved": lg["achieved"], "peak": BF16_PEAK_TFLOPS, "unit": "TFLOP/s",
                         "frac": lg["frac"], "flop_per_launch": lg["algorithmic"], "avg_ms": lg["ms"]}
        for key, prefix in (("c3_step_reference_schedule", "c3.lm_head fwd+bwd (chunk 1024, one GEMM group per chunk and bf16"),
                            ("c3_step_8_chunks_per_group_opt_in", "c3.lm_head fwd+bwd (chunk 1024 x 8"),
                            ("c5_moe_block", "c5.moe block fwd+bwd")):
            row = next((r for r in op_rows if r["op"].startswith(prefix)), None)
            if row is not None:
                roofline_mfma[key] = {"ms": row["ms"], "achieved": row["achieved"], "frac": row["frac"]}

    # Last key of the line on purpose: a reader who keeps only the end of the output still sees one
    # figure per configuration (milliseconds, fraction of the roofline that bounds the row).
    def brief(prefix, label):
        row = next((r for r in op_rows if r["op"].startswith(prefix)), None)
        return None if row is None else f"{label} {row['ms']}ms {row['frac']}"

    summary = [t for t in (
        brief("c1.rmsnorm_fwd", "c1.norm_fwd"), brief("c1.rmsnorm_bwd(dX+=,dW+=)", "c1.norm_bwd"),
        brief("c1x16.rmsnorm_fwd", "c1x16.norm_fwd"), brief("c1x16.rmsnorm_bwd", "c1x16.norm_bwd"),
        brief("c2.rope_fwd", "c2.rope_fwd"), brief("c2.rope_bwd", "c2.rope_bwd"), brief("c2.swiglu_fwd", "c2.swiglu_fwd"),
        brief("c2.swiglu_bwd", "c2.swiglu_bwd"),
        brief("c3.lm_head fwd+bwd (chunk 1024, one GEMM group per chunk and bf16", "c3.head chunk1024 bf16dW(ref schedule)"),
        brief("c3.lm_head fwd+bwd (chunk 1024, one GEMM group per chunk, fp32", "c3.head chunk1024 fp32dW"),
        brief("c3.lm_head fwd+bwd (chunk 1024 x 8", "c3.head 8chunks(opt-in) fp32dW"),
        brief("c3.logits gemm [", "c3.logits"), brief("c3.dW gemm [128256,1024]x[1024,4096] (+= fp32)", "c3.dW fp32"),
        brief("c3.dW gemm [128256,1024]x[1024,4096] (+= bf16)", "c3.dW bf16"), brief("c3.dX gemm [", "c3.dX"),
        brief("c3.softmax_ce", "c3.softmax_ce"),
        brief("c4.adamw(fp32 p/m/v, bf16 g, bf16 copy-out)", "c4.adamw+copy"), brief("c4.adamw(fp32 p/m/v, bf16 g)", "c4.adamw"),
        brief("c5.moe block fwd (", "c5.moe_fwd"), brief("c5.moe block bwd", "c5.moe_bwd"), brief("c5.moe block fwd+bwd", "c5.moe"),
        brief("moe_ref.routed MLP, the reference's micro-benchmark shape (16384 tokens, d 2048, F 512, 256 experts, top-8) fwd+bwd", "moe_ref"),
        brief("ffn.gate gemm [", "ffn.gate"), brief("ffn.gate gemm, vendor", "ffn.gate vendor"),
        brief("ffn.down gemm [", "ffn.down"), brief("ffn.down gemm, vendor", "ffn.down vendor"),
        brief("ffn.dense block fwd+bwd", "ffn.block"), brief("attn.projections fwd+bwd", "attn.proj"),
        brief("probe.save-level", "gemm8192^3")) if t is not None]
    solver = [r for r in op_rows if r["op"].startswith("a15.")]
    if solver:
        summary.append("a15.solver " + " vs ".join(f"{r['ms']}ms" + (" (reference, same answer)" if r.get("same_answer") else "")
                                                  for r in solver))
    summary += [f"{r['op']}: {r['error']}" for r in op_rows if "error" in r]

    result = {
        "metric": METRIC,
        "value": round(value, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16 storage, fp32 arithmetic",
        "data": "synthetic",
        "config": {"workload": "configs[1]: Llama-3.1-8B-shaped RoPE (q [8192,32,128], k [8192,8,128], "
                               "theta 5e5; 6 rotating q/k buffer sets) + SwiGLU (gate/up/dout [8192,14336]) "
                               "forward+backward",
                   "algorithmic_bytes_per_step": step_bytes},
        "roofline": roofline,
        "cpu_baseline": cpu,
        "roofline_mfma": roofline_mfma,
        "mfma_probe": mfma_probe,
        "ops": op_rows,
        "summary": summary,
    }
    print(json.dumps(result))


if __name__ == "__main__":
    try:
        main()
    except Exception as exc:  # noqa: BLE001 - the headline itself failed: say so in the one line, then fail
        import traceback

        traceback.print_exc()
        print(json.dumps({"metric": METRIC, "value": None, "unit": "GB/s", "n_gpus": 1,
                          "error": f"{type(exc).__name__}: {exc}"}))
        sys.exit(1)
