"""The bandwidth-bound kernels at the exact shapes bench.py launches them with, in the host simulation on
guard-paged buffers: the headline RoPE and SwiGLU launches (8192 tokens, 32 + 8 heads of 128, 14336-wide
FFN), RMSNorm at 2048 and 32768 tokens of 4096, AdamW on the 218,112,000-parameter chunk and on the
streamed sub-chunks.  Too slow for the test suite (about four minutes, 6 GB); run by hand:

    python -m tests.hostsim.bench_shapes

Every call must return 0; an access outside any buffer ends the process with SIGSEGV."""
from __future__ import annotations

import time

import torch

from . import sim

BF, F32 = torch.bfloat16, torch.float32
G, P = sim.guard, sim.p


def _timed(name, fn):
    t0 = time.time()
    rc = fn()
    print(f"{name}: rc {rc}, {time.time() - t0:.1f} s", flush=True)
    assert rc == 0, name


def main():
    L = sim.lib()
    D = 4096
    for rows in (2048, 32768):
        x, dy, w = G(torch.randn(rows, D).to(BF)), G(torch.randn(rows, D).to(BF)), G(torch.ones(D).to(BF))
        y, rstd = G(torch.empty(rows, D, dtype=BF)), G(torch.empty(rows, dtype=F32))
        _timed(f"rmsnorm fwd [{rows}, {D}]", lambda: L.fx_rmsnorm_fwd(P(x), P(w), P(y), P(rstd), rows, D, 1e-5, 2, 2, 0, None))
        dx, dw = G(torch.zeros(rows, D, dtype=BF)), G(torch.zeros(D))
        nb = int(L.fx_rmsnorm_bwd_ws_bytes(rows, D))
        ws = G(torch.empty(nb // 4))
        for yo in (None, y):
            _timed(f"rmsnorm bwd [{rows}, {D}] (dX +=, dW +=" + (", y)" if yo is not None else ")"),
                   lambda: L.fx_rmsnorm_bwd(P(dy), P(x), P(w), P(rstd), P(dx), 1, P(dw), 0, 1, P(yo) if yo is not None else None, rows, D,
                                            2, 2, P(ws), nb, None))
    T, HQ, HK, HD, F = 8192, 32, 8, 128, 14336
    q, k = G(torch.randn(T, HQ, HD).to(BF)), G(torch.randn(T, HK, HD).to(BF))
    pos, inv = G(torch.arange(T, dtype=torch.int32).view(T, 1)), G(torch.rand(HD // 2))
    strides = lambda t: sim.pi64(G(torch.tensor(t.stride(), dtype=torch.int64)))
    for backward in (0, 1):
        _timed(f"rope q [{T}, {HQ}, {HD}] k [{T}, {HK}, {HD}] backward = {backward}",
               lambda: L.fx_rope(P(q), P(k), P(pos), 1, P(inv), 1, T, HQ, HK, HD, HD, strides(q), strides(k), 2, backward, None))
    n = T * F
    a, b, d = (G(torch.randn(n).to(BF)) for _ in range(3))
    o1, o2 = G(torch.empty(n, dtype=BF)), G(torch.empty(n, dtype=BF))
    _timed(f"swiglu fwd [{T}, {F}]", lambda: L.fx_glu_fwd(P(a), P(b), P(o1), n, 2, 2, 0, None))
    _timed(f"swiglu bwd [{T}, {F}]", lambda: L.fx_glu_bwd(P(a), P(b), P(d), P(o1), P(o2), None, n, 2, 0, None))
    del a, b, d, o1, o2
    chunk, sub = 218_112_000, 4 * 1024 * 1024
    for n in (chunk, sub, chunk % sub):
        p, m, v = G(torch.zeros(n)), G(torch.zeros(n)), G(torch.zeros(n))
        g, c = G(torch.zeros(n, dtype=BF)), G(torch.empty(n, dtype=BF))
        for copy in (c, None):
            _timed(f"adamw {n} parameters, bf16 copy-out = {copy is not None}",
                   lambda: L.fx_adamw_step(P(p), P(g), P(m), P(v), P(copy) if copy is not None else None, n, 0, 2, 0, 3e-5, 0.9, 0.95,
                                           1e-8, 0.1, 0.1, 0.05, None))
    print("all launches stayed inside their buffers")


if __name__ == "__main__":
    main()
