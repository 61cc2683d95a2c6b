"""The per-expert GEMM launches (device-side plan, one-tile and walking workgroups, gated epilogue, gathered
operands, dgrad with the SwiGLU backward in its epilogue) and the fused dense forms, run on the CPU by the
host simulation on guard-paged operands, outputs, row maps and workspaces of exactly the documented sizes,
against fp32 references.  Expert sizes are ragged and include experts without rows, first, in the middle
and last."""
from __future__ import annotations

import ctypes

import pytest
import torch

from oracle import moe as o_moe
from tests.hostsim import sim

from tests.hostsim.build import needs_host_clang

pytestmark = needs_host_clang

BF, F32 = torch.bfloat16, torch.float32
G, P = sim.guard, sim.p


@pytest.fixture(autouse=True, params=["loads land late", "loads land early"])
def dma_timing(request):
    """Every test runs at both extremes of what the hardware may do with a load into LDS: landing only when
    the issuing lane's counted wait says it must have (a read that the wait does not cover sees stale data),
    and landing at its issue (a load into a buffer that other lanes still read shows as wrong results)."""
    sim.lib().hostsim_set_dma_eager(int(request.param == "loads land early"))
    yield
    sim.lib().hostsim_set_dma_eager(0)


def _counts(E, total, g, empty=()):
    w = torch.rand(E, generator=g) + 0.2
    for e in empty:
        w[e] = 0
    c = torch.floor(w / w.sum() * total).to(torch.int64)
    c[int(torch.argmax(c))] += total - int(c.sum())
    return c.to(torch.int32)


def _ws(E, rows):
    n = int(sim.lib().fx_grouped_ws_bytes(E, rows))
    return G(torch.empty(n // 4, dtype=torch.int32)), n


def _close(a, e, tol=1e-2):
    scale = float(e.float().abs().max()) + 1e-6
    torch.testing.assert_close(a.float(), e.float(), rtol=tol, atol=tol * scale)


def _routing(T, K, E, g, empty=()):
    """ids with some experts never chosen -> (mapping (T,K), counts, row sources)."""
    allowed = torch.tensor([e for e in range(E) if e not in empty])
    ids = torch.stack([allowed[torch.randperm(len(allowed), generator=g)[:K]] for _ in range(T)]).to(torch.int32)
    mapping, counts = o_moe.moe_sort(ids, E)
    src = torch.empty(T * K, dtype=torch.int32)
    src[mapping.reshape(-1).long()] = torch.arange(T * K, dtype=torch.int32) // K
    return mapping, counts, src


@pytest.mark.parametrize("E,rows,N,K,empty,trans_b", [
    (4, 300, 136, 72, (), 1),            # small experts: 128-row tiles, 64-wide steps
    (4, 300, 264, 96, (0,), 0),          # K a multiple of 32: the three-stage 32-wide loop; first expert empty
    (3, 1500, 264, 200, (2,), 1),        # 256-row tiles, walking workgroups, last expert empty, K tail
    (5, 2400, 136, 64, (1, 3), 0),
    (2, 9, 8, 8, (), 1),
])
def test_rows(E, rows, N, K, empty, trans_b):
    g = torch.Generator().manual_seed(E * rows + N)
    counts = _counts(E, rows, g, empty)
    A = torch.randn(rows, K, generator=g).to(BF)
    B = (torch.randn(E, N, K, generator=g) if trans_b else torch.randn(E, K, N, generator=g)).to(BF)
    C = torch.randn(rows, N, generator=g).to(BF)
    ws, ws_bytes = _ws(E, rows)
    L = sim.lib()
    for beta in (0.0, 1.0):
        D = G(C) if beta else G(torch.full((rows, N), 3.0, dtype=BF))
        assert L.fx_grouped_gemm_rows(P(G(A)), K, P(G(B)), B.stride(1), B.stride(0), trans_b, P(D) if beta else None, N, P(D), N,
                                      P(G(counts)), E, rows, N, K, 1.0, beta, 2, P(ws), ws_bytes, None) == 0
        ref, off = torch.empty(rows, N), 0
        for e in range(E):
            c = int(counts[e])
            w = B[e].float().t() if trans_b else B[e].float()
            ref[off:off + c] = A[off:off + c].float() @ w + beta * C[off:off + c].float()
            off += c
        _close(D, ref.to(BF))
    # the plan made once, then consumed by a launch that is given no counts
    assert L.fx_grouped_plan(P(G(counts)), E, rows, P(ws), ws_bytes, None) == 0
    D2 = G(torch.empty(rows, N, dtype=BF))
    assert L.fx_grouped_gemm_rows(P(G(A)), K, P(G(B)), B.stride(1), B.stride(0), trans_b, None, N, P(D2), N, None, E, rows, N, K, 1.0,
                                  0.0, 2, P(ws), ws_bytes, None) == 0
    assert torch.equal(D2, D) or True            # (D holds the beta = 1 result); compared below
    D3 = G(torch.empty(rows, N, dtype=BF))
    assert L.fx_grouped_gemm_rows(P(G(A)), K, P(G(B)), B.stride(1), B.stride(0), trans_b, None, N, P(D3), N, P(G(counts)), E, rows, N, K,
                                  1.0, 0.0, 2, P(ws), ws_bytes, None) == 0
    assert torch.equal(D2, D3)


def test_a_foreign_plan_is_not_walked():
    g = torch.Generator().manual_seed(3)
    E, rows, N, K = 4, 1600, 136, 64
    counts = _counts(E, rows, g)
    L = sim.lib()
    ws, ws_bytes = _ws(E, rows)
    ws.fill_(0x7fffffff)                                   # never planned: garbage tile counts and indices
    A, B = torch.randn(rows, K, generator=g).to(BF), torch.randn(E, N, K, generator=g).to(BF)
    D = G(torch.full((rows, N), 5.0, dtype=BF))
    assert L.fx_grouped_gemm_rows(P(G(A)), K, P(G(B)), K, N * K, 1, None, N, P(D), N, None, E, rows, N, K, 1.0, 0.0, 2, P(ws), ws_bytes,
                                  None) == 0
    assert bool((D == 5.0).all())                          # nothing consumed, nothing written, nothing read out of bounds
    small = _counts(E, 300, g)                             # a plan for 128-row tiles offered to a 256-row launch
    ws2, ws2_bytes = _ws(E, rows)
    assert L.fx_grouped_plan(P(G(small)), E, 300, P(ws2), ws2_bytes, None) == 0
    assert L.fx_grouped_gemm_rows(P(G(A)), K, P(G(B)), K, N * K, 1, None, N, P(D), N, None, E, rows, N, K, 1.0, 0.0, 2, P(ws2), ws2_bytes,
                                  None) == 0
    assert bool((D == 5.0).all())


@pytest.mark.parametrize("T,K_top,E,d,F,empty,gathered", [
    (300, 2, 4, 128, 72, (), False),       # 150 rows per expert: 128-row tiles
    (300, 2, 4, 128, 72, (3,), True),
    (1200, 2, 4, 192, 136, (0,), True),    # 600 rows per expert: 256-row tiles
    (1100, 2, 3, 64, 264, (), False),
])
def test_up_projection_with_the_gated_epilogue(T, K_top, E, d, F, empty, gathered):
    g = torch.Generator().manual_seed(T + d + F)
    mapping, counts, src = _routing(T, K_top, E, g, empty)
    rows = T * K_top
    x = torch.randn(T, d, generator=g).to(BF)
    xs = o_moe.moe_scatter(x, mapping)
    w_up = (torch.randn(E, 2 * F, d, generator=g) * d ** -0.5).to(BF)       # rows [value (F) | gate (F)]
    L = sim.lib()
    ws, ws_bytes = _ws(E, rows)
    pre, act = G(torch.empty(rows, 2 * F, dtype=BF)), G(torch.empty(rows, F, dtype=BF))
    a = G(x) if gathered else G(xs)
    rc = L.fx_grouped_gemm_rows_glu(P(a), d, P(G(w_up)), d, 2 * F * d, 1, F * d, P(pre), pre.data_ptr() + 2 * F, 2 * F, P(act), F,
                                    P(G(counts)), E, rows, F, d, 0, 2, P(ws), ws_bytes, P(G(src)) if gathered else None,
                                    T if gathered else 0, None)
    assert rc == 0
    ref_pre, off = torch.empty(rows, 2 * F), 0
    for e in range(E):
        c = int(counts[e])
        ref_pre[off:off + c] = xs[off:off + c].float() @ w_up[e].float().t()
        off += c
    _close(pre, ref_pre.to(BF))
    assert torch.equal(act, o_moe.swiglu_moe_fwd(pre))       # from the rounded products, as a separate kernel would


@pytest.mark.parametrize("T,K_top,E,d,F,empty", [(700, 2, 3, 200, 136, ()), (900, 2, 4, 72, 264, (3,)), (640, 2, 2, 64, 72, ())])
def test_backward_launches_gathered_against_sorted(T, K_top, E, d, F, empty):
    g = torch.Generator().manual_seed(T + d + F + 1)
    mapping, counts, src = _routing(T, K_top, E, g, empty)
    rows = T * K_top
    dy, x = torch.randn(T, d, generator=g).to(BF), torch.randn(T, d, generator=g).to(BF)
    sdy, sx = o_moe.moe_scatter(dy, mapping), o_moe.moe_scatter(x, mapping)
    w_down = (torch.randn(E, d, F, generator=g) * 0.1).to(BF)
    x_up = torch.randn(rows, 2 * F, generator=g).to(BF)
    srw = torch.rand(rows, generator=g).to(BF)
    L = sim.lib()
    ws, ws_bytes = _ws(E, rows)
    part_bytes = int(L.fx_grouped_swiglu_bwd_ws_bytes(rows, F))

    def fused(dy_arg, row_map, dy_rows):
        dx, act, dw = G(torch.empty(rows, 2 * F, dtype=BF)), G(torch.empty(rows, F, dtype=BF)), G(torch.empty(rows, dtype=BF))
        part = G(torch.empty(part_bytes // 4, dtype=F32))
        assert L.fx_grouped_gemm_rows_swiglu_bwd(P(G(dy_arg)), d, P(G(w_down)), F, d * F, 0, P(G(x_up)), 2 * F, P(G(srw)), 2, P(dx), 2 * F,
                                                 P(act), F, P(dw), 2, P(G(counts)), E, rows, F, d, 2, P(ws), ws_bytes, P(part), part_bytes,
                                                 P(G(row_map)) if row_map is not None else None, dy_rows, None) == 0
        return dx, act, dw

    a, b = fused(dy, src, T), fused(sdy, None, 0)
    for got, want in zip(a, b):
        assert torch.equal(got, want)
    # ... and against the two-launch reference: dgrad rounded to bf16, then the weighted SwiGLU backward
    dx_act, off = torch.empty(rows, F), 0
    for e in range(E):
        c = int(counts[e])
        dx_act[off:off + c] = sdy[off:off + c].float() @ w_down[e].float()
        off += c
    rdx, rdw, ract = o_moe.swiglu_moe_bwd(dx_act.to(BF), x_up, srw)
    _close(b[0], rdx, 2e-2), _close(b[1], ract, 2e-2)
    torch.testing.assert_close(b[2].float(), rdw, rtol=3e-2, atol=3e-2 * float(rdw.abs().max()))
    # weight gradients: gathered A (g_down = dy^T act) and gathered B (g_up = dx_up^T x)
    act, dx_up = b[1], b[0]
    for gdt in (BF, F32):
        def wgrad(A, lda, B, ldb, M, N, amap, arows, bmap, brows, base):
            out = G(base)
            assert L.fx_grouped_gemm_wgrad(P(G(A)), lda, P(G(B)), ldb, P(out), N, M * N, sim.DT[gdt], P(G(counts)), E, rows, M, N, 1.0, 1.0, 2,
                                           P(ws), ws_bytes, P(G(amap)) if amap is not None else None, arows,
                                           P(G(bmap)) if bmap is not None else None, brows, None) == 0
            return out
        g0 = torch.randn(E, d, F, generator=g).to(gdt)
        sorted_down = wgrad(sdy, d, act, F, d, F, None, 0, None, 0, g0)
        assert torch.equal(wgrad(dy, d, act, F, d, F, src, T, None, 0, g0), sorted_down)
        ref = g0.float().clone()
        off = 0
        for e in range(E):
            c = int(counts[e])
            ref[e] += sdy[off:off + c].float().t() @ act[off:off + c].float()
            off += c
        _close(sorted_down, ref.to(gdt), 1e-2 if gdt == BF else 1e-5)
        g1 = torch.randn(E, 2 * F, d, generator=g).to(gdt)
        sorted_up = wgrad(dx_up, 2 * F, sx, d, 2 * F, d, None, 0, None, 0, g1)
        assert torch.equal(wgrad(dx_up, 2 * F, x, d, 2 * F, d, None, 0, src, T, g1), sorted_up)
        bad = src.clone()
        bad[::5], bad[1::7] = 1 << 30, -3                        # entries outside the source are clamped
        assert torch.equal(wgrad(dx_up, 2 * F, x, d, 2 * F, d, None, 0, bad, T, g1),
                           wgrad(dx_up, 2 * F, x, d, 2 * F, d, None, 0, bad.clamp(0, T - 1), T, g1))


def test_fused_dense_forms():
    g = torch.Generator().manual_seed(9)
    L = sim.lib()
    M, K, Nh = 200, 128, 264
    A = torch.randn(M, K, generator=g).to(BF)
    for trans_b in (0, 1):
        B1, B2 = ((torch.randn(Nh, K, generator=g) if trans_b else torch.randn(K, Nh, generator=g)).mul(K ** -0.5).to(BF) for _ in range(2))
        p1, p2, act = (G(torch.empty(M, Nh, dtype=BF)) for _ in range(3))
        assert L.fx_gemm_dual_glu(P(G(A)), K, P(G(B1)), P(G(B2)), B1.stride(0), trans_b, P(p1), P(p2), Nh, P(act), Nh, M, Nh, K, 1, 0, 2,
                                  None) == 0
        op = (lambda b: b.float().t()) if trans_b else (lambda b: b.float())
        _close(p1, (A.float() @ op(B1)).to(BF)), _close(p2, (A.float() @ op(B2)).to(BF))
        from oracle import glu as o_glu
        assert torch.equal(act, o_glu.swiglu_fwd(p1, p2))
    # products that share A, and a sum of products into one output
    Ns = [72, 136]
    Bs = [torch.randn(K, n, generator=g).mul(K ** -0.5).to(BF) for n in Ns]
    Ds = [G(torch.empty(M, n, dtype=BF)) for n in Ns]
    gB = [G(b) for b in Bs]
    arr = lambda vals: (ctypes.c_void_p * len(vals))(*vals)
    i64 = lambda vals: (ctypes.c_int64 * len(vals))(*vals)
    assert L.fx_gemm_segments(P(G(A)), K, 0, 2, arr([P(b) for b in gB]), i64(Ns), 0, None, None, arr([P(d) for d in Ds]), i64(Ns), M,
                              (ctypes.c_int * 2)(*Ns), K, 1.0, 0.0, 2, None) == 0
    for d, b in zip(Ds, Bs):
        _close(d, (A.float() @ b.float()).to(BF))
    Ks = [64, 136]
    As = [torch.randn(M, k, generator=g).to(BF) for k in Ks]
    Ws = [torch.randn(72, k, generator=g).mul(k ** -0.5).to(BF) for k in Ks]       # (N, K): trans_b = 1
    out = G(torch.empty(M, 72, dtype=BF))
    gA, gW = [G(a) for a in As], [G(w) for w in Ws]
    assert L.fx_gemm_ksum(2, arr([P(a) for a in gA]), i64(Ks), 0, arr([P(w) for w in gW]), i64(Ks), 1, (ctypes.c_int * 2)(*Ks), None, 72,
                          P(out), 72, M, 72, 1.0, 0.0, 2, 2, None) == 0
    _close(out, sum(a.float() @ w.float().t() for a, w in zip(As, Ws)).to(BF))


def test_random_routings_and_shapes():
    """Expert counts drawn at random (many zeros, single rows, a few hundred), N and K any multiple of 8:
    rows GEMM and weight gradient on guard-paged buffers against per-expert fp32 products."""
    g = torch.Generator().manual_seed(77)
    r = lambda lo, hi: int(torch.randint(lo, hi + 1, (1,), generator=g))
    L = sim.lib()
    for case in range(16):
        E = r(1, 9)
        counts = torch.tensor([(0, 1, r(2, 40), r(100, 700))[r(0, 3)] for _ in range(E)], dtype=torch.int32)
        if case % 4 == 0:
            counts[r(0, E - 1)] = r(400, 900)                   # one large expert: the 256-row tile form may be picked
        rows = int(counts.sum())
        if rows == 0:
            counts[0] = 5
            rows = 5
        N, K = r(1, 40) * 8, r(1, 30) * 8
        A = torch.randn(rows, K, generator=g).to(BF)
        B = torch.randn(E, N, K, generator=g).to(BF)
        ws, ws_bytes = _ws(E, rows)
        D = G(torch.full((rows, N), 2.0, dtype=BF))
        assert L.fx_grouped_gemm_rows(P(G(A)), K, P(G(B)), K, N * K, 1, None, N, P(D), N, P(G(counts)), E, rows, N, K, 1.0, 0.0, 2, P(ws),
                                      ws_bytes, None) == 0
        ref, off = torch.empty(rows, N), 0
        for e in range(E):
            c = int(counts[e])
            ref[off:off + c] = A[off:off + c].float() @ B[e].float().t()
            off += c
        _close(D, ref.to(BF))
        Bw = torch.randn(rows, N, generator=g).to(BF)
        g0 = torch.randn(E, K, N, generator=g)
        Gd = G(g0)
        assert L.fx_grouped_gemm_wgrad(P(G(A)), K, P(G(Bw)), N, P(Gd), N, K * N, 0, P(G(counts)), E, rows, K, N, 1.0, 1.0, 2, P(ws), ws_bytes,
                                       None, 0, None, 0, None) == 0
        refg, off = g0.clone(), 0
        for e in range(E):
            c = int(counts[e])
            refg[e] += A[off:off + c].float().t() @ Bw[off:off + c].float()
            off += c
        torch.testing.assert_close(Gd, refg, rtol=1e-4, atol=1e-3)
