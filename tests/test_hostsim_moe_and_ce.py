"""MoE routing / permutation / expert activation kernels and the softmax / cross-entropy family: the
kernels' own source run on the CPU by the host simulation (tests/hostsim) on guard-paged buffers, against
the oracle.  Integer results (ids, mappings, counts, argmax) must be equal, floating-point ones within the
package's tolerances."""
from __future__ import annotations

import pytest
import torch

from oracle import linear_ce as o_ce
from oracle import moe as o_moe
from tests.hostsim import sim

from tests.hostsim.build import needs_host_clang

pytestmark = needs_host_clang

BF, F32 = torch.bfloat16, torch.float32
G = sim.guard
P = sim.p


def _close(a, e, tol=1e-2):
    torch.testing.assert_close(a.float(), e.float(), rtol=tol, atol=tol)


# ------------------------------------------------------------------ routing
@pytest.mark.parametrize("T,E,K", [(7, 8, 2), (33, 128, 8), (5, 256, 8), (9, 60, 4), (4, 512, 8), (3, 4, 4), (6, 1000, 6)])
@pytest.mark.parametrize("mode", [0, 1])
def test_topk_softmax(T, E, K, mode):
    g = torch.Generator().manual_seed(T * E + mode)
    logits = torch.randn(T, E, generator=g).to(BF)
    logits[0, : min(E, 5)] = logits[0, 0]                       # ties: the smallest index wins
    ids, w = G(torch.empty(T, K, dtype=torch.int32)), G(torch.empty(T, K, dtype=BF))
    assert sim.lib().fx_topk_softmax(P(G(logits)), P(ids), P(w), T, E, K, 2, 2, mode, None) == 0
    w_ref, ids_ref = o_moe.topk_softmax(logits, K, mode=("topk_then_softmax", "softmax_then_topk")[mode])
    assert torch.equal(ids, ids_ref)
    _close(w, w_ref)


@pytest.mark.parametrize("T,K,E,idt", [(100, 4, 16, torch.int32), (1, 1, 4, torch.int32), (700, 8, 128, torch.int64),
                                       (64, 2, 300, torch.int32), (257, 1, 8, torch.int32)])
def test_sort(T, K, E, idt):
    g = torch.Generator().manual_seed(T + E)
    ids = torch.randint(0, E, (T, K), generator=g).to(idt)
    if E >= 8:
        ids[ids == 3] = 4                                       # an expert without rows
    L = sim.lib()
    n = T * K
    ws_bytes = int(L.fx_moe_sort_ws_bytes(n, E))
    mapping, counts, host = G(torch.empty(T, K, dtype=idt)), G(torch.empty(E, dtype=torch.int32)), G(torch.empty(E, dtype=torch.int32))
    ws = G(torch.empty(ws_bytes // 4, dtype=torch.int32))
    i64 = int(idt == torch.int64)
    assert L.fx_moe_sort(P(G(ids)), i64, n, E, P(mapping), i64, P(counts), P(host), P(ws), ws_bytes, None) == 0
    map_ref, cnt_ref = o_moe.moe_sort(ids, E)
    assert torch.equal(mapping, map_ref) and torch.equal(counts, cnt_ref) and torch.equal(host, cnt_ref)
    m2, c2 = G(torch.empty(T, K, dtype=idt)), G(torch.empty(E, dtype=torch.int32))
    assert L.fx_moe_sort_noalloc(P(G(ids)), i64, n, E, P(m2), i64, P(c2), None, None) == 0
    assert torch.equal(m2, map_ref) and torch.equal(c2, cnt_ref)
    src = G(torch.empty(n, dtype=torch.int32))
    assert L.fx_moe_row_sources(P(mapping), i64, T, K, P(src), None) == 0
    want = torch.empty(n, dtype=torch.int32)
    want[map_ref.reshape(-1).long()] = torch.arange(n, dtype=torch.int32) // K
    assert torch.equal(src, want)
    dst = G(torch.empty(E, dtype=torch.int32))
    assert L.fx_copy_i32(P(counts), P(dst), E, None) == 0 and torch.equal(dst, cnt_ref)


def test_sort_with_ids_outside_the_expert_range():
    g = torch.Generator().manual_seed(11)
    T, K, E = 300, 2, 8
    ids = torch.randint(0, E, (T, K), generator=g, dtype=torch.int32)
    bad = torch.rand(T, K, generator=g) < 0.1
    ids[bad] = torch.where(torch.rand(int(bad.sum()), generator=g) < 0.5, -3, E + 5).to(torch.int32)
    L = sim.lib()
    ws_bytes = int(L.fx_moe_sort_ws_bytes(T * K, E))
    mapping = G(torch.full((T, K), 1 << 30, dtype=torch.int32))
    counts, ws = G(torch.empty(E, dtype=torch.int32)), G(torch.empty(ws_bytes // 4, dtype=torch.int32))
    assert L.fx_moe_sort(P(G(ids)), 0, T * K, E, P(mapping), 0, P(counts), None, P(ws), ws_bytes, None) == 0
    flat, ok = ids.reshape(-1), ~bad.reshape(-1)
    assert torch.equal(counts, torch.bincount(flat[ok].long(), minlength=E).to(torch.int32))
    m = mapping.reshape(-1).long()
    assert bool((m[~ok] == 0).all())
    order = torch.argsort(flat[ok].long(), stable=True)
    want = torch.empty_like(order)
    want[order] = torch.arange(order.numel())
    assert torch.equal(m[ok], want)


@pytest.mark.parametrize("T,K,E", [(50, 2, 8), (9, 8, 128), (130, 4, 60)])
@pytest.mark.parametrize("mode", [0, 1])
def test_router_backward(T, K, E, mode):
    g = torch.Generator().manual_seed(T + K + mode)
    logits = torch.randn(T, E, generator=g).to(BF)
    probs, chosen = o_moe.topk_softmax(logits, K, mode=("topk_then_softmax", "softmax_then_topk")[mode])
    mapping, counts = o_moe.moe_sort(chosen, E)
    dprobs = torch.randn(T * K, generator=g).to(BF)
    base = torch.randn(T, E, generator=g).to(BF)
    dl = G(base)
    L = sim.lib()
    assert L.fx_router_gate_bwd(P(dl), P(G(dprobs)), P(G(probs)), P(G(mapping)), 0, P(G(chosen)), P(G(logits)) if mode else None, T, K, E,
                                2, 2, mode, None) == 0
    ref = o_moe.router_gate_bwd(probs, dprobs, mapping, chosen, E, dlogits=base,
                                mode=("topk_then_softmax", "softmax_then_topk")[mode], logits=logits)
    _close(dl, ref, 2e-2)
    lb = G(base)
    scale = 0.01 * E / T
    assert L.fx_load_balance_bwd(P(G(logits)), P(G(counts)), P(lb), T, E, K, scale, 2, 2, None) == 0
    _close(lb, o_moe.load_balance_bwd(logits, counts, K, dlogits=base))


# ------------------------------------------------------------------ data movement and expert activation
@pytest.mark.parametrize("T,K,E,D", [(100, 2, 8, 128), (37, 4, 6, 100), (5, 3, 4, 8), (64, 8, 128, 2048), (9, 1, 2, 24)])
def test_scatter_gather(T, K, E, D):
    g = torch.Generator().manual_seed(T + D)
    ids = torch.stack([torch.randperm(E, generator=g)[:K] for _ in range(T)]).to(torch.int32)
    mapping, _ = o_moe.moe_sort(ids, E)
    x = torch.randn(T, D, generator=g).to(BF)
    w = torch.softmax(torch.randn(T, K, generator=g), -1).to(BF)
    res = torch.randn(T, D, generator=g).to(BF)
    L = sim.lib()
    xs = G(torch.empty(T * K, D, dtype=BF))
    assert L.fx_moe_scatter(P(G(x)), P(G(mapping)), 0, None, 0, P(xs), T, D, K, D, 2, None) == 0
    assert torch.equal(xs, o_moe.moe_scatter(x, mapping))
    xw = G(torch.empty(T * K, D, dtype=BF))
    assert L.fx_moe_scatter(P(G(x)), P(G(mapping.long())), 1, P(G(w)), 2, P(xw), T, D, K, D, 2, None) == 0
    _close(xw, o_moe.moe_scatter(x, mapping, scales=w))
    sw = G(torch.empty(T * K, dtype=BF))
    assert L.fx_moe_scatter_weights(P(G(w)), P(G(mapping)), 0, P(sw), T * K, 2, None) == 0
    assert torch.equal(sw, o_moe.moe_scatter_routing_weights(w, mapping))
    y = torch.randn(T * K, D, generator=g).to(BF)
    for weights, residual in ((None, None), (w, None), (w, res), (None, res)):
        out = G(torch.empty(T, D, dtype=BF))
        assert L.fx_moe_gather(P(G(y)), P(G(mapping)), 0, P(G(weights)) if weights is not None else None, 2,
                               P(G(residual)) if residual is not None else None, 2, P(out), 2, T, D, K, 2, None) == 0
        _close(out, o_moe.moe_gather(y, mapping, weights=weights, residual=residual), 2e-2)
    # a mapping that leaves the buffer reads the clamped rows
    bad = mapping.clone()
    bad[0, 0], bad[T - 1, K - 1] = 1 << 28, -9
    a, b = G(torch.empty(T, D, dtype=BF)), G(torch.empty(T, D, dtype=BF))
    assert L.fx_moe_gather(P(G(y)), P(G(bad)), 0, None, 0, None, 0, P(a), 2, T, D, K, 2, None) == 0
    assert L.fx_moe_gather(P(G(y)), P(G(bad.clamp(0, T * K - 1))), 0, None, 0, None, 0, P(b), 2, T, D, K, 2, None) == 0
    assert torch.equal(a, b)


@pytest.mark.parametrize("rows,F", [(5, 64), (130, 768), (3, 100), (64, 8), (7, 1032)])
def test_expert_activation(rows, F):
    g = torch.Generator().manual_seed(rows + F)
    x = torch.randn(rows, 2 * F, generator=g).to(BF)
    w = torch.rand(rows, generator=g).to(BF)
    d = torch.randn(rows, F, generator=g).to(BF)
    L = sim.lib()
    for weights in (None, w):
        out = G(torch.empty(rows, F, dtype=BF))
        assert L.fx_swiglu_moe_fwd(P(G(x)), P(G(weights)) if weights is not None else None, 2, P(out), 2, rows, F, 2 * F, F, 2, None) == 0
        _close(out, o_moe.swiglu_moe_fwd(x, weights))
    for prescaled in (0, 1):
        dx, dw, act = G(torch.empty(rows, 2 * F, dtype=BF)), G(torch.empty(rows, dtype=F32)), G(torch.empty(rows, F, dtype=BF))
        assert L.fx_swiglu_moe_bwd(P(dx), P(dw), 0, P(G(d)), P(G(x)), P(G(w)), 2, P(act), rows, F, 2 * F, F, 2 * F, F, 2, prescaled,
                                   None) == 0
        rdx, rdw, ract = o_moe.swiglu_moe_bwd(d, x, w, prescaled=bool(prescaled))
        _close(dx, rdx, 2e-2), _close(act, ract)
        torch.testing.assert_close(dw, rdw, rtol=2e-2, atol=2e-2 * F ** 0.5)


# ------------------------------------------------------------------ softmax / cross-entropy / soft cap
@pytest.mark.parametrize("rows,V", [(3, 8), (5, 1000), (4, 1024), (2, 4104), (3, 12345), (2, 128256)])
def test_softmax_and_cross_entropy(rows, V):
    g = torch.Generator().manual_seed(V)
    x = (torch.randn(rows, V, generator=g) * 3).to(BF)
    labels = torch.randint(0, V, (rows,), generator=g)
    labels[0] = -100
    L = sim.lib()
    probs, idx, val = G(torch.empty(rows, V, dtype=BF)), G(torch.empty(rows, dtype=torch.int64)), G(torch.empty(rows, dtype=F32))
    assert L.fx_softmax(P(G(x)), P(probs), P(idx), P(val), rows, V, V, V, 1.0, 2, 2, None) == 0
    p_ref, first, mx = o_ce.softmax(x)
    _close(probs, p_ref, 1e-2)
    assert torch.equal(idx, first)
    torch.testing.assert_close(val, mx, rtol=1e-4, atol=1e-6)
    loss, valid = G(torch.empty(rows, dtype=F32)), G(torch.empty(rows, dtype=F32))
    dz = G(p_ref)
    assert L.fx_cross_entropy(P(dz), P(G(labels)), 1, P(loss), P(valid), rows, V, V, 1, 100.0, 2, None) == 0
    dz_ref, loss_ref, valid_ref = o_ce.cross_entropy_from_probs(p_ref, labels)
    assert torch.equal(dz, dz_ref) and torch.equal(valid, valid_ref)
    torch.testing.assert_close(loss, loss_ref, rtol=1e-5, atol=1e-6)


@pytest.mark.parametrize("rows,V", [(3, 8), (5, 1000), (4, 1024), (2, 4104), (3, 12347), (2, 128256)])
@pytest.mark.parametrize("cap", [0.0, 30.0])
def test_fused_softmax_cross_entropy(rows, V, cap):
    g = torch.Generator().manual_seed(V + int(cap))
    x = (torch.randn(rows, V, generator=g) * 4).to(BF)
    labels = torch.randint(0, V, (rows,), generator=g)
    labels[0] = -100
    mask = torch.ones(rows, dtype=torch.uint8)
    mask[-1] = 0
    L = sim.lib()
    dz, loss = G(torch.empty(rows, V, dtype=BF)), G(torch.empty(rows, dtype=F32))
    idx, val = G(torch.empty(rows, dtype=torch.int64)), G(torch.empty(rows, dtype=F32))
    assert L.fx_softmax_ce(P(G(x)), P(dz), P(G(labels)), 1, P(G(mask)), P(loss), P(idx), P(val), rows, V, V, V, -100, 100.0, cap, 2,
                           None) == 0
    dz_ref, loss_ref, first, mx = o_ce.softmax_ce(x, labels, loss_mask=mask, logit_softcap=cap or None)
    _close(dz, dz_ref, 1e-2)
    torch.testing.assert_close(loss, loss_ref, rtol=1e-4, atol=1e-4)
    assert torch.equal(idx, first)
    torch.testing.assert_close(val, mx, rtol=1e-3, atol=1e-6)
    inplace = G(x)
    assert L.fx_softmax_ce(P(inplace), P(inplace), P(G(labels.to(torch.int32))), 0, P(G(mask)), P(loss), None, None, rows, V, V, V, -100,
                           100.0, cap, 2, None) == 0
    assert torch.equal(inplace, dz)
    if cap:
        y, gate = G(x), G(torch.empty(rows, V, dtype=BF))
        assert L.fx_softcap_fwd(P(y), P(gate), rows, V, V, V, cap, 2, None) == 0
        y_ref, gate_ref = o_ce.softcap(x, cap)
        _close(y, y_ref), _close(gate, gate_ref)
        d = G(dz_ref)
        assert L.fx_softcap_bwd(P(d), P(gate), rows, V, V, V, 2, None) == 0
        _close(d, (dz_ref.float() * gate.float()).to(BF))
