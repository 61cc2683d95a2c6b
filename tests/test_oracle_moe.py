"""Pins the CPU MoE oracle: brute force, library routines and autograd.  CPU only."""
import itertools

import pytest
import torch

from oracle import moe as o_moe
from util import gen, randn


def test_topk_ids_equal_stable_descending_sort_with_ties():
    g = gen(1)
    # values drawn from a tiny set => many exact ties inside every row
    logits = torch.randint(-3, 4, (200, 16), generator=g).float().to(torch.bfloat16)
    for K in (1, 2, 8, 16):
        w, ids = o_moe.topk_softmax(logits, K)
        order = torch.sort(-logits.float(), dim=1, stable=True).indices[:, :K]
        assert torch.equal(ids.long(), order)
        sel = logits.float().gather(1, order)
        torch.testing.assert_close(w.float(), torch.softmax(sel, -1).to(torch.bfloat16).float(), rtol=0, atol=0)
        torch.testing.assert_close(w.float().sum(-1), torch.ones(200), rtol=0, atol=2e-2)


def test_topk_exhaustive_tiny():
    # every row over {0,1}^4 with K=2: python brute force
    rows = torch.tensor(list(itertools.product([0.0, 1.0], repeat=4)))
    _, ids = o_moe.topk_softmax(rows, 2)
    for r, got in zip(rows.tolist(), ids.tolist()):
        best = sorted(range(4), key=lambda j: (-r[j], j))[:2]
        assert got == best


def test_topk_softmax_then_topk_mode():
    g = gen(2)
    logits = randn(g, 64, 32, dtype=torch.float32)
    w, ids = o_moe.topk_softmax(logits, 4, mode="softmax_then_topk")
    p = torch.softmax(logits, -1)
    tv, ti = torch.topk(p, 4, dim=-1)  # no ties in random fp32 => topk is well defined
    assert torch.equal(ids.long(), ti)
    torch.testing.assert_close(w, tv)
    assert (w.sum(-1) <= 1 + 1e-6).all()


def test_topk_minus_inf_rows_follow_the_iterative_rule():
    # reference rule (moe.py:283-296): once everything left is -inf the smallest
    # index is picked again, so duplicates appear
    logits = torch.tensor([[1.0, float("-inf"), float("-inf")]])
    _, ids = o_moe.topk_softmax(logits, 3)
    assert ids.tolist() == [[0, 0, 0]]


def test_sort_matches_quadratic_rank_count():
    g = gen(3)
    T, K, E = 37, 4, 6
    ids = torch.randint(0, E, (T, K), generator=g, dtype=torch.int32)
    mapping, counts = o_moe.moe_sort(ids, E)
    flat = ids.reshape(-1).tolist()
    starts = [sum(1 for v in flat if v < e) for e in range(E)]
    want = [starts[v] + sum(1 for j in range(i) if flat[j] == v) for i, v in enumerate(flat)]
    assert mapping.reshape(-1).tolist() == want
    assert counts.tolist() == [flat.count(e) for e in range(E)]
    assert sorted(want) == list(range(T * K))
    assert mapping.dtype == torch.int32


def test_scatter_gather_identities():
    g = gen(4)
    T, K, E, D = 50, 4, 8, 32
    ids = torch.randint(0, E, (T, K), generator=g, dtype=torch.int32)
    mapping, counts = o_moe.moe_sort(ids, E)
    x = randn(g, T, D, dtype=torch.float32)
    xs = o_moe.moe_scatter(x, mapping)
    for t in range(0, T, 7):
        for k in range(K):
            assert torch.equal(xs[mapping[t, k]], x[t])
    # rows of expert e are contiguous and carry that expert's tokens
    off = o_moe.expert_offsets(counts)
    owner = torch.empty(T * K, dtype=torch.int32)
    owner[mapping.reshape(-1).long()] = ids.reshape(-1)
    for e in range(E):
        assert (owner[off[e]:off[e + 1]] == e).all()
    w = torch.full((T, K), 1.0 / K)
    torch.testing.assert_close(o_moe.moe_gather(xs, mapping, w), x, rtol=1e-6, atol=1e-6)
    res = randn(g, T, D, dtype=torch.float32)
    torch.testing.assert_close(o_moe.moe_gather(xs, mapping, None, res), res + K * x, rtol=1e-5, atol=1e-5)
    ws = randn(g, T, K, dtype=torch.float32)
    sorted_w = o_moe.moe_scatter_routing_weights(ws, mapping)
    assert torch.equal(sorted_w[mapping.reshape(-1).long()], ws.reshape(-1))
    xsc = o_moe.moe_scatter(x, mapping, ws)
    torch.testing.assert_close(xsc[mapping[:, 1].long()], x * ws[:, 1:2])


def test_swiglu_moe_fwd_bwd_autograd_and_no_w_equals_ones():
    g = gen(5)
    R, F = 33, 48
    x = randn(g, R, 2 * F, dtype=torch.float64).requires_grad_()
    w = (randn(g, R, dtype=torch.float64).abs() + 0.1).requires_grad_()
    d = randn(g, R, F, dtype=torch.float64)
    y = torch.nn.functional.silu(x[:, F:]) * x[:, :F] * w[:, None]
    gx, gw = torch.autograd.grad(y, (x, w), d)
    xf, wf, df = x.detach().float(), w.detach().float(), d.float()
    torch.testing.assert_close(o_moe.swiglu_moe_fwd(xf, wf).double(), y.detach(), rtol=1e-5, atol=1e-6)
    dx, dw, act = o_moe.swiglu_moe_bwd(df, xf, wf)
    torch.testing.assert_close(dx.double(), gx, rtol=1e-4, atol=1e-5)
    torch.testing.assert_close(dw.double(), gw, rtol=1e-4, atol=1e-4)
    torch.testing.assert_close(act.double(), y.detach(), rtol=1e-5, atol=1e-6)
    # prescaled variant: feed dout*w, expect the same dx and dw, unscaled activation
    dx2, dw2, act2 = o_moe.swiglu_moe_bwd(df * wf[:, None], xf, wf, prescaled=True)
    torch.testing.assert_close(dx2, dx, rtol=1e-5, atol=1e-6)
    torch.testing.assert_close(dw2, dw, rtol=1e-4, atol=1e-5)
    torch.testing.assert_close(act2 * wf[:, None], act, rtol=1e-5, atol=1e-6)
    # tests/scratch/test_swiglu_fwd_no_w.py:28-33: w=None == w=ones
    assert torch.equal(o_moe.swiglu_moe_fwd(xf), o_moe.swiglu_moe_fwd(xf, torch.ones(R)))


@pytest.mark.parametrize("mode", ["topk_then_softmax", "softmax_then_topk"])
def test_router_gate_bwd_matches_autograd(mode):
    g = gen(6)
    T, E, K = 20, 12, 3
    logits = randn(g, T, E, dtype=torch.float32).requires_grad_()
    w, ids = o_moe.topk_softmax(logits.detach(), K, mode=mode)
    ce = ids.long()
    if mode == "topk_then_softmax":
        p = torch.softmax(logits.gather(1, ce), -1)
    else:
        p = torch.softmax(logits, -1).gather(1, ce)
    torch.testing.assert_close(p.detach(), w, rtol=1e-5, atol=1e-6)
    mapping, _ = o_moe.moe_sort(ids, E)
    dprobs_sorted = randn(g, T * K, dtype=torch.float32)     # lives in expert-grouped order
    dp = dprobs_sorted[mapping.reshape(-1).long()].reshape(T, K)
    (want,) = torch.autograd.grad(p, logits, dp)
    got = o_moe.router_gate_bwd(w, dprobs_sorted, mapping, ids, E, mode=mode, logits=logits.detach())
    torch.testing.assert_close(got, want, rtol=1e-4, atol=1e-6)
    base = randn(g, T, E, dtype=torch.float32)
    got2 = o_moe.router_gate_bwd(w, dprobs_sorted, mapping, ids, E, dlogits=base, mode=mode, logits=logits.detach())
    torch.testing.assert_close(got2, base + want, rtol=1e-4, atol=1e-6)


def test_load_balance_bwd_matches_autograd():
    g = gen(7)
    T, E, K, alpha = 40, 8, 2, 0.01
    logits = randn(g, T, E, dtype=torch.float64).requires_grad_()
    counts = torch.randint(0, 20, (E,), generator=g, dtype=torch.int32)
    f = counts.double() / (T * K)
    loss = alpha * E * (f * torch.softmax(logits, -1).mean(0)).sum()   # f is a constant
    (want,) = torch.autograd.grad(loss, logits)
    got = o_moe.load_balance_bwd(logits.detach().float(), counts, K, alpha)
    torch.testing.assert_close(got.double(), want, rtol=1e-4, atol=1e-8)
    got_half = o_moe.load_balance_bwd(logits.detach().float(), counts, K, alpha, tokens_per_step=2 * T)
    torch.testing.assert_close(got_half, got / 2, rtol=1e-5, atol=1e-9)


def test_grouped_expert_block_matches_eager_autograd():
    """tests/moe/test_moe_backend_parity.py:45-107 restated: per-expert eager MLP +
    index_add_ + autograd, compared token-major on out, dx, d_expert_p, g_up, g_down."""
    g = gen(8)
    T, K, E, F, d = 64, 2, 8, 16, 32
    x = randn(g, T, d, dtype=torch.float32).requires_grad_()
    w_up = randn(g, E, 2 * F, d, dtype=torch.float32, std=0.1).requires_grad_()
    w_down = randn(g, E, d, F, dtype=torch.float32, std=0.1).requires_grad_()
    probs = torch.softmax(randn(g, T, K, dtype=torch.float32), -1).requires_grad_()
    ids = torch.stack([torch.randperm(E, generator=g)[:K] for _ in range(T)]).to(torch.int32)
    dy = randn(g, T, d, dtype=torch.float32)
    out = torch.zeros(T, d)
    for e in range(E):
        tok, slot = (ids == e).nonzero(as_tuple=True)
        if tok.numel() == 0:
            continue
        pre = x[tok] @ w_up[e].t()
        act = torch.nn.functional.silu(pre[:, F:]) * pre[:, :F]
        out = out.index_add(0, tok, (act @ w_down[e].t()) * probs[tok, slot][:, None])
    gx, gp, gu, gd = torch.autograd.grad(out, (x, probs, w_up, w_down), dy)

    mapping, counts = o_moe.moe_sort(ids, E)
    xd, wu, wd, pr = x.detach(), w_up.detach(), w_down.detach(), probs.detach()
    xg = o_moe.moe_scatter(xd, mapping)
    pre, act, y = o_moe.grouped_expert_fwd(xg, counts, wu, wd)
    torch.testing.assert_close(o_moe.moe_gather(y, mapping, pr), out.detach(), rtol=1e-4, atol=1e-5)
    dyg = o_moe.moe_scatter(dy, mapping)
    wsorted = o_moe.moe_scatter_routing_weights(pr, mapping)
    dxg, dprobs, g_up, g_down = o_moe.grouped_expert_bwd(dyg, xg, pre, wsorted, counts, wu, wd)
    torch.testing.assert_close(o_moe.moe_gather(dxg, mapping), gx, rtol=1e-4, atol=1e-5)
    torch.testing.assert_close(dprobs[mapping.reshape(-1).long()].reshape(T, K), gp, rtol=1e-4, atol=1e-5)
    torch.testing.assert_close(g_up, gu, rtol=1e-4, atol=1e-5)
    torch.testing.assert_close(g_down, gd, rtol=1e-4, atol=1e-5)


# ------------------------------------------------------------------ whole block
def _eager_block(x, w_router, w_up, w_down, residual, dy, ids, mode, lb_coef, tokens_per_step, counts, keep=None):
    """The routed block as one differentiable fp64 expression with the selection held
    constant (tests/moe/test_moe_backend_parity.py:45-107 for the experts, the router
    path of flextrain/ops/full_moe.py:306-349 around it): autograd gives every gradient."""
    T, d = x.shape
    E, F2, _ = w_up.shape
    K = ids.shape[1]
    x = x.double().requires_grad_()
    w_router = w_router.double().requires_grad_()
    w_up = w_up.double().requires_grad_()
    w_down = w_down.double().requires_grad_()
    logits = x @ w_router
    ce = ids.long()
    if mode == "topk_then_softmax":
        p = torch.softmax(logits.gather(1, ce), -1)
    else:
        p = torch.softmax(logits, -1).gather(1, ce)
    out = residual.double().clone()
    for t in range(T):
        for k in range(K):
            e = int(ce[t, k])
            if keep is not None and e not in keep:
                continue
            pre = w_up[e] @ x[t]
            h = torch.nn.functional.silu(pre[F2 // 2:]) * pre[:F2 // 2]
            out = out + torch.nn.functional.one_hot(torch.tensor(t), T).double()[:, None] * (p[t, k] * (w_down[e] @ h))
    loss = (out * dy.double()).sum()
    if lb_coef > 0.0 and tokens_per_step is not None:
        f = counts.double() / (T * K)                                  # a constant of the step
        loss = loss + lb_coef * E * (f * torch.softmax(logits, -1).sum(0)).sum() / tokens_per_step
    dx, g_router, g_up, g_down = torch.autograd.grad(loss, (x, w_router, w_up, w_down))
    return out.detach(), dx, g_router, g_up, g_down


def _block_case(seed, T=24, d=16, E=6, F=10, K=3):
    g = gen(seed)
    x = randn(g, T, d, dtype=torch.float32)
    w_router = randn(g, d, E, dtype=torch.float32) * 0.5
    w_up = randn(g, E, 2 * F, d, dtype=torch.float32) * 0.3
    w_down = randn(g, E, d, F, dtype=torch.float32) * 0.3
    residual = randn(g, T, d, dtype=torch.float32)
    dy = randn(g, T, d, dtype=torch.float32)
    logits = (x.double() @ w_router.double()).float()
    return x, w_router, w_up, w_down, residual, dy, logits, K


@pytest.mark.parametrize("mode", ["topk_then_softmax", "softmax_then_topk"])
@pytest.mark.parametrize("lb", [0.0, 0.05])
def test_routed_block_matches_autograd_of_the_eager_block(mode, lb):
    x, w_router, w_up, w_down, residual, dy, logits, K = _block_case(11)
    T = x.shape[0]
    tps = 2 * T if lb else None
    got = o_moe.routed_block_fwd_bwd(x, logits, w_router, w_up, w_down, residual, dy, K, mode=mode,
                                     load_balance_coef=lb, tokens_per_step=tps)
    out, dx, g_router, g_up, g_down = _eager_block(x, w_router, w_up, w_down, residual, dy, got["ids"], mode, lb,
                                                   tps, got["counts"])
    torch.testing.assert_close(got["out"].double(), out, rtol=1e-4, atol=1e-5)
    torch.testing.assert_close(got["dx"].double(), dx, rtol=1e-4, atol=1e-5)
    torch.testing.assert_close(got["g_router"].double(), g_router, rtol=1e-4, atol=1e-5)
    torch.testing.assert_close(got["g_up"].double(), g_up, rtol=1e-4, atol=1e-5)
    torch.testing.assert_close(got["g_down"].double(), g_down, rtol=1e-4, atol=1e-5)
    # the load-balance term must actually move the router path when it is on
    if lb:
        off = o_moe.routed_block_fwd_bwd(x, logits, w_router, w_up, w_down, residual, dy, K, mode=mode)
        assert (off["g_router"] - got["g_router"]).abs().max() > 1e-5
        torch.testing.assert_close(off["g_up"], got["g_up"], rtol=0, atol=0)


def test_routed_block_load_balance_needs_both_arguments():
    # full_moe.py:327: the aux gradient is added only when the coefficient is positive AND a step size is given
    x, w_router, w_up, w_down, residual, dy, logits, K = _block_case(12)
    a = o_moe.routed_block_fwd_bwd(x, logits, w_router, w_up, w_down, residual, dy, K)
    b = o_moe.routed_block_fwd_bwd(x, logits, w_router, w_up, w_down, residual, dy, K, load_balance_coef=0.05)
    assert torch.equal(a["dx"], b["dx"]) and torch.equal(a["g_router"], b["g_router"])


def test_routed_block_expert_subset_is_the_block_with_the_other_experts_removed():
    x, w_router, w_up, w_down, residual, dy, logits, K = _block_case(13)
    keep = (1, 4)
    full = o_moe.routed_block_fwd_bwd(x, logits, w_router, w_up, w_down, residual, dy, K)
    sub = o_moe.routed_block_fwd_bwd(x, logits, w_router, w_up, w_down, residual, dy, K, experts=keep)
    assert torch.equal(sub["ids"], full["ids"]) and torch.equal(sub["mapping"], full["mapping"])
    assert torch.equal(sub["counts"], full["counts"])
    assert full["counts"][list(keep)].min() > 0
    for e in range(w_up.shape[0]):
        if e in keep:
            assert torch.equal(sub["g_up"][e], full["g_up"][e]) and torch.equal(sub["g_down"][e], full["g_down"][e])
            assert sub["g_up"][e].abs().max() > 0
        else:
            assert not sub["g_up"][e].any() and not sub["g_down"][e].any()
    off = o_moe.expert_offsets(full["counts"])
    for e in range(w_up.shape[0]):
        rows = slice(int(off[e]), int(off[e + 1]))
        if e in keep:
            assert torch.equal(sub["pre"][rows], full["pre"][rows])
        else:
            assert not sub["pre"][rows].any()
    # and as a whole it is the differentiable block with only those experts present
    out, dx, g_router, g_up, g_down = _eager_block(x, w_router, w_up, w_down, residual, dy, full["ids"],
                                                   "topk_then_softmax", 0.0, None, full["counts"], keep=keep)
    torch.testing.assert_close(sub["out"].double(), out, rtol=1e-4, atol=1e-5)
    torch.testing.assert_close(sub["dx"].double(), dx, rtol=1e-4, atol=1e-5)
    torch.testing.assert_close(sub["g_router"].double(), g_router, rtol=1e-4, atol=1e-5)
    torch.testing.assert_close(sub["g_up"].double(), g_up, rtol=1e-4, atol=1e-5)


def test_routed_block_rounding_points_in_bf16():
    # bf16 inputs: out / dx stay within bf16 tolerance of the fp64 block built from the same bf16 values
    x, w_router, w_up, w_down, residual, dy, _, K = _block_case(14)
    bf = lambda t: t.to(torch.bfloat16)
    xb, wrb, wub, wdb, rb, dyb = map(bf, (x, w_router, w_up, w_down, residual, dy))
    logits = (xb.double() @ wrb.double()).to(torch.bfloat16)
    got = o_moe.routed_block_fwd_bwd(xb, logits, wrb, wub, wdb, rb, dyb, K)
    assert got["out"].dtype == torch.bfloat16 and got["dx"].dtype == torch.bfloat16
    out, dx, g_router, g_up, g_down = _eager_block(xb.float(), wrb.float(), wub.float(), wdb.float(), rb.float(),
                                                   dyb.float(), got["ids"], "topk_then_softmax", 0.0, None,
                                                   got["counts"])
    torch.testing.assert_close(got["out"].double(), out, rtol=2e-2, atol=3e-2)
    torch.testing.assert_close(got["dx"].double(), dx, rtol=2e-2, atol=3e-2)
    torch.testing.assert_close(got["g_up"].double(), g_up, rtol=2e-2, atol=3e-2)
    torch.testing.assert_close(got["g_down"].double(), g_down, rtol=2e-2, atol=3e-2)
    torch.testing.assert_close(got["g_router"].double(), g_router, rtol=3e-2, atol=5e-2)


def test_routed_block_tokens_are_independent():
    # out[t] and dx[t] depend on token t alone (no load-balance term): the block on a subset of the
    # tokens gives exactly the rows of the block on all of them.  The full-size GPU test samples tokens this way.
    x, w_router, w_up, w_down, residual, dy, logits, K = _block_case(15, T=40)
    full = o_moe.routed_block_fwd_bwd(x, logits, w_router, w_up, w_down, residual, dy, K)
    tok = torch.tensor([3, 0, 39, 17, 18])
    sub = o_moe.routed_block_fwd_bwd(x[tok], logits[tok], w_router, w_up, w_down, residual[tok], dy[tok], K)
    assert torch.equal(sub["ids"], full["ids"][tok])
    torch.testing.assert_close(sub["out"], full["out"][tok], rtol=1e-6, atol=1e-6)
    torch.testing.assert_close(sub["dx"], full["dx"][tok], rtol=1e-6, atol=1e-6)
