"""HIP MoE routing / permutation / activation kernels against the CPU oracle.
Expert ids, index mapping and counts: torch.equal.  Copies (scatter): bit-exact.
bf16 floating point: rtol = atol = 1e-2."""
import pytest
import torch

from flextrain_amd.ops import moe as ops
from oracle import moe as o_moe
from util import close, gen, randn

pytestmark = pytest.mark.gpu


# ------------------------------------------------------------------ top-k
@pytest.mark.parametrize("T,E,K", [(8192, 128, 8), (1000, 256, 8), (77, 64, 2), (50, 8, 8), (33, 12, 3),
                                   (9, 512, 4), (5, 1000, 6), (1, 4, 1)])
@pytest.mark.parametrize("mode", ["topk_then_softmax", "softmax_then_topk"])
def test_topk_ids_bit_exact(dev, T, E, K, mode):
    g = gen(1004)
    logits = randn(g, T, E, std=0.5)          # bf16 logits: plenty of exact ties at E >= 128
    w_ref, ids_ref = o_moe.topk_softmax(logits, K, mode=mode)
    w, ids = ops.flextrain_fused_topk_softmax(logits.to(dev), K, mode=mode)
    assert ids.dtype == torch.int32 and w.dtype == torch.bfloat16
    if mode == "topk_then_softmax":
        assert torch.equal(ids.cpu(), ids_ref)
    else:
        # Selection happens on fp32 probabilities.  softmax is monotone in the logit, so wherever two
        # logits differ the larger must be picked first UNLESS their fp32 probabilities round to the
        # same value, in which case the lower index wins -- and whether they do depends on the last
        # bit of exp / sum / divide, which no two implementations share.  So: (1) on every row whose
        # ordering does not hinge on that bit (the first K+1 distinct logit values of the row are
        # each separated by more than 4 ulp of probability in fp64) the ids must be bit-equal to the
        # oracle's; (2) on the other rows the pick must still be a valid one: distinct ids whose
        # logits equal the oracle's picks' logits up to that rounding, position by position.
        got = ids.cpu().long()
        p64 = torch.softmax(logits.double(), -1)
        srt = torch.sort(p64, dim=1, descending=True).values[:, :min(K + 1, E)]
        gaps = srt[:, :-1] - srt[:, 1:]
        ulp4 = 4 * srt[:, :-1] * 2.0 ** -23
        tied = gaps == 0                                   # equal logits: index order decides, exactly
        decided = ((gaps > ulp4) | tied).all(dim=1)
        assert torch.equal(got[decided], ids_ref.long()[decided])
        assert float(decided.float().mean()) > 0.5
        assert (torch.sort(got, dim=1).values.diff(dim=1) != 0).all() or E < K + 1      # distinct experts
        pg, pr = p64.gather(1, got), p64.gather(1, ids_ref.long())
        torch.testing.assert_close(pg, pr, rtol=2e-6, atol=0)
    close(w, w_ref, what="weights")


def test_topk_ties_and_minus_inf(dev):
    g = gen(5)
    logits = torch.randint(-2, 3, (512, 128), generator=g).float().to(torch.bfloat16)
    logits[::7, 5:] = float("-inf")           # fewer finite experts than K on some rows
    w_ref, ids_ref = o_moe.topk_softmax(logits, 8)
    w, ids = ops.flextrain_fused_topk_softmax(logits.to(dev), 8)
    assert torch.equal(ids.cpu(), ids_ref)
    fp32 = logits.float()
    w2, ids2 = ops.flextrain_fused_topk_softmax(fp32.to(dev), 8)
    assert torch.equal(ids2.cpu(), ids_ref) and w2.dtype == torch.float32


def test_topk_out_buffers_and_errors(dev):
    logits = torch.zeros(4, 8, device=dev, dtype=torch.bfloat16)
    ids = torch.empty(4, 2, dtype=torch.int32, device=dev)
    w = torch.empty(4, 2, dtype=torch.float32, device=dev)
    rw, ri = ops.flextrain_fused_topk_softmax(logits, 2, ids, w)
    assert rw is w and ri is ids
    assert ids.cpu().tolist() == [[0, 1]] * 4 and torch.equal(w.cpu(), torch.full((4, 2), 0.5))
    with pytest.raises(ValueError):
        ops.flextrain_fused_topk_softmax(logits, 9)
    with pytest.raises(ValueError):
        ops.flextrain_fused_topk_softmax(logits.t(), 2)
    with pytest.raises(ValueError):
        ops.flextrain_fused_topk_softmax(logits, 2, mode="nope")


# ------------------------------------------------------------------- sort
@pytest.mark.parametrize("T,K,E", [(8192, 8, 128), (131072, 8, 128), (1000, 2, 8), (257, 1, 3), (1, 8, 128),
                                   (300, 8, 256)])
@pytest.mark.parametrize("idt", [torch.int32, torch.int64])
def test_sort_bit_exact(dev, T, K, E, idt):
    g = gen(1005)
    ids = torch.randint(0, E, (T, K), generator=g).to(idt)
    if E >= 8:
        ids[ids == 3] = 4                      # an expert with zero rows
    map_ref, cnt_ref = o_moe.moe_sort(ids, E)
    pinned = torch.zeros(E, dtype=torch.int32).pin_memory()
    mapping, counts = ops.flextrain_moe_sort(ids.to(dev), E, expert_counts_pinned=pinned)
    assert mapping.dtype == idt and mapping.shape == ids.shape
    assert torch.equal(mapping.cpu(), map_ref)
    assert torch.equal(counts.cpu(), cnt_ref)
    torch.cuda.synchronize()
    assert torch.equal(pinned, cnt_ref)
    # size-independent: a permutation of 0..TK-1
    assert torch.equal(torch.sort(mapping.reshape(-1).cpu().long()).values, torch.arange(T * K))


def test_sort_maps_ids_outside_the_expert_range_to_row_zero(dev):
    """A caller error the reference leaves undefined: such a pair is not counted, and its map entry is 0 (inside
    every buffer) instead of whatever the output held; the valid pairs keep the stable order among themselves."""
    g = gen(1011)
    T, K, E = 512, 4, 16
    ids = torch.randint(0, E, (T, K), generator=g, dtype=torch.int32)
    bad = torch.rand(T, K, generator=g) < 0.05
    ids[bad] = torch.where(torch.rand(int(bad.sum()), generator=g) < 0.5, -3, E + 5).to(torch.int32)
    out = torch.full((T, K), 1 << 30, dtype=torch.int32, device=dev)
    mapping, counts = ops.flextrain_moe_sort(ids.to(dev), E, indices=out)
    flat, ok = ids.reshape(-1), ~bad.reshape(-1)
    cnt_ref = torch.bincount(flat[ok].long(), minlength=E).to(torch.int32)
    assert torch.equal(counts.cpu(), cnt_ref)
    m = mapping.reshape(-1).cpu().long()
    assert bool((m[~ok] == 0).all())
    order = torch.argsort(flat[ok].long(), stable=True)          # valid pairs, grouped by expert, first come first
    want = torch.empty_like(order)
    want[order] = torch.arange(order.numel())
    assert torch.equal(m[ok], want)


def test_gather_clamps_a_mapping_that_leaves_the_buffer(dev):
    """A caller's own mapping with entries outside the routed rows reads the clamped rows, never past the buffer."""
    g = gen(1012)
    T, K, D = 64, 2, 64
    y = randn(g, T * K, D).to(dev)
    mapping = torch.randperm(T * K, generator=g).view(T, K).to(torch.int32)
    bad = mapping.clone()
    bad[3, 1], bad[10, 0], bad[63, 1] = 1 << 28, -7, T * K
    clamped = bad.clamp(0, T * K - 1)
    assert torch.equal(ops.flextrain_moe_gather(y, bad.to(dev)), ops.flextrain_moe_gather(y, clamped.to(dev)))
    assert torch.equal(ops.flextrain_moe_gather(y, bad.long().to(dev)), ops.flextrain_moe_gather(y, clamped.to(dev)))


def test_sort_slot_buffers_and_copy_counts(dev):
    g = gen(6)
    ids = torch.randint(0, 16, (100, 4), generator=g, dtype=torch.int32)
    idx = torch.empty(100, 4, dtype=torch.int32, device=dev)
    cnt = torch.empty(16, dtype=torch.int32, device=dev)
    m, c = ops.flextrain_moe_sort(ids.to(dev), 16, indices=idx, expert_counts_gpu=cnt)
    assert m is idx and torch.equal(cnt, c)
    host = torch.zeros(16, dtype=torch.int32).pin_memory()
    ops.flextrain_copy_expert_counts(cnt, host)
    torch.cuda.current_stream().synchronize()
    assert torch.equal(host, o_moe.moe_sort(ids, 16)[1])
    with pytest.raises(ValueError):
        ops.flextrain_copy_expert_counts(cnt, torch.zeros(16, dtype=torch.int32))


# -------------------------------------------------------- scatter / gather
@pytest.mark.parametrize("T,K,E,D", [(8192, 8, 128, 2048), (100, 2, 8, 128), (37, 4, 6, 100), (5, 3, 4, 8)])
def test_scatter_gather(dev, T, K, E, D):
    g = gen(1006)
    ids = torch.stack([torch.randperm(E, generator=g)[:K] for _ in range(min(T, 512))])
    ids = ids.repeat((T + 511) // 512, 1)[:T].to(torch.int32)
    mapping, _ = o_moe.moe_sort(ids, E)
    x = randn(g, T, D)
    w = torch.softmax(randn(g, T, K, dtype=torch.float32), -1).to(torch.bfloat16)
    md = mapping.to(dev)
    xs = ops.flextrain_moe_scatter(x.to(dev), md)
    assert torch.equal(xs.cpu(), o_moe.moe_scatter(x, mapping)), "scatter is a copy: bit exact"
    xsw = ops.flextrain_moe_scatter(x.to(dev), md, scales=w.to(dev))
    close(xsw, o_moe.moe_scatter(x, mapping, w), what="scaled scatter")
    ws = ops.flextrain_moe_scatter_routing_weights(w.to(dev), md)
    assert torch.equal(ws.cpu(), o_moe.moe_scatter_routing_weights(w, mapping))
    y = randn(g, T * K, D)
    res = randn(g, T, D)
    close(ops.flextrain_moe_gather(y.to(dev), md, w.to(dev), res.to(dev)), o_moe.moe_gather(y, mapping, w, res),
          what="gather w+res")
    close(ops.flextrain_moe_gather(y.to(dev), md), o_moe.moe_gather(y, mapping), what="gather plain")
    # int64 indices take the same path
    assert torch.equal(ops.flextrain_moe_scatter(x.to(dev), md.long()), xs)
    # gather(scatter(x), 1/K) == x up to bf16 rounding of the 1/K weights
    if K in (2, 4, 8):
        ones = torch.full((T, K), 1.0 / K, dtype=torch.bfloat16, device=dev)
        assert torch.equal(ops.flextrain_moe_gather(xs, md, ones), x.to(dev))


def test_scatter_into_strided_slot_and_errors(dev):
    g = gen(7)
    T, K, D = 32, 2, 64
    ids = torch.randint(0, 4, (T, K), generator=g, dtype=torch.int32)
    mapping, _ = o_moe.moe_sort(ids, 4)
    x = randn(g, T, D)
    big = torch.zeros(T * K, 2 * D, dtype=torch.bfloat16, device=dev)
    ops.flextrain_moe_scatter(x.to(dev), mapping.to(dev), out=big[:, :D])
    assert torch.equal(big[:, :D].cpu(), o_moe.moe_scatter(x, mapping)) and not big[:, D:].any()
    with pytest.raises(ValueError):
        ops.flextrain_moe_scatter(x.to(dev), mapping.to(dev)[:5])
    with pytest.raises(ValueError):
        ops.flextrain_moe_gather(x.to(dev), mapping.to(dev))


# ------------------------------------------------------ expert activation
@pytest.mark.parametrize("R,F", [(65536, 768), (1000, 512), (33, 100), (4, 8)])
def test_swiglu_moe(dev, R, F):
    g = gen(1007)
    x = randn(g, R, 2 * F)
    w = torch.softmax(randn(g, R, 8, dtype=torch.float32), -1)[:, 0].to(torch.bfloat16)
    d = randn(g, R, F)
    close(ops.flextrain_swiglu_moe_fwd(x.to(dev), w.to(dev)), o_moe.swiglu_moe_fwd(x, w), what="fwd w")
    plain = ops.flextrain_swiglu_moe_fwd(x.to(dev))
    close(plain, o_moe.swiglu_moe_fwd(x), what="fwd")
    # tests/scratch/test_swiglu_fwd_no_w.py:28-33
    ones = torch.ones(R, dtype=torch.bfloat16, device=dev)
    assert (ops.flextrain_swiglu_moe_fwd(x.to(dev), ones).float() - plain.float()).abs().max() < 1e-3
    for prescaled, fn in ((False, ops.flextrain_swiglu_moe_bwd), (True, ops.flextrain_swiglu_moe_bwd_prescaled)):
        act = torch.empty(R, F, dtype=torch.bfloat16, device=dev)
        dx, dw = fn(d.to(dev), x.to(dev), w.to(dev), fwd_act=act)
        rdx, rdw, ract = o_moe.swiglu_moe_bwd(d, x, w, prescaled=prescaled)
        assert dw.dtype == torch.float32
        close(dx, rdx, what=f"dx prescaled={prescaled}")
        close(act, ract, what="fwd_act")
        scale = (1.0 / w.float().clamp(min=1e-8)) if prescaled else torch.ones(R)
        close(dw, rdw, rtol=1e-3, atol=1e-3 * float((F ** 0.5) * scale.max()), what="dw")
    # bf16 dprobs buffer shaped (R, 1), as the backend allocates it (moe_backend.py:470)
    dwb = torch.zeros(R, 1, dtype=torch.bfloat16, device=dev)
    ops.flextrain_swiglu_moe_bwd(d.to(dev), x.to(dev), w.to(dev), dw=dwb)
    close(dwb.reshape(-1), o_moe.swiglu_moe_bwd(d, x, w)[1], rtol=2e-2, atol=0.5, what="bf16 dw")


# -------------------------------------------------------- router backward
@pytest.mark.parametrize("mode", ["topk_then_softmax", "softmax_then_topk"])
@pytest.mark.parametrize("T,E,K", [(8192, 128, 8), (100, 12, 3), (7, 300, 70)])
def test_router_gate_bwd(dev, mode, T, E, K):
    g = gen(1008)
    logits = randn(g, T, E, std=0.5)
    w, ids = o_moe.topk_softmax(logits, K, mode=mode)
    mapping, counts = o_moe.moe_sort(ids, E)
    dprobs = randn(g, T * K, 1)
    base = randn(g, T, E, std=0.1)
    want = o_moe.router_gate_bwd(w, dprobs, mapping, ids, E, dlogits=base, mode=mode, logits=logits)
    dl = base.to(dev)
    out = ops.flextrain_moe_router_gate_bwd(w.to(dev), dprobs.to(dev), mapping.to(dev), ids.to(dev), dlogits=dl,
                                            mode=mode, logits=logits.to(dev))
    assert out is dl
    close(out, want, what="dlogits")
    fresh = ops.flextrain_moe_router_gate_bwd(w.to(dev), dprobs.to(dev), mapping.to(dev), ids.to(dev),
                                              num_experts=E, mode=mode, logits=logits.to(dev))
    close(fresh, o_moe.router_gate_bwd(w, dprobs, mapping, ids, E, mode=mode, logits=logits))
    lb = ops.flextrain_load_balance_bwd(logits.to(dev), counts.to(dev), E, K, alpha=0.01, tokens_per_step=4 * T,
                                        dlogits=base.to(dev))
    close(lb, o_moe.load_balance_bwd(logits, counts, K, 0.01, 4 * T, base), what="load balance")
    lb32 = ops.flextrain_load_balance_bwd(logits.float().to(dev), counts.to(dev), E, K, alpha=1.0)
    close(lb32, o_moe.load_balance_bwd(logits.float(), counts, K, 1.0), rtol=1e-4, atol=1e-7, what="lb fp32")
