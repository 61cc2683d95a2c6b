"""Softmax, cross-entropy, the fused logits -> (loss, dZ) kernel and the chunked LM
head against the CPU oracle.  Tolerances: bf16 tensors rtol 1e-2 / atol 1e-2, fp32
loss rtol 1e-4 (against fp32 cross-entropy of the same bf16 logits)."""
import pytest
import torch
import torch.nn.functional as F

from flextrain_amd import ops
from flextrain_amd.head import LMHead, LMHeadConfig
from flextrain_amd.loss import CrossEntropyLoss, TokenContext
from oracle import linear_ce as o_ce
from oracle.rmsnorm import rmsnorm_bwd as o_norm_bwd
from oracle.rmsnorm import rmsnorm_fwd as o_norm_fwd
from util import F32_RTOL, close, gen, randn

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("T,V", [(64, 128256), (7, 1000), (33, 50257), (5, 8), (16, 32000)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_softmax_matches_oracle(dev, T, V, dtype):
    g = gen(T + V)
    x = randn(g, T, V, dtype=dtype, std=3.0)
    x[0, 3] = x[0, V - 1] = x[0].max() + 1          # a tie: first occurrence wins
    p_ref, idx_ref, mx_ref = o_ce.softmax(x, temperature=0.8)
    idx = torch.empty(T, dtype=torch.int64, device=dev)
    mx = torch.empty(T, dtype=torch.float32, device=dev)
    out, i2, m2 = ops.flextrain_softmax(x.to(dev), max_idx_out=idx, max_val_out=mx, temperature=0.8)
    assert i2 is idx and m2 is mx and out.dtype == dtype
    close(out, p_ref, rtol=1e-2, atol=1e-5, what="probs")
    assert torch.equal(idx.cpu(), idx_ref) and idx[0] == 3
    close(mx, mx_ref, rtol=1e-4, atol=0, what="max prob")


def test_softmax_errors(dev):
    x = torch.zeros(4, 8, device=dev)
    with pytest.raises(ValueError):
        ops.flextrain_softmax(x[:, ::2])
    with pytest.raises(ValueError):
        ops.flextrain_softmax(x, temperature=0.0)
    with pytest.raises(ValueError):
        ops.flextrain_softmax(x.view(2, 2, 8))
    with pytest.raises(TypeError):
        ops.flextrain_softmax(x.to(torch.int32))
    with pytest.raises(ValueError):
        ops.flextrain_softmax(x, max_idx_out=torch.empty(4, dtype=torch.int32, device=dev))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_cross_entropy_from_probs_in_place(dev, dtype):
    g = gen(11)
    T, V = 130, 4099
    p = torch.softmax(randn(g, T, V, dtype=torch.float32, std=2.0), -1).to(dtype)
    labels = torch.randint(0, V, (T,), generator=g)
    labels[3], labels[4] = -100, V
    dz_ref, loss_ref, valid_ref = o_ce.cross_entropy_from_probs(p, labels)
    pd = p.to(dev)
    valid = torch.empty(T, dtype=torch.float32, device=dev)
    dz, loss = ops.flextrain_cross_entropy_loss(pd, labels.to(dev), Valid_Count_out=valid)
    assert dz.data_ptr() == pd.data_ptr()
    close(loss, loss_ref, rtol=1e-5, atol=1e-6, what="loss")
    close(dz, dz_ref, rtol=1e-2, atol=1e-6, what="dZ")
    assert torch.equal(valid.cpu(), valid_ref)
    # int32 labels take the same path
    pd2 = p.to(dev)
    _, loss2 = ops.flextrain_cross_entropy_loss(pd2, labels.to(torch.int32).to(dev))
    assert torch.equal(loss2, loss) and torch.equal(pd2, pd)
    # the summary wrapper: same kernel, then the three scalars on the host
    pd3 = p.to(dev)
    X, L, total, avg, n_valid = ops.flextrain_softmax_cross_entropy_loss(pd3, labels.to(dev))
    assert X.data_ptr() == pd3.data_ptr() and torch.equal(pd3, pd) and torch.equal(L, loss)
    assert n_valid == float(valid_ref.sum()) and isinstance(total, float)
    assert total == pytest.approx(float(loss_ref.sum()), rel=1e-5)
    assert avg == pytest.approx(float(loss_ref.sum()) / float(valid_ref.sum()), rel=1e-5)


@pytest.mark.parametrize("T,V", [(40, 128256), (9, 777), (16, 4096)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_fused_softmax_ce(dev, T, V, dtype):
    g = gen(V)
    x = randn(g, T, V, dtype=dtype, std=2.0)
    labels = torch.randint(0, V, (T,), generator=g)
    labels[::5] = -100
    mask = torch.ones(T, dtype=torch.bool)
    mask[1] = False
    dz_ref, loss_ref, idx_ref, mx_ref = o_ce.softmax_ce(x, labels, mask)
    # the oracle itself against the library on these inputs
    want = F.cross_entropy(x.float(), labels, ignore_index=-100, reduction="none") * mask
    torch.testing.assert_close(loss_ref, want, rtol=1e-5, atol=1e-5)
    xd = x.to(dev)
    idx = torch.empty(T, dtype=torch.int64, device=dev)
    mx = torch.empty(T, dtype=torch.float32, device=dev)
    dz, loss = ops.flextrain_softmax_cross_entropy(xd, labels.to(dev), loss_mask=mask.to(dev), max_idx_out=idx,
                                                   max_val_out=mx)
    assert dz.data_ptr() == xd.data_ptr()
    close(loss, loss_ref, rtol=F32_RTOL, atol=1e-5, what="loss")
    close(dz, dz_ref, rtol=1e-2, atol=1e-5, what="dZ")
    assert torch.equal(idx.cpu(), idx_ref)
    close(mx, mx_ref, rtol=1e-4, atol=0)
    assert not dz[0].any() and not dz[1].any() and loss[0] == 0 and loss[1] == 0
    # out of place leaves the logits alone
    xd2 = x.to(dev)
    out = torch.empty_like(xd2)
    ops.flextrain_softmax_cross_entropy(xd2, labels.to(dev), dZ=out, loss_mask=mask.to(dev))
    assert torch.equal(xd2.cpu(), x) and torch.equal(out, dz)


@pytest.mark.parametrize("T,V", [(24, 128256), (9, 777)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_fused_softmax_ce_with_logit_softcap(dev, T, V, dtype):
    """Final-logit soft cap inside the fused kernel (flextrain/nn/head.py:273-298) against the oracle
    (pinned by autograd through F.cross_entropy(cap * tanh(l / cap))), and against the two-pass form
    (cap in place + gate, loss, gate multiply) built from the stand-alone softcap kernels."""
    g = gen(V + 1)
    cap = 30.0
    x = randn(g, T, V, dtype=dtype, std=20.0)
    labels = torch.randint(0, V, (T,), generator=g)
    labels[::5] = -100
    mask = torch.ones(T, dtype=torch.bool)
    mask[1] = False
    dz_ref, loss_ref, idx_ref, mx_ref = o_ce.softmax_ce(x, labels, mask, logit_softcap=cap)
    xd = x.to(dev)
    idx = torch.empty(T, dtype=torch.int64, device=dev)
    mx = torch.empty(T, dtype=torch.float32, device=dev)
    dz, loss = ops.flextrain_softmax_cross_entropy(xd, labels.to(dev), loss_mask=mask.to(dev), max_idx_out=idx,
                                                   max_val_out=mx, logit_softcap=cap)
    assert dz.data_ptr() == xd.data_ptr()
    close(loss, loss_ref, rtol=F32_RTOL, atol=1e-4, what="loss")
    close(dz, dz_ref, rtol=1e-2, atol=1e-5, what="dZ")
    # near the cap many capped logits round to the same bf16 value: the argmax is any of the tied maxima
    y_ref, _ = o_ce.softcap(x, cap)
    top_got, top_ref = y_ref[torch.arange(T), idx.cpu()].float(), y_ref[torch.arange(T), idx_ref].float()
    assert bool((top_got >= top_ref * (1 - 2.0 ** -7)).all())          # within one bf16 step of the maximum
    if dtype == torch.float32:
        assert torch.equal(idx.cpu(), idx_ref)
    close(mx, mx_ref, rtol=1e-3, atol=0)
    assert not dz[0].any() and not dz[1].any() and loss[0] == 0 and loss[1] == 0
    # two-pass form: same loss, dZ within one more rounding
    x2 = x.to(dev)
    gate = ops.flextrain_logit_softcap_fwd(x2, cap)
    y_ref, gate_ref = o_ce.softcap(x, cap)
    close(x2, y_ref, rtol=1e-2, atol=1e-5, what="capped logits")
    close(gate, gate_ref.to(dtype), rtol=1e-2, atol=1e-2, what="gate")
    dz2, loss2 = ops.flextrain_softmax_cross_entropy(x2, labels.to(dev), loss_mask=mask.to(dev))
    ops.flextrain_logit_softcap_bwd(dz2, gate)
    close(loss2, loss_ref, rtol=F32_RTOL, atol=1e-4, what="loss, two passes")
    close(dz2, dz_ref, rtol=2e-2 if dtype == torch.bfloat16 else 1e-4, atol=1e-5, what="dZ, two passes (bf16: two roundings)")
    with pytest.raises(ValueError):
        ops.flextrain_softmax_cross_entropy(xd, labels.to(dev), logit_softcap=0.0)
    with pytest.raises(ValueError):
        ops.flextrain_logit_softcap_fwd(xd[:, ::2], cap)


class _OpaqueLoss:
    """A loss object the head knows nothing about (no ``supports_logit_softcap``): the head must cap the
    logits itself before ``compute`` and multiply dZ by the gate afterwards."""

    def __init__(self):
        self.inner = CrossEntropyLoss()

    def compute(self, logits, token_slice, *, loss_scale, per_token_loss_out):
        return self.inner.compute(logits, token_slice, loss_scale=loss_scale, per_token_loss_out=per_token_loss_out)


@pytest.mark.parametrize("loss_kind", ["fused", "opaque"])
def test_lm_head_final_logit_softcap(dev, loss_kind):
    T, d, V, chunk, cap = 300, 256, 5000, 128, 30.0
    g = gen(23)
    x = randn(g, T, d)
    w_norm = randn(g, d, dtype=torch.float32, std=0.02, mean=1.0)
    w = randn(g, V, d, std=2.0)                        # logits ~ N(0, 32^2): a third of them beyond the cap
    labels = torch.randint(0, V, (T,), generator=g)
    labels[torch.rand(T, generator=g) < 0.1] = -100
    scale = 1.0 / int((labels != -100).sum())
    ref = o_ce.head_forward_backward(x, w_norm, w.t(), labels, chunk=chunk, loss_scale=scale, logit_softcap=cap)
    nocap = o_ce.head_forward_backward(x, w_norm, w.t(), labels, chunk=chunk, loss_scale=scale)
    assert (ref["dx"].float() - nocap["dx"].float()).abs().max() > 0.1 * nocap["dx"].float().abs().max()   # the cap matters here
    g_head = torch.zeros(d, V, dtype=torch.float32, device=dev)
    g_norm = torch.zeros(d, dtype=torch.float32, device=dev)
    head = LMHead(LMHeadConfig(d_model=d, vocab_size=V, head_chunk_size=chunk, fuse_chunks=1, final_logit_softcap=cap))
    xd = x.to(dev)
    dx, stats = head.forward_backward(xd, TokenContext(labels=labels.to(dev)), None,
                                      {"w_final_norm": w_norm.to(dev), "w_head_proj": w.to(dev).t()},
                                      {"g_head_proj": g_head, "g_final_norm": g_norm}, None, loss_scale=scale,
                                      loss_fn=CrossEntropyLoss() if loss_kind == "fused" else _OpaqueLoss())
    close(stats.per_token_loss.sum() * scale, ref["per_token_loss"].sum() * scale, rtol=5e-3, atol=0, what="mean loss")
    close(dx, ref["dx"], rtol=1e-2, atol=1e-2 * ref["dx"].float().abs().max().item(), what="dx")
    close(g_head, ref["g_head"], rtol=1e-2, atol=1e-2 * ref["g_head"].abs().max().item(), what="g_head")
    close(g_norm, ref["g_norm"], rtol=1e-2, atol=1e-2 * ref["g_norm"].abs().max().item(), what="g_norm")


class _KeepLogits:
    """A loss object (the head's ``loss_fn=`` hook) that keeps a copy of the bf16 logits the head
    produced before the wrapped loss turns them into dZ in place, so that the fp32 loss can be
    checked against ``F.cross_entropy`` of the SAME logits at the fp32 tolerance."""

    def __init__(self, inner):
        self.inner, self.kept = inner, []

    def compute(self, logits, token_slice, *, loss_scale, per_token_loss_out):
        self.kept.append(logits.cpu())
        return self.inner.compute(logits, token_slice, loss_scale=loss_scale, per_token_loss_out=per_token_loss_out)

    def logits(self):
        return torch.cat(self.kept)


def _head_inputs(seed, T, d, V, hf_layout):
    g = gen(seed)
    x = randn(g, T, d)
    w_norm = randn(g, d, dtype=torch.float32, std=0.02, mean=1.0)
    w = randn(g, V, d, std=0.02)                    # (V, d) as Hugging Face stores it
    labels = torch.randint(0, V, (T,), generator=g)
    labels[torch.rand(T, generator=g) < 0.1] = -100
    return x, w_norm, w, labels


@pytest.mark.parametrize("hf_layout", [True, False])
@pytest.mark.parametrize("fused", [True, False])
@pytest.mark.parametrize("fuse_chunks", [None, 1, 2])
def test_lm_head_forward_backward(dev, hf_layout, fused, fuse_chunks):
    T, d, V, chunk = 300, 256, 5000, 128
    x, w_norm, w, labels = _head_inputs(21, T, d, V, hf_layout)
    scale = 1.0 / int((labels != -100).sum())
    ref = o_ce.head_forward_backward(x, w_norm, w.t(), labels, chunk=chunk, loss_scale=scale)

    wd = w.to(dev).t() if hf_layout else w.t().contiguous().to(dev)         # logical (d, V) either way
    g_store = torch.zeros((V, d) if hf_layout else (d, V), dtype=torch.float32, device=dev)
    g_head = g_store.t() if hf_layout else g_store
    g_norm = torch.zeros(d, dtype=torch.float32, device=dev)
    head = LMHead(LMHeadConfig(d_model=d, vocab_size=V, head_chunk_size=chunk, fuse_chunks=fuse_chunks))
    xd = x.to(dev)
    keep = _KeepLogits(CrossEntropyLoss(fused=fused))
    dx, stats = head.forward_backward(xd, TokenContext(labels=labels.to(dev)), None,
                                      {"w_final_norm": w_norm.to(dev), "w_head_proj": wd},
                                      {"g_head_proj": g_head, "g_final_norm": g_norm}, None, loss_scale=scale,
                                      loss_fn=keep)
    assert dx is xd and stats.token_count == T
    if fused:
        close(stats.per_token_loss, ref["per_token_loss"], rtol=1e-2, atol=2e-2, what="per-token loss")
        # fp32 loss at rtol 1e-4: against fp32 cross-entropy of the very bf16 logits the head produced
        # (the oracle's own logits differ from them by GEMM accumulation order, a bf16-sized effect)
        want = F.cross_entropy(keep.logits().float(), labels, ignore_index=-100, reduction="none")
        close(stats.per_token_loss, want, rtol=F32_RTOL, atol=1e-5, what="per-token loss from the same logits")
        close(stats.per_token_loss.sum() * scale, want.sum() * scale, rtol=F32_RTOL, atol=0, what="mean loss")
        close(stats.per_token_loss.sum() * scale, ref["per_token_loss"].sum() * scale, rtol=1e-3, atol=0,
              what="mean loss against the oracle's own logits")
    else:
        close(stats.per_token_loss.sum() * scale, ref["per_token_loss"].sum() * scale, rtol=1e-2, atol=0, what="mean loss")
    ign = labels == -100
    assert not stats.per_token_loss.cpu()[ign].any()
    close(dx, ref["dx"], rtol=1e-2, atol=1e-2 * ref["dx"].abs().max().item(), what="dx")
    gh = ref["g_head"]
    close(g_head, gh, rtol=1e-2, atol=1e-2 * gh.abs().max().item(), what="g_head")
    close(g_norm, ref["g_norm"], rtol=1e-2, atol=1e-2 * ref["g_norm"].abs().max().item(), what="g_norm")
    agree = (stats.next_prediction.cpu() == ref["next_prediction"]).float().mean().item()
    assert agree > 0.97, agree      # argmax of bf16 logits: near-ties may flip with accumulation order


def test_lm_head_skips_missing_grads_and_bf16_accumulator(dev):
    T, d, V = 64, 128, 1024
    x, w_norm, w, labels = _head_inputs(22, T, d, V, False)
    ref = o_ce.head_forward_backward(x, w_norm, w.t(), labels, chunk=1024, loss_scale=0.5)
    head = LMHead(LMHeadConfig(d_model=d, vocab_size=V))
    wd = w.t().contiguous().to(dev)
    dx, _ = head.forward_backward(x.to(dev), TokenContext(labels=labels.to(dev)), None,
                                  {"w_final_norm": w_norm.to(dev), "w_head_proj": wd}, {}, None, loss_scale=0.5)
    close(dx, ref["dx"], rtol=1e-2, atol=1e-2 * ref["dx"].abs().max().item(), what="dx")
    g_head = torch.zeros(d, V, dtype=torch.bfloat16, device=dev)
    head.forward_backward(x.to(dev), TokenContext(labels=labels.to(dev)), None,
                          {"w_final_norm": w_norm.to(dev), "w_head_proj": wd}, {"g_head_proj": g_head}, None,
                          loss_scale=0.5)
    close(g_head, ref["g_head"], rtol=1e-2, atol=1e-2 * ref["g_head"].abs().max().item(), what="g_head bf16")
    with pytest.raises(ValueError):
        head.forward_backward(x.to(dev), TokenContext(labels=labels[:10].to(dev)), None,
                              {"w_final_norm": w_norm.to(dev), "w_head_proj": wd}, {}, None)


def test_full_size_llama_head(dev):
    """hidden [8192,4096], lm_head [128256,4096], 10 % ignored labels, micro-chunk 1024.  The oracle runs
    on a sample of token rows (whole vocabulary rows of logits, loss, dZ and the row's dx); everything
    else is checked through properties that hold at any size: two-chunk groups, eight-chunk groups and the
    per-chunk schedule (the default) agree, ignored rows have zero loss, and the head gradient sums to ~0
    over the vocabulary (every kept row of dZ sums to 0)."""
    T, d, V, chunk = 8192, 4096, 128256, 1024
    g = gen(1002)
    x = randn(g, T, d)
    w = (torch.empty(V, d).normal_(0, 0.02, generator=g)).to(torch.bfloat16)
    w_norm = torch.ones(d)
    labels = torch.randint(0, V, (T,), generator=g)
    labels[torch.rand(T, generator=g) < 0.1] = -100
    scale = 1.0 / int((labels != -100).sum())
    wd, ld, wn = w.to(dev), labels.to(dev), w_norm.to(dev)

    def run(fuse, loss_fn=None):
        xd = x.to(dev)
        gh = torch.zeros(V, d, dtype=torch.float32, device=dev)
        gn = torch.zeros(d, dtype=torch.float32, device=dev)
        head = LMHead(LMHeadConfig(d_model=d, vocab_size=V, head_chunk_size=chunk, fuse_chunks=fuse))
        dx, stats = head.forward_backward(xd, TokenContext(labels=ld), None, {"w_final_norm": wn, "w_head_proj": wd.t()},
                                          {"g_head_proj": gh.t(), "g_final_norm": gn}, None, loss_scale=scale,
                                          loss_fn=loss_fn)
        return dx, stats, gh, gn

    dx, stats, gh, gn = run(2)
    dx8, stats8, gh8, gn8 = run(8)
    keep = _KeepLogits(CrossEntropyLoss())
    dx1, stats1, gh1, gn1 = run(1, keep)
    # fp32 loss at rtol 1e-4, all 8192 tokens: fp32 cross-entropy (library routine, CPU) of the bf16
    # logits the head itself produced, one micro-chunk at a time
    want = torch.cat([F.cross_entropy(lg.float(), labels[i * chunk:(i + 1) * chunk], ignore_index=-100,
                                      reduction="none") for i, lg in enumerate(keep.kept)])
    # The backward at full size against the oracle's formulas, from the kept logits (so that the
    # comparison is not blurred by the logits GEMM's own rounding): dZ = softmax - onehot rounded to
    # bf16, dh = scale * dZ @ W rounded to bf16, RMSNorm backward of dh -> dx of all 8192 tokens and
    # g_norm; g_head rows of 40 sampled vocabulary entries = scale * dZ[:, v]^T @ h.
    vs = torch.cat([torch.tensor([0, 1, 2, 3, V - 4, V - 3, V - 2, V - 1]), torch.randint(0, V, (32,), generator=g)])
    wf = w.float()
    h_all, rstd_all = o_norm_fwd(x, w_norm)
    gh_ref = torch.zeros(len(vs), d)
    gn_ref = torch.zeros(d)
    dx_all = torch.empty(T, d, dtype=torch.bfloat16)
    for i, lg in enumerate(keep.kept):
        sl = slice(i * chunk, (i + 1) * chunk)
        dz, _, _, _ = o_ce.softmax_ce(lg, labels[sl])
        dzf = dz.float()
        gh_ref += scale * (dzf[:, vs].t() @ h_all[sl].float())
        dh = (scale * (dzf @ wf)).to(torch.bfloat16)
        dx_all[sl], gn_ref, _ = o_norm_bwd(dh, x[sl], w_norm, rstd_all[sl], dw_old=gn_ref)
        del dz, dzf, dh
    keep.kept.clear()
    del wf
    close(stats8.per_token_loss, stats1.per_token_loss, rtol=1e-4, atol=1e-4, what="loss, 8-chunk groups vs per chunk")
    for what, got_h, got_n, got_x in (("per chunk", gh1, gn1, dx1), ("2-chunk groups", gh, gn, dx), ("8-chunk groups", gh8, gn8, dx8)):
        close(got_h.cpu()[vs], gh_ref, rtol=1e-2, atol=1e-2 * gh_ref.abs().max().item(), what=f"g_head rows, {what}")
        close(got_n, gn_ref, rtol=1e-2, atol=1e-2 * gn_ref.abs().max().item(), what=f"g_norm, {what}")
        close(got_x, dx_all, rtol=1e-2, atol=1e-2 * dx_all.float().abs().max().item(), what=f"dx of all tokens, {what}")
    close(stats1.per_token_loss, want, rtol=F32_RTOL, atol=1e-5, what="per-token loss from the same logits")
    close(stats1.per_token_loss.sum() * scale, want.sum() * scale, rtol=F32_RTOL, atol=0, what="mean loss of 8192 tokens")
    close(stats.per_token_loss.sum() * scale, want.sum() * scale, rtol=F32_RTOL, atol=0, what="mean loss, grouped schedule")
    # schedule independence (accumulation order differs: bf16 dx, fp32 head gradient)
    close(stats.per_token_loss, stats1.per_token_loss, rtol=1e-4, atol=1e-4, what="loss grouped vs per chunk")
    close(dx, dx1, rtol=1e-2, atol=1e-2 * dx1.float().abs().max().item(), what="dx grouped vs per chunk")
    close(gh, gh1, rtol=1e-2, atol=1e-2 * gh1.abs().max().item(), what="g_head grouped vs per chunk")
    close(gn, gn1, rtol=1e-2, atol=1e-2 * gn1.abs().max().item(), what="g_norm grouped vs per chunk")
    loss = stats.per_token_loss.cpu()
    assert not loss[labels == -100].any() and bool((loss[labels != -100] > 0).all())
    col = gh.sum(dim=0)                       # sum over the vocabulary of d(loss)/dW[v, :]
    assert float(col.abs().max()) <= 2e-3 * float(gh.abs().sum(dim=0).max()), "head gradient must sum to ~0 over V"
    # sampled rows against the oracle
    rows = torch.cat([torch.arange(0, 8), torch.arange(4090, 4098), torch.tensor([T - 1])])
    h, rstd = o_norm_fwd(x[rows], w_norm)
    logits = (h.float() @ w.float().t()).to(torch.bfloat16)
    dz_ref, loss_ref, _, _ = o_ce.softmax_ce(logits, labels[rows])
    close(loss[rows], loss_ref, rtol=1e-3, atol=1e-3, what="sampled per-token loss")
    dh = (scale * (dz_ref.float() @ w.float())).to(torch.bfloat16)
    dx_ref, _, _ = o_norm_bwd(dh, x[rows], w_norm, rstd)
    close(dx.cpu()[rows], dx_ref, rtol=1e-2, atol=1e-2 * dx_ref.float().abs().max().item(), what="sampled dx")
