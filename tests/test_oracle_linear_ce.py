"""Pins the softmax / cross-entropy / LM-head oracle against library routines and
autograd.  CPU only."""
import torch
import torch.nn.functional as F

from oracle import linear_ce as o_ce
from util import gen, randn


def test_softmax_matches_library_argmax_first_occurrence():
    g = gen(1)
    x = randn(g, 16, 1000, dtype=torch.float32, std=3.0)
    x[3, 10] = x[3, 500] = x[3].max() + 1.0       # a tie: the first index must be reported
    p, idx, mx = o_ce.softmax(x, temperature=0.7)
    torch.testing.assert_close(p, torch.softmax(x / 0.7, -1), rtol=1e-5, atol=1e-7)
    assert torch.equal(idx, torch.argmax(x, dim=1)) and idx[3] == 10
    torch.testing.assert_close(mx, p.max(dim=1).values, rtol=1e-5, atol=0)
    pb, _, _ = o_ce.softmax(x.to(torch.bfloat16))
    assert pb.dtype == torch.bfloat16


def test_cross_entropy_from_probs_matches_nll():
    g = gen(2)
    x = randn(g, 32, 50, dtype=torch.float32)
    labels = torch.randint(0, 50, (32,), generator=g)
    labels[5], labels[6] = -100, 50                 # both outside [0, V)
    p = torch.softmax(x, -1)
    dz, loss, valid = o_ce.cross_entropy_from_probs(p, labels)
    ok = valid.bool()
    torch.testing.assert_close(loss[ok], F.cross_entropy(x[ok], labels[ok], reduction="none"), rtol=1e-5, atol=1e-6)
    assert loss[5] == 0 and loss[6] == 0 and not ok[5] and not ok[6]
    onehot = F.one_hot(labels.clamp(0, 49), 50).float() * valid[:, None]
    torch.testing.assert_close(dz, p - onehot, rtol=1e-6, atol=1e-7)
    tiny = torch.full((1, 4), 1e-60)
    assert o_ce.cross_entropy_from_probs(tiny, torch.tensor([0]))[1][0] == 100.0   # clamp


def test_fused_softmax_ce_matches_functional_cross_entropy_and_autograd():
    g = gen(3)
    x = randn(g, 64, 300, dtype=torch.float32, std=2.0).requires_grad_()
    labels = torch.randint(0, 300, (64,), generator=g)
    labels[::10] = -100
    mask = torch.ones(64, dtype=torch.bool)
    mask[3] = False
    total = F.cross_entropy(x, labels, ignore_index=-100, reduction="none")
    total = (total * mask).sum()
    (gx,) = torch.autograd.grad(total, x)
    dz, loss, idx, mx = o_ce.softmax_ce(x.detach(), labels, mask)
    torch.testing.assert_close(loss.sum(), total.detach(), rtol=1e-5, atol=1e-5)
    torch.testing.assert_close(dz, gx, rtol=1e-5, atol=1e-7)
    assert not dz[0].any() and loss[0] == 0 and not dz[3].any() and loss[3] == 0
    kept = (labels != -100) & mask
    torch.testing.assert_close(dz[kept].sum(-1), torch.zeros(int(kept.sum())), rtol=0, atol=1e-5)


def test_head_matches_autograd_and_is_chunk_independent():
    g = gen(4)
    T, d, V = 48, 32, 200
    x = randn(g, T, d, dtype=torch.float32)
    w_norm = randn(g, d, dtype=torch.float32, std=0.1, mean=1.0)
    w_head = randn(g, d, V, dtype=torch.float32, std=0.2)
    labels = torch.randint(0, V, (T,), generator=g)
    labels[torch.rand(T, generator=g) < 0.1] = -100
    scale = 1.0 / int((labels != -100).sum())
    xa, wn, wh = x.clone().requires_grad_(), w_norm.clone().requires_grad_(), w_head.clone().requires_grad_()
    h = F.rms_norm(xa, (d,), wn, eps=1e-5)
    loss = F.cross_entropy((h @ wh).float(), labels, ignore_index=-100, reduction="sum") * scale   # parity.py:374-379
    gx, gn, gh = torch.autograd.grad(loss, (xa, wn, wh))
    for chunk in (48, 16, 7):
        r = o_ce.head_forward_backward(x, w_norm, w_head, labels, chunk=chunk, loss_scale=scale)
        torch.testing.assert_close(r["per_token_loss"].sum() * scale, loss.detach(), rtol=1e-5, atol=1e-6)
        torch.testing.assert_close(r["dx"], gx, rtol=1e-4, atol=1e-6)
        torch.testing.assert_close(r["g_head"], gh, rtol=1e-4, atol=1e-6)
        torch.testing.assert_close(r["g_norm"], gn, rtol=1e-4, atol=1e-6)
    # loss_scale is linear; accumulators add
    r1 = o_ce.head_forward_backward(x, w_norm, w_head, labels, loss_scale=1.0)
    r2 = o_ce.head_forward_backward(x, w_norm, w_head, labels, loss_scale=2.0, g_head=r1["g_head"])
    torch.testing.assert_close(r2["dx"], 2 * r1["dx"], rtol=1e-5, atol=1e-7)
    torch.testing.assert_close(r2["g_head"], 3 * r1["g_head"], rtol=1e-5, atol=1e-6)


def test_softcap_oracle_matches_autograd_through_capped_cross_entropy():
    """fp32 inputs (no rounding of the capped logits): the oracle's loss and dZ against autograd
    through F.cross_entropy(cap * tanh(logits / cap)); a dropped gate, a gate taken from the uncapped
    logits or a cap applied after the softmax all fail here."""
    g = gen(31)
    cap = 30.0
    x = randn(g, 40, 257, dtype=torch.float32, std=25.0).requires_grad_()      # well into the saturating range
    labels = torch.randint(0, 257, (40,), generator=g)
    labels[::7] = -100
    mask = torch.ones(40, dtype=torch.bool)
    mask[2] = False
    capped = torch.tanh(x / cap) * cap
    per_token = F.cross_entropy(capped, labels, ignore_index=-100, reduction="none") * mask
    (gx,) = torch.autograd.grad(per_token.sum(), x)
    dz, loss, idx, mx = o_ce.softmax_ce(x.detach(), labels, mask, logit_softcap=cap)
    torch.testing.assert_close(loss, per_token.detach(), rtol=1e-5, atol=1e-5)
    torch.testing.assert_close(dz, gx, rtol=1e-4, atol=1e-7)
    assert torch.equal(idx, capped.detach().argmax(-1))
    torch.testing.assert_close(mx, torch.softmax(capped.detach(), -1).max(-1).values, rtol=1e-5, atol=0)
    # the two-pass form of the reference (cap in place, loss, multiply by the saved gate) is the same thing
    y, gate = o_ce.softcap(x.detach(), cap)
    dz2, loss2, _, _ = o_ce.softmax_ce(y, labels, mask)
    torch.testing.assert_close(dz2 * gate, dz, rtol=1e-6, atol=1e-9)
    torch.testing.assert_close(loss2, loss, rtol=0, atol=0)
    # a very large cap is no cap
    dz3, loss3, _, _ = o_ce.softmax_ce(x.detach() * 0.01, labels, mask, logit_softcap=1e6)
    dz4, loss4, _, _ = o_ce.softmax_ce(x.detach() * 0.01, labels, mask)
    torch.testing.assert_close(dz3, dz4, rtol=1e-4, atol=1e-7)
    torch.testing.assert_close(loss3, loss4, rtol=1e-4, atol=1e-5)


def test_head_with_softcap_matches_autograd():
    g = gen(32)
    T, d, V, cap = 40, 32, 150, 5.0
    x = randn(g, T, d, dtype=torch.float32)
    w_norm = randn(g, d, dtype=torch.float32, std=0.1, mean=1.0)
    w_head = randn(g, d, V, dtype=torch.float32, std=1.0)               # logits of a few units: the cap bites
    labels = torch.randint(0, V, (T,), generator=g)
    labels[torch.rand(T, generator=g) < 0.1] = -100
    scale = 1.0 / int((labels != -100).sum())
    xa, wn, wh = x.clone().requires_grad_(), w_norm.clone().requires_grad_(), w_head.clone().requires_grad_()
    logits = F.rms_norm(xa, (d,), wn, eps=1e-5) @ wh
    assert float(logits.detach().abs().max()) > cap
    loss = F.cross_entropy(torch.tanh(logits / cap) * cap, labels, ignore_index=-100, reduction="sum") * scale
    gx, gn, gh = torch.autograd.grad(loss, (xa, wn, wh))
    for chunk in (40, 16):
        r = o_ce.head_forward_backward(x, w_norm, w_head, labels, chunk=chunk, loss_scale=scale, logit_softcap=cap)
        torch.testing.assert_close(r["per_token_loss"].sum() * scale, loss.detach(), rtol=1e-5, atol=1e-6)
        torch.testing.assert_close(r["dx"], gx, rtol=1e-4, atol=1e-6)
        torch.testing.assert_close(r["g_head"], gh, rtol=1e-4, atol=1e-6)
        torch.testing.assert_close(r["g_norm"], gn, rtol=1e-4, atol=1e-6)
