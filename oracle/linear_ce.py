"""Softmax / cross-entropy / LM-head oracle (CPU, fp32).  Test infrastructure —
see oracle/__init__.py.

``head_forward_backward`` restates the micro-chunk loop of
flextrain/nn/head.py:255-365 on top of the reference-held formula
``F.cross_entropy((rmsnorm(h) @ W).float(), labels, ignore_index=-100)``
(flextrain/bench/parity.py:374-379): logits are rounded to the compute dtype by
the GEMM, the loss is fp32 cross-entropy of those logits, dZ = softmax - onehot is
rounded to the compute dtype before the two backward GEMMs, ``loss_scale`` enters
only through the GEMM alpha (head.py:325-346).

``softmax`` / ``cross_entropy_from_probs`` restate the two reference kernels
(flextrain/ops/_kernels/softmax.py:13-108, cross_entropy.py:14-57) including the
rounding of the probabilities to the output dtype.

Pinned by tests/test_oracle_linear_ce.py: torch.softmax / argmax,
F.cross_entropy(reduction="none"/"sum") and torch.autograd through the whole head,
with and without the final-logit soft cap (autograd through
``F.cross_entropy(cap * tanh(logits / cap))``).
"""
from __future__ import annotations

import torch

from . import rmsnorm as o_norm


def softmax(x, out_dtype=None, temperature=1.0):
    """-> (probs in out_dtype, argmax int64 (first occurrence), max prob fp32 = 1/l)."""
    z = x.float() / temperature
    m = z.max(dim=1, keepdim=True).values
    e = torch.exp(z - m)
    l = e.sum(dim=1, keepdim=True)
    probs = (e / l).to(x.dtype if out_dtype is None else out_dtype)
    V = x.shape[1]
    first = torch.where(z == m, torch.arange(V).expand_as(z), torch.full_like(z, V, dtype=torch.int64)).min(dim=1).values
    return probs, first, (1.0 / l)[:, 0]


def cross_entropy_from_probs(p, labels, max_loss=100.0):
    """-> (dZ = p - onehot in p.dtype, loss fp32, valid fp32); labels outside [0,V) give loss 0."""
    T, V = p.shape
    lab = labels.long()
    valid = (lab >= 0) & (lab < V)
    safe = torch.where(valid, lab, torch.zeros_like(lab))
    pc = p[torch.arange(T), safe].float()
    loss = torch.where(valid, torch.clamp(-torch.log(pc), max=max_loss), torch.zeros(T))
    dz = p.clone()
    rows = torch.arange(T)[valid]
    dz[rows, safe[valid]] = (pc[valid] - 1.0).to(p.dtype)
    return dz, loss, valid.float()


def softcap(logits, cap):
    """Final-logit soft cap of flextrain/nn/head.py:273-282: -> (capped logits in logits.dtype,
    gate = 1 - (capped / cap)^2 in fp32, from the ROUNDED capped logits as the reference computes it)."""
    y = (torch.tanh(logits.float() / cap) * cap).to(logits.dtype)
    r = y.float() / cap
    return y, 1.0 - r * r


def softmax_ce(logits, labels, loss_mask=None, ignore_index=-100, max_loss=100.0, logit_softcap=None):
    """The fused op: -> (dZ in logits.dtype, loss fp32, argmax, max prob).  With ``logit_softcap`` the
    loss, argmax and probabilities are those of the capped logits and dZ is chained through the cap's
    derivative (flextrain/nn/head.py:295-297), i.e. the gradient at the uncapped logits."""
    T, V = logits.shape
    gate = None
    if logit_softcap is not None:
        logits, gate = softcap(logits, logit_softcap)
    z = logits.float()
    lab = labels.long()
    keep = lab != ignore_index
    if loss_mask is not None:
        keep = keep & loss_mask.bool()
    valid = (lab >= 0) & (lab < V)
    lse = torch.logsumexp(z, dim=1)
    safe = torch.where(valid, lab, torch.zeros_like(lab))
    loss = torch.where(keep & valid, torch.clamp(lse - z[torch.arange(T), safe], max=max_loss), torch.zeros(T))
    dz = torch.exp(z - lse[:, None])
    hot = keep & valid
    dz[torch.arange(T)[hot], safe[hot]] -= 1.0
    dz = dz * keep[:, None].float()
    if gate is not None:
        dz = dz * gate
    _, first, mx = softmax(logits)
    return dz.to(logits.dtype), loss, first, mx


def head_forward_backward(x, w_norm, w_head, labels, eps=1e-5, chunk=1024, loss_scale=1.0, loss_mask=None,
                          g_head=None, g_norm=None, ignore_index=-100, logit_softcap=None):
    """x (T,d) compute dtype; w_head (d,V); returns dict(dx, per_token_loss, g_head fp32, g_norm fp32,
    next_prediction, next_prediction_prob)."""
    T, d = x.shape
    V = w_head.shape[1]
    dt = x.dtype
    dx = torch.empty_like(x)
    loss = torch.empty(T, dtype=torch.float32)
    pred = torch.empty(T, dtype=torch.int64)
    prob = torch.empty(T, dtype=torch.float32)
    gh = torch.zeros(d, V) if g_head is None else g_head.float().clone()
    gn = torch.zeros(d) if g_norm is None else g_norm.float().clone()
    wf = w_head.float()
    for o in range(0, T, chunk):
        s = slice(o, min(o + chunk, T))
        h, rstd = o_norm.rmsnorm_fwd(x[s], w_norm, eps)
        logits = (h.float() @ wf).to(dt)
        dz, loss[s], pred[s], prob[s] = softmax_ce(logits, labels[s], None if loss_mask is None else loss_mask[s],
                                                   ignore_index, logit_softcap=logit_softcap)
        gh += loss_scale * (h.float().t() @ dz.float())
        dh = (loss_scale * (dz.float() @ wf.t())).to(dt)
        dx[s], gn, _ = o_norm.rmsnorm_bwd(dh, x[s], w_norm, rstd, dw_old=gn)
    return dict(dx=dx, per_token_loss=loss, g_head=gh, g_norm=gn, next_prediction=pred, next_prediction_prob=prob)
