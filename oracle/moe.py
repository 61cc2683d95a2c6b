"""MoE routing / permutation / expert-activation oracle (CPU).  Test
infrastructure — see oracle/__init__.py.

Restates flextrain/ops/_kernels/moe.py (kernels :29-642) and the expert loop of
flextrain/ops/full_moe.py:393-626 with plain PyTorch.  Integer results (expert
ids, index mapping, counts) are exact; floating-point results are fp32 with the
reference's rounding points (selected logits pass through the weights dtype,
moe.py:292-293; gather accumulates in fp32 starting from the residual,
moe.py:577-595).

Pinned by tests/test_oracle_moe.py: stable descending sort for top-k (with
deliberate ties), stable argsort / bincount and an O(n^2) rank count for the
sort, indexing identities for scatter/gather, torch.autograd through
softmax / silu for every backward, and an eager per-expert MLP with autograd
for the grouped expert block (tests/moe/test_moe_backend_parity.py:45-107), and -- for
the composed block ``routed_block_fwd_bwd`` (routing weights, gather with residual,
router path, load-balance term, ``experts=`` subset) -- fp64 autograd through the whole
block written as one differentiable expression with the selection held constant.
"""
from __future__ import annotations

import torch


# ------------------------------------------------------------------ routing
def topk_softmax(logits, top_k, mode="topk_then_softmax", weights_dtype=None):
    """-> (weights [T,K] in weights_dtype, ids [T,K] int32).  moe.py:255-314."""
    T, E = logits.shape
    wd = logits.dtype if weights_dtype is None else weights_dtype
    rem = logits.float().clone()
    if mode == "softmax_then_topk":
        rem = torch.softmax(rem, dim=-1)
    elif mode != "topk_then_softmax":
        raise ValueError(mode)
    ids = torch.empty(T, top_k, dtype=torch.int32)
    vals = torch.empty(T, top_k, dtype=torch.float32)
    ar = torch.arange(E).expand(T, E)
    rows = torch.arange(T)
    for k in range(top_k):
        mx = rem.max(dim=1, keepdim=True).values
        cand = torch.where(rem == mx, ar, torch.full_like(ar, E))
        pick = cand.min(dim=1).values                    # smallest index among the maxima
        ids[:, k] = pick.to(torch.int32)
        vals[:, k] = mx[:, 0]
        rem[rows, pick] = float("-inf")
    stored = vals.to(wd)                                 # through the weights buffer
    if mode == "topk_then_softmax":
        stored = torch.softmax(stored.float(), dim=-1).to(wd)
    return stored, ids


def moe_sort(topk_ids, num_experts):
    """-> (index_mapping like topk_ids, counts [E] int32): destination row of
    every (token, slot) pair in expert-major, flat-index-stable order.  moe.py:461-495,649-783."""
    flat = topk_ids.reshape(-1).to(torch.int64)
    order = torch.argsort(flat, stable=True)
    mapping = torch.empty_like(flat)
    mapping[order] = torch.arange(flat.numel())
    counts = torch.bincount(flat, minlength=num_experts).to(torch.int32)
    return mapping.to(topk_ids.dtype).reshape(topk_ids.shape), counts


def router_gate_bwd(probs, dprobs, indices, chosen_experts, num_experts, dlogits=None,
                    mode="topk_then_softmax", logits=None):
    """moe.py:360-458.  dprobs is indexed through ``indices``; result accumulates into dlogits."""
    T, K = probs.shape
    out = torch.zeros(T, num_experts, dtype=probs.dtype) if dlogits is None else dlogits.clone()
    dp = dprobs.reshape(-1).float()[indices.reshape(-1).long()].reshape(T, K)
    ce = chosen_experts.long()
    if mode == "topk_then_softmax":
        p = probs.float()
        dz = p * (dp - (dp * p).sum(-1, keepdim=True))
        cur = out.gather(1, ce)
        out.scatter_(1, ce, (cur.float() + dz.to(out.dtype).float()).to(out.dtype))
    else:
        P = torch.softmax(logits.float(), dim=-1)
        tp = P.gather(1, ce)
        row = (dp * tp).sum(-1, keepdim=True)
        dz = -P * row
        dz.scatter_add_(1, ce, dp * tp)
        out = (out.float() + dz.to(out.dtype).float()).to(out.dtype)
    return out


def load_balance_bwd(logits, expert_counts, top_k, alpha=0.01, tokens_per_step=0, dlogits=None):
    """moe.py:601-642,1719-1731."""
    T, E = logits.shape
    f = expert_counts.float() / (T * top_k)
    scale = alpha * E / (tokens_per_step if tokens_per_step else T)
    p = torch.softmax(logits.float(), dim=-1)
    grad = scale * p * (f - (f * p).sum(-1, keepdim=True))
    base = torch.zeros_like(logits) if dlogits is None else dlogits
    return (base.float() + grad).to(base.dtype)


# ------------------------------------------------------------ data movement
def moe_scatter(x, indices, scales=None):
    """out[indices[t,k]] = x[t] * scales[t,k].  moe.py:508-543."""
    T, D = x.shape
    K = indices.shape[1]
    out = torch.empty(T * K, D, dtype=x.dtype)
    for k in range(K):
        v = x if scales is None else (x.float() * scales.reshape(T, K)[:, k:k + 1].float()).to(x.dtype)
        out[indices[:, k].long()] = v
    return out


def moe_scatter_routing_weights(weights, indices):
    out = torch.empty(weights.numel(), dtype=weights.dtype)
    out[indices.reshape(-1).long()] = weights.reshape(-1)
    return out


def moe_gather(expert_out, indices, weights=None, residual=None, out_dtype=None):
    """moe.py:560-598."""
    T, K = indices.shape
    acc = residual.float().clone() if residual is not None else torch.zeros(T, expert_out.shape[1])
    for k in range(K):
        v = expert_out[indices[:, k].long()].float()
        acc = acc + (v * weights[:, k:k + 1].float() if weights is not None else v)
    if out_dtype is None:
        out_dtype = residual.dtype if residual is not None else expert_out.dtype
    return acc.to(out_dtype)


# -------------------------------------------------------- expert activation
def swiglu_moe_fwd(x, w=None):
    """x rows packed [value | gate].  moe.py:29-74."""
    F = x.shape[1] // 2
    x3, x1 = x[:, :F].float(), x[:, F:].float()
    y = (x1 * torch.sigmoid(x1)) * x3
    if w is not None:
        y = y * w.reshape(-1, 1).float()
    return y.to(x.dtype)


def swiglu_moe_bwd(dout, x, w, prescaled=False):
    """-> (dx packed [d value | d gate], dw fp32 (rows,), fwd_act).  moe.py:77-215."""
    F = dout.shape[1]
    x3, x1, d = x[:, :F].float(), x[:, F:].float(), dout.float()
    wv = w.reshape(-1, 1).float()
    s = torch.sigmoid(x1)
    silu = x1 * s
    un = silu * x3
    ds = s + silu * (1.0 - s)
    if prescaled:
        dw = ((d * (1.0 / torch.clamp(wv, min=1e-8))) * un).sum(-1)
        dx3, dx1, act = d * silu, d * x3 * ds, un
    else:
        dw = (d * un).sum(-1)
        dx3, dx1, act = d * wv * silu, d * wv * x3 * ds, un * wv
    return torch.cat([dx3, dx1], dim=1).to(x.dtype), dw, act.to(x.dtype)


# ----------------------------------------------------- grouped expert block
def expert_offsets(counts):
    off = torch.zeros(counts.numel() + 1, dtype=torch.int64)
    off[1:] = torch.cumsum(counts.long(), 0)
    return off


def grouped_expert_fwd(xg, counts, w_up, w_down):
    """Per expert e over rows [off[e], off[e+1]): pre = x_e @ w_up[e].T (bf16),
    act = silu(gate)*value (bf16), y = act @ w_down[e].T (bf16).
    flextrain/ops/full_moe.py:428-466."""
    off = expert_offsets(counts)
    TK = xg.shape[0]
    E, F2, d = w_up.shape
    pre = torch.zeros(TK, F2, dtype=xg.dtype)
    act = torch.zeros(TK, F2 // 2, dtype=xg.dtype)
    y = torch.zeros(TK, d, dtype=xg.dtype)
    for e in range(E):
        a, b = int(off[e]), int(off[e + 1])
        if a == b:
            continue
        pre[a:b] = (xg[a:b].float() @ w_up[e].float().t()).to(xg.dtype)
        act[a:b] = swiglu_moe_fwd(pre[a:b])
        y[a:b] = (act[a:b].float() @ w_down[e].float().t()).to(xg.dtype)
    return pre, act, y


def grouped_expert_bwd(dyg, xg, pre, wsorted, counts, w_up, w_down, g_up=None, g_down=None):
    """Backward of the expert block on grouped rows (full_moe.py:545-626):
    dx_act = dy_e @ w_down[e]; (dx_up, dprobs, act*w) = swiglu bwd;
    g_down[e] += dy_e.T @ (act*w); dx = dx_up @ w_up[e]; g_up[e] += dx_up.T @ x_e.
    Returns (dx_grouped, dprobs fp32 (TK,), g_up fp32, g_down fp32)."""
    off = expert_offsets(counts)
    E, F2, d = w_up.shape
    TK = xg.shape[0]
    dx = torch.zeros(TK, d, dtype=xg.dtype)
    dprobs = torch.zeros(TK, dtype=torch.float32)
    gu = torch.zeros(E, F2, d) if g_up is None else g_up.float().clone()
    gd = torch.zeros(E, d, F2 // 2) if g_down is None else g_down.float().clone()
    for e in range(E):
        a, b = int(off[e]), int(off[e + 1])
        if a == b:
            continue
        dact = (dyg[a:b].float() @ w_down[e].float()).to(xg.dtype)
        dx_up, dw, act_w = swiglu_moe_bwd(dact, pre[a:b], wsorted[a:b])
        dprobs[a:b] = dw
        gd[e] += dyg[a:b].float().t() @ act_w.float()
        dx[a:b] = (dx_up.float() @ w_up[e].float()).to(xg.dtype)
        gu[e] += dx_up.float().t() @ xg[a:b].float()
    return dx, dprobs, gu, gd


# ------------------------------------------------------------ whole block
def routed_block_fwd_bwd(x, logits, w_router, w_up, w_down, residual, dy, top_k, mode="topk_then_softmax",
                         load_balance_coef=0.0, tokens_per_step=None, experts=None):
    """The routed-SwiGLU block of flextrain/ops/full_moe.py:177-362 from given router
    logits (so that routing does not depend on GEMM rounding): forward output, and
    backward dx (including the router path), g_up, g_down, g_router.

    ``experts``: optional subset of expert ids to evaluate the expert MLP for (rows
    of other experts contribute zero) — used to bound CPU time at full size.
    Returns a dict of tensors."""
    T, d = x.shape
    E = w_up.shape[0]
    w, ids = topk_softmax(logits, top_k, mode=mode)
    mapping, counts = moe_sort(ids, E)
    if experts is not None:
        keep = torch.zeros(E, dtype=torch.bool)
        keep[list(experts)] = True
        counts_eval = torch.where(keep, counts, torch.zeros_like(counts))
    xg = moe_scatter(x, mapping)
    wsorted = moe_scatter_routing_weights(w, mapping)
    off = expert_offsets(counts)

    def run(fn_rows):
        # evaluate per expert on its true row range, skipping unselected experts
        for e in range(E):
            a, b = int(off[e]), int(off[e + 1])
            if a == b or (experts is not None and e not in experts):
                continue
            fn_rows(e, a, b)

    TK = T * top_k
    F2 = w_up.shape[1]
    pre = torch.zeros(TK, F2, dtype=x.dtype)
    y = torch.zeros(TK, d, dtype=x.dtype)

    def fwd_rows(e, a, b):
        pre[a:b] = (xg[a:b].float() @ w_up[e].float().t()).to(x.dtype)
        act = swiglu_moe_fwd(pre[a:b])
        y[a:b] = (act.float() @ w_down[e].float().t()).to(x.dtype)

    run(fwd_rows)
    out = moe_gather(y, mapping, w, residual)

    dyg = moe_scatter(dy, mapping)
    dxg = torch.zeros(TK, d, dtype=x.dtype)
    dprobs = torch.zeros(TK, dtype=torch.float32)
    g_up = torch.zeros(E, F2, d)
    g_down = torch.zeros(E, d, F2 // 2)

    def bwd_rows(e, a, b):
        dact = (dyg[a:b].float() @ w_down[e].float()).to(x.dtype)
        dx_up, dw, act_w = swiglu_moe_bwd(dact, pre[a:b], wsorted[a:b])
        dprobs[a:b] = dw
        g_down[e] = dyg[a:b].float().t() @ act_w.float()
        dxg[a:b] = (dx_up.float() @ w_up[e].float()).to(x.dtype)
        g_up[e] = dx_up.float().t() @ xg[a:b].float()

    run(bwd_rows)
    dx = moe_gather(dxg, mapping)
    dprobs_b = dprobs.to(x.dtype)                      # the backend's dprobs buffer is in compute dtype
    dlogits = router_gate_bwd(w, dprobs_b, mapping, ids, E, mode=mode, logits=logits)
    if load_balance_coef > 0.0 and tokens_per_step is not None:
        dlogits = load_balance_bwd(logits, counts, top_k, load_balance_coef, tokens_per_step, dlogits)
    dx_total = (dx.float() + dlogits.float() @ w_router.float().t()).to(x.dtype)
    g_router = x.float().t() @ dlogits.float()
    return dict(out=out, dx=dx_total, dx_experts=dx, g_up=g_up, g_down=g_down, g_router=g_router, ids=ids,
                weights=w, mapping=mapping, counts=counts, pre=pre, dlogits=dlogits)
