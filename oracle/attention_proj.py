"""CPU restatement of the attention block around its core (flextrain/nn/blocks/attention.py:424-463,
:493-500, :614-629, :712-775, :777-823).  Test infrastructure only.

Every tensor the reference stores between kernels in the compute dtype (the projected Q / K / V,
their normed and rotated versions, the gradient entering the core, the three partial sums of the
input gradient) is rounded to that dtype here as well; GEMMs accumulate in fp32.
"""
import torch

from . import rmsnorm, rope


def _mm(a, b, dtype):
    return (a.float() @ b.float()).to(dtype)


def qkv_fwd(x, pos, w, cfg, inv_freq):
    """x (T, d) -> q (T, H, D), k, v (T, Hkv, D), rstd_q, rstd_k (or None): projection, bias,
    per-head RMSNorm, RoPE (attention.py:424-463)."""
    dt = x.dtype
    T = x.shape[0]
    q, k, v = _mm(x, w["w_q"], dt), _mm(x, w["w_k"], dt), _mm(x, w["w_v"], dt)
    if cfg.qkv_bias:
        q, k, v = (q.float() + w["b_q"].float()).to(dt), (k.float() + w["b_k"].float()).to(dt), (v.float() + w["b_v"].float()).to(dt)
    rq = rk = None
    if cfg.qk_norm:
        q, rq = rmsnorm.rmsnorm_fwd(q, w["w_q_norm"], cfg.rms_norm_eps, head_dim=cfg.head_dim)
        k, rk = rmsnorm.rmsnorm_fwd(k, w["w_k_norm"], cfg.rms_norm_eps, head_dim=cfg.head_dim)
    q = rope.rope(q.view(T, cfg.n_heads, cfg.head_dim), pos, inv_freq)
    k = rope.rope(k.view(T, cfg.n_kv_heads, cfg.head_dim), pos, inv_freq)
    return q, k, v.view(T, cfg.n_kv_heads, cfg.head_dim), rq, rk


def o_fwd(x_resid, attn_result, w):
    """x_resid + attn_result W_o, one rounding (attention.py:493-500)."""
    T = x_resid.shape[0]
    return (x_resid.float() + attn_result.reshape(T, -1).float() @ w["w_o"].float()).to(x_resid.dtype)


def o_bwd(dx_resid, attn_result, w, g_o):
    """-> (gradient entering the core (T, H*D), g_o') (attention.py:614-629)."""
    T = dx_resid.shape[0]
    g = (g_o.float() + attn_result.reshape(T, -1).float().t() @ dx_resid.float()).to(g_o.dtype)
    return _mm(dx_resid, w["w_o"].t(), dx_resid.dtype), g


def qkv_bwd(dq, dk, dv, x, pos, w, cfg, inv_freq, rq=None, rk=None):
    """Core gradients (post-RoPE) -> (dx, dict of parameter gradients) (attention.py:712-823);
    the dict holds g_q, g_k, g_v and, when configured, g_b_q / g_b_k / g_b_v (sums over tokens of
    the rounded projection gradients) and g_q_norm / g_k_norm (fp32)."""
    dt = dq.dtype
    T = dq.shape[0]
    dq = rope.rope(dq.view(T, cfg.n_heads, cfg.head_dim), pos, inv_freq, backward=True).reshape(T, -1)
    dk = rope.rope(dk.view(T, cfg.n_kv_heads, cfg.head_dim), pos, inv_freq, backward=True).reshape(T, -1)
    dv = dv.reshape(T, -1)
    out = {}
    if cfg.qk_norm:
        xq, xk = _mm(x, w["w_q"], dt), _mm(x, w["w_k"], dt)
        if cfg.qkv_bias:
            xq, xk = (xq.float() + w["b_q"].float()).to(dt), (xk.float() + w["b_k"].float()).to(dt)
        dq, out["g_q_norm"], _ = rmsnorm.rmsnorm_bwd(dq, xq, w["w_q_norm"], rq, head_dim=cfg.head_dim)
        dk, out["g_k_norm"], _ = rmsnorm.rmsnorm_bwd(dk, xk, w["w_k_norm"], rk, head_dim=cfg.head_dim)
    if cfg.qkv_bias:
        out["g_b_q"], out["g_b_k"], out["g_b_v"] = dq.float().sum(0), dk.float().sum(0), dv.float().sum(0)
    dx = _mm(dq, w["w_q"].t(), dt)
    dx = (dx.float() + dk.float() @ w["w_k"].float().t()).to(dt)
    dx = (dx.float() + dv.float() @ w["w_v"].float().t()).to(dt)
    out["g_q"], out["g_k"], out["g_v"] = x.float().t() @ dq.float(), x.float().t() @ dk.float(), x.float().t() @ dv.float()
    return dx, out
