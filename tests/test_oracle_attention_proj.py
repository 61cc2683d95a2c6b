"""The attention-projection oracle against torch.autograd through an independent formulation
(fp32 throughout, RoPE written with complex numbers, RMSNorm with torch.nn.functional, the core
replaced by dense causal attention): no rounding between the steps, so the comparison is tight."""
import math

import pytest
import torch
import torch.nn.functional as F

from flextrain_amd.attention_proj import GQAProjectionConfig
from oracle import attention_proj as o_ap
from oracle import rope as o_rope
from util import gen, randn


def _rope_complex(x, pos, inv_freq):
    T, H, D = x.shape
    ang = pos.float().view(T, 1, 1) * inv_freq.view(1, 1, D // 2)
    z = torch.view_as_complex(x.reshape(T, H, D // 2, 2).contiguous()) * torch.polar(torch.ones_like(ang), ang)
    return torch.view_as_real(z).reshape(T, H, D)


def _core(q, k, v):
    """Dense causal grouped-query attention, (T, H, D) in and out."""
    T, H, D = q.shape
    rep = H // k.shape[1]
    kk, vv = k.repeat_interleave(rep, dim=1), v.repeat_interleave(rep, dim=1)
    s = torch.einsum("thd,shd->hts", q, kk) / math.sqrt(D)
    s = s.masked_fill(torch.triu(torch.ones(T, T, dtype=torch.bool), 1), float("-inf"))
    return torch.einsum("hts,shd->thd", s.softmax(-1), vv)


@pytest.mark.parametrize("bias,qk_norm", [(False, False), (True, False), (False, True), (True, True)])
def test_oracle_matches_autograd(bias, qk_norm):
    g = gen(17)
    f32 = torch.float32
    cfg = GQAProjectionConfig(d_model=24, n_heads=4, n_kv_heads=2, head_dim=8, rope_theta=10000.0, qkv_bias=bias,
                              qk_norm=qk_norm, rms_norm_eps=1e-5)
    T = 12
    x, resid, dy = (randn(g, T, cfg.d_model, dtype=f32) for _ in range(3))
    pos = torch.arange(3, 3 + T, dtype=torch.int32)
    inv_freq = o_rope.vanilla_inv_freq(cfg.head_dim, cfg.rope_theta)
    w = {"w_q": randn(g, cfg.d_model, cfg.attn_dim, dtype=f32, std=0.3), "w_k": randn(g, cfg.d_model, cfg.kv_dim, dtype=f32, std=0.3),
         "w_v": randn(g, cfg.d_model, cfg.kv_dim, dtype=f32, std=0.3), "w_o": randn(g, cfg.attn_dim, cfg.d_model, dtype=f32, std=0.3),
         "b_q": randn(g, cfg.attn_dim, dtype=f32), "b_k": randn(g, cfg.kv_dim, dtype=f32), "b_v": randn(g, cfg.kv_dim, dtype=f32),
         "w_q_norm": randn(g, cfg.head_dim, dtype=f32, mean=1.0, std=0.1), "w_k_norm": randn(g, cfg.head_dim, dtype=f32, mean=1.0, std=0.1)}
    leaf = {k: v.clone().requires_grad_() for k, v in w.items()}
    xx = x.clone().requires_grad_()

    def proj(name, b, heads):
        y = xx @ leaf[name]
        if bias:
            y = y + leaf[b]
        return y.view(T, heads, cfg.head_dim)

    q, k, v = proj("w_q", "b_q", cfg.n_heads), proj("w_k", "b_k", cfg.n_kv_heads), proj("w_v", "b_v", cfg.n_kv_heads)
    if qk_norm:
        q = F.rms_norm(q, (cfg.head_dim,), leaf["w_q_norm"], cfg.rms_norm_eps)
        k = F.rms_norm(k, (cfg.head_dim,), leaf["w_k_norm"], cfg.rms_norm_eps)
    q, k = _rope_complex(q, pos, inv_freq), _rope_complex(k, pos, inv_freq)
    q.retain_grad(), k.retain_grad(), v.retain_grad()
    attn = _core(q, k, v)
    attn.retain_grad()
    out_ref = resid + attn.reshape(T, -1) @ leaf["w_o"]
    (out_ref * dy).sum().backward()

    # forward halves
    oq, ok, ov, rq, rk = o_ap.qkv_fwd(x, pos, w, cfg, inv_freq)
    torch.testing.assert_close(oq, q.detach(), rtol=1e-5, atol=1e-5)
    torch.testing.assert_close(ok, k.detach(), rtol=1e-5, atol=1e-5)
    torch.testing.assert_close(ov, v.detach(), rtol=1e-5, atol=1e-5)
    torch.testing.assert_close(o_ap.o_fwd(resid, attn.detach(), w), out_ref.detach(), rtol=1e-5, atol=1e-5)
    # backward halves, fed with autograd's own gradients at the core's boundary
    g_o0 = randn(g, cfg.attn_dim, cfg.d_model, dtype=f32)
    d_attn, g_o = o_ap.o_bwd(dy, attn.detach(), w, g_o0)
    torch.testing.assert_close(d_attn.view(T, cfg.n_heads, cfg.head_dim), attn.grad, rtol=1e-4, atol=1e-5)
    torch.testing.assert_close(g_o, g_o0 + leaf["w_o"].grad, rtol=1e-4, atol=1e-5)
    dx, pg = o_ap.qkv_bwd(q.grad.clone(), k.grad.clone(), v.grad.clone(), x, pos, w, cfg, inv_freq, rq, rk)
    torch.testing.assert_close(dx, xx.grad, rtol=1e-4, atol=1e-5)
    for name, key in (("g_q", "w_q"), ("g_k", "w_k"), ("g_v", "w_v")):
        torch.testing.assert_close(pg[name], leaf[key].grad, rtol=1e-4, atol=1e-5)
    if bias:
        for name, key in (("g_b_q", "b_q"), ("g_b_k", "b_k"), ("g_b_v", "b_v")):
            torch.testing.assert_close(pg[name], leaf[key].grad, rtol=1e-4, atol=1e-5)
    if qk_norm:
        torch.testing.assert_close(pg["g_q_norm"], leaf["w_q_norm"].grad, rtol=1e-4, atol=1e-5)
        torch.testing.assert_close(pg["g_k_norm"], leaf["w_k_norm"].grad, rtol=1e-4, atol=1e-5)


def test_config_and_flops():
    from flextrain_amd.attention_proj import GQAAttentionProjections
    cfg = GQAProjectionConfig(d_model=4096, n_heads=32, n_kv_heads=8, head_dim=128)
    assert (cfg.attn_dim, cfg.kv_dim) == (4096, 1024)
    assert GQAAttentionProjections(cfg).projection_flops(10) == 2 * 10 * 4096 * (2 * 4096 + 2 * 1024)
    with pytest.raises(ValueError):
        GQAAttentionProjections(GQAProjectionConfig(d_model=64, n_heads=6, n_kv_heads=4, head_dim=8))
