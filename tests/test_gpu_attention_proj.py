"""Attention block around its core (MFMA dispatcher GEMMs, per-head RMSNorm and RoPE kernels, residual
in the output projection's epilogue) against the CPU oracle: bf16 tensors at rtol = atol = 1e-2
relative to each tensor's scale, fp32 norm-weight gradients at rtol 1e-2 of their scale as well
(they are sums of bf16-rounded products)."""
from types import SimpleNamespace

import pytest
import torch

from flextrain_amd.attention_proj import GQAAttentionProjections, GQAProjectionConfig
from oracle import attention_proj as o_ap
from oracle import rope as o_rope
from util import gen, randn

pytestmark = pytest.mark.gpu
bf = torch.bfloat16


def _close(a, e, what):
    a, e = a.float().cpu(), e.float()
    assert a.shape == e.shape, f"{what}: {tuple(a.shape)} vs {tuple(e.shape)}"
    scale = max(1.0, float(e.abs().max()))
    torch.testing.assert_close(a, e, rtol=1e-2, atol=1e-2 * scale, msg=lambda m: f"{what}: {m}")


def _setup(g, cfg, T, gdt):
    w = {"w_q": randn(g, cfg.d_model, cfg.attn_dim, std=cfg.d_model ** -0.5), "w_k": randn(g, cfg.d_model, cfg.kv_dim, std=cfg.d_model ** -0.5),
         "w_v": randn(g, cfg.d_model, cfg.kv_dim, std=cfg.d_model ** -0.5), "w_o": randn(g, cfg.attn_dim, cfg.d_model, std=cfg.attn_dim ** -0.5)}
    g0 = {"g_q": randn(g, cfg.d_model, cfg.attn_dim, dtype=gdt), "g_k": randn(g, cfg.d_model, cfg.kv_dim, dtype=gdt),
          "g_v": randn(g, cfg.d_model, cfg.kv_dim, dtype=gdt), "g_o": randn(g, cfg.attn_dim, cfg.d_model, dtype=gdt)}
    if cfg.qkv_bias:
        w.update(b_q=randn(g, cfg.attn_dim, std=0.5), b_k=randn(g, cfg.kv_dim, std=0.5), b_v=randn(g, cfg.kv_dim, std=0.5))
        g0.update(g_b_q=randn(g, cfg.attn_dim, dtype=gdt), g_b_k=randn(g, cfg.kv_dim, dtype=gdt), g_b_v=randn(g, cfg.kv_dim, dtype=gdt))
    if cfg.qk_norm:
        w.update(w_q_norm=randn(g, cfg.head_dim, dtype=torch.float32, mean=1.0, std=0.1),
                 w_k_norm=randn(g, cfg.head_dim, dtype=torch.float32, mean=1.0, std=0.1))
        g0.update(g_q_norm=randn(g, cfg.head_dim, dtype=torch.float32), g_k_norm=randn(g, cfg.head_dim, dtype=torch.float32))
    return w, g0


def _slot(cfg, T, dev):
    return SimpleNamespace(
        xq=torch.empty(T, cfg.n_heads, cfg.head_dim, dtype=bf, device=dev), xk=torch.empty(T, cfg.n_kv_heads, cfg.head_dim, dtype=bf, device=dev),
        xv=torch.empty(T, cfg.n_kv_heads, cfg.head_dim, dtype=bf, device=dev), attn_result=torch.empty(T, cfg.n_heads, cfg.head_dim, dtype=bf, device=dev),
        xo=torch.empty(T, cfg.d_model, dtype=bf, device=dev), q_norm_rstd=torch.empty(T, cfg.n_heads, dtype=torch.float32, device=dev),
        k_norm_rstd=torch.empty(T, cfg.n_kv_heads, dtype=torch.float32, device=dev), aux={})


@pytest.mark.parametrize("T,d,H,Hkv,D", [(256, 256, 8, 2, 64), (200, 136, 6, 3, 32)])
@pytest.mark.parametrize("bias,qk_norm", [(False, False), (True, False), (False, True)])
@pytest.mark.parametrize("gdt", [bf, torch.float32])
def test_halves_against_oracle(dev, T, d, H, Hkv, D, bias, qk_norm, gdt):
    g = gen(T + d + 7 * bias + 3 * qk_norm)
    cfg = GQAProjectionConfig(d_model=d, n_heads=H, n_kv_heads=Hkv, head_dim=D, rope_theta=500000.0, qkv_bias=bias, qk_norm=qk_norm)
    w, g0 = _setup(g, cfg, T, gdt)
    x, resid, dy = randn(g, T, d), randn(g, T, d), randn(g, T, d)
    attn = randn(g, T, H, D)
    dq, dk, dv = randn(g, T, H, D), randn(g, T, Hkv, D), randn(g, T, Hkv, D)
    pos = torch.arange(5, 5 + T, dtype=torch.int32)
    inv_freq = o_rope.vanilla_inv_freq(D, cfg.rope_theta)

    q_ref, k_ref, v_ref, rq, rk = o_ap.qkv_fwd(x, pos, w, cfg, inv_freq)
    out_ref = o_ap.o_fwd(resid, attn, w)
    dattn_ref, g_o_ref = o_ap.o_bwd(dy, attn, w, g0["g_o"])
    dx_ref, pg = o_ap.qkv_bwd(dq, dk, dv, x, pos, w, cfg, inv_freq, rq, rk)

    blk = GQAAttentionProjections(cfg)
    W = {k: v.to(dev) for k, v in w.items()}
    G = {k: v.to(dev) for k, v in g0.items()}
    slot = _slot(cfg, T, dev)
    xd, posd = x.to(dev), pos.to(dev).view(T, 1)
    blk.fwd_qkv(xd, posd, W, slot)
    _close(slot.xq, q_ref, "xq"), _close(slot.xk, k_ref, "xk"), _close(slot.xv, v_ref, "xv")
    if qk_norm:
        _close(slot.q_norm_rstd, rq, "rstd_q")
    # Q rebuilt from the saved rstd is the same Q, bit for bit
    q_saved = slot.xq.clone()
    slot.xq.zero_()
    blk.fwd_recompute_q(xd, posd, W, slot)
    assert torch.equal(slot.xq, q_saved)

    slot.attn_result.copy_(attn.to(dev))
    out = blk.fwd_o(resid.to(dev), W, slot)
    assert out is slot.xo
    _close(out, out_ref, "xo")

    dattn = blk.bwd_o(dy.to(dev), W, G, slot)
    _close(dattn.reshape(T, -1), dattn_ref, "dx_up_attn"), _close(G["g_o"], g_o_ref, "g_o")

    dx = blk.bwd_qkv(dq.to(dev), dk.to(dev), dv.to(dev), posd, W, G, slot, attn_norm_output=xd)
    assert set(slot.aux) == {"bwd_dq", "bwd_local_dk", "bwd_local_dv"}
    blk.bwd_accumulate_qkv_grads(xd, G, slot)
    assert not slot.aux
    _close(dx, dx_ref, "dx")
    for name in ("g_q", "g_k", "g_v"):
        _close(G[name], g0[name].float() + pg[name], name)
    if bias:
        for name in ("g_b_q", "g_b_k", "g_b_v"):
            _close(G[name], g0[name].float() + pg[name], name)
    if qk_norm:
        for name in ("g_q_norm", "g_k_norm"):
            _close(G[name], g0[name] + pg[name], name)


def test_whole_block_with_a_dense_causal_core(dev):
    """fwd / bwd with the core supplied by the caller (plain torch attention here)."""
    import math
    g = gen(41)
    T = 192
    cfg = GQAProjectionConfig(d_model=128, n_heads=4, n_kv_heads=2, head_dim=32, rope_theta=10000.0)
    w, g0 = _setup(g, cfg, T, bf)
    x, resid, dy = randn(g, T, cfg.d_model), randn(g, T, cfg.d_model), randn(g, T, cfg.d_model)
    pos = torch.arange(T, dtype=torch.int32)
    inv_freq = o_rope.vanilla_inv_freq(cfg.head_dim, cfg.rope_theta)

    def core(q, k, v):
        rep = q.shape[1] // k.shape[1]
        kk, vv = k.float().repeat_interleave(rep, dim=1), v.float().repeat_interleave(rep, dim=1)
        s = torch.einsum("thd,shd->hts", q.float(), kk) / math.sqrt(q.shape[-1])
        s = s.masked_fill(torch.triu(torch.ones(T, T, dtype=torch.bool, device=q.device), 1), float("-inf"))
        return torch.einsum("hts,shd->thd", s.softmax(-1), vv)

    def core_fwd(q, k, v, out):
        out.copy_(core(q, k, v))

    def core_bwd(d_out, q, k, v, out):
        ql, kl, vl = (t.detach().float().requires_grad_() for t in (q, k, v))
        core(ql, kl, vl).backward(d_out.float())
        return ql.grad.to(q.dtype), kl.grad.to(k.dtype), vl.grad.to(v.dtype)

    # oracle side: the same core on the CPU between the oracle's halves
    q_ref, k_ref, v_ref, _, _ = o_ap.qkv_fwd(x, pos, w, cfg, inv_freq)
    attn_ref = core(q_ref, k_ref, v_ref).to(bf)
    out_ref = o_ap.o_fwd(resid, attn_ref, w)
    dattn_ref, g_o_ref = o_ap.o_bwd(dy, attn_ref, w, g0["g_o"])
    dq_r, dk_r, dv_r = core_bwd(dattn_ref.view(T, cfg.n_heads, cfg.head_dim), q_ref, k_ref, v_ref, attn_ref)
    dx_ref, pg = o_ap.qkv_bwd(dq_r, dk_r, dv_r, x, pos, w, cfg, inv_freq)

    blk = GQAAttentionProjections(cfg)
    W = {k: v.to(dev) for k, v in w.items()}
    G = {k: v.to(dev) for k, v in g0.items()}
    slot = _slot(cfg, T, dev)
    xd, posd = x.to(dev), pos.to(dev).view(T, 1)
    out = blk.fwd(resid.to(dev), xd, posd, W, slot, core_fwd)
    _close(out, out_ref, "xo")
    dx = blk.bwd(dy.to(dev), posd, W, G, slot, xd, core_bwd)
    blk.bwd_accumulate_qkv_grads(xd, G, slot)
    _close(dx, dx_ref, "dx"), _close(G["g_o"], g_o_ref, "g_o")
    for name in ("g_q", "g_k", "g_v"):
        _close(G[name], g0[name].float() + pg[name], name)


def test_skip_grads_hands_back_operands(dev):
    g = gen(5)
    T = 128
    cfg = GQAProjectionConfig(d_model=64, n_heads=4, n_kv_heads=2, head_dim=16)
    w, g0 = _setup(g, cfg, T, bf)
    W = {k: v.to(dev) for k, v in w.items()}
    G = {k: v.to(dev) for k, v in g0.items()}
    before = {k: v.clone() for k, v in G.items()}
    slot = _slot(cfg, T, dev)
    slot.attn_result.copy_(randn(g, T, cfg.n_heads, cfg.head_dim).to(dev))
    blk = GQAAttentionProjections(cfg)
    x, dy = randn(g, T, cfg.d_model).to(dev), randn(g, T, cfg.d_model).to(dev)
    pos = torch.arange(T, dtype=torch.int32, device=dev).view(T, 1)
    cap = {}
    blk.bwd_o(dy, W, G, slot, skip_grads=frozenset({"g_o"}), capture_xy=cap)
    assert torch.equal(G["g_o"], before["g_o"]) and torch.equal(cap["g_o"][1], dy)
    blk.bwd_qkv(randn(g, T, cfg.n_heads, cfg.head_dim).to(dev), randn(g, T, cfg.n_kv_heads, cfg.head_dim).to(dev),
                randn(g, T, cfg.n_kv_heads, cfg.head_dim).to(dev), pos, W, G, slot)
    dq_kept = slot.aux["bwd_dq"]
    blk.bwd_accumulate_qkv_grads(x, G, slot, skip_grads=frozenset({"g_q", "g_k"}), capture_xy=cap)
    assert torch.equal(G["g_q"], before["g_q"]) and torch.equal(G["g_k"], before["g_k"])
    assert not torch.equal(G["g_v"], before["g_v"])
    assert cap["g_q"][0] is x and cap["g_q"][1] is dq_kept
    with pytest.raises(ValueError):
        GQAAttentionProjections(GQAProjectionConfig(d_model=64, n_heads=4, n_kv_heads=2, head_dim=16, qk_norm=True)).bwd_qkv(
            randn(g, T, 4, 16).to(dev), randn(g, T, 2, 16).to(dev), randn(g, T, 2, 16).to(dev), pos,
            dict(W, w_q_norm=torch.ones(16, device=dev), w_k_norm=torch.ones(16, device=dev)), G, slot)


class _MatmulOnly:
    """A dispatcher with the reference's surface only (``matmul``)."""

    def __init__(self):
        from flextrain_amd.matmul_dispatcher import CublasLtDispatcher
        self._d = CublasLtDispatcher()
        self.calls = 0

    def matmul(self, stream_ptr, A, B, C=None, D=None, alpha=1.0, beta=0.0):
        self.calls += 1
        return self._d.matmul(stream_ptr, A, B, C=C, D=D, alpha=alpha, beta=beta)


def test_block_over_a_dispatcher_without_fused_launches(dev):
    """The one-launch forms (key / value projections and weight gradients, the summed input gradient) are
    optional: over a dispatcher that only has ``matmul`` the block issues the reference's 12 calls and
    gives the same results within rounding."""
    g = gen(23)
    T, d, H, Hkv, D = 256, 256, 8, 2, 64
    cfg = GQAProjectionConfig(d_model=d, n_heads=H, n_kv_heads=Hkv, head_dim=D, rope_theta=10000.0)
    w, _ = _setup(g, cfg, T, bf)
    x, resid, dy = randn(g, T, d), randn(g, T, d), randn(g, T, d)
    attn = randn(g, T, H, D)
    dq, dk, dv = randn(g, T, H, D), randn(g, T, Hkv, D), randn(g, T, Hkv, D)
    pos = torch.arange(T, dtype=torch.int32).view(T, 1)
    results = []
    for disp in (None, _MatmulOnly()):
        blk = GQAAttentionProjections(cfg, dispatcher=disp)
        W = {k: v.to(dev) for k, v in w.items()}
        G = {"g_" + k: torch.zeros_like(W["w_" + k]) for k in "qkvo"}
        slot = _slot(cfg, T, dev)
        blk.fwd_qkv(x.to(dev), pos.to(dev), W, slot)
        slot.attn_result.copy_(attn.to(dev))
        out = blk.fwd_o(resid.to(dev), W, slot)
        dattn = blk.bwd_o(dy.to(dev), W, G, slot)
        dx = blk.bwd_qkv(dq.to(dev), dk.to(dev), dv.to(dev), pos.to(dev), W, G, slot, attn_norm_output=x.to(dev))
        blk.bwd_accumulate_qkv_grads(x.to(dev), G, slot)
        results.append((slot.xq, slot.xk, slot.xv, out, dattn, dx, G["g_q"], G["g_k"], G["g_v"], G["g_o"]))
        if disp is not None:
            assert disp.calls == 12
    for name, a, b in zip(("xq", "xk", "xv", "xo", "dattn", "dx", "g_q", "g_k", "g_v", "g_o"), *results):
        _close(b.reshape(a.shape), a.float().cpu(), name)
