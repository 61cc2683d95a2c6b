"""The dense-FFN oracle against torch.autograd through the textbook formula (fp32: no rounding
between the steps, so the comparison is tight)."""
import pytest
import torch
import torch.nn.functional as F

from oracle import ffn_dense as o_ffn
from util import gen, randn


@pytest.mark.parametrize("activation", ["silu", "gelu_tanh"])
def test_ffn_oracle_matches_autograd(activation):
    g = gen(31)
    T, d, f = 24, 16, 40
    f32 = torch.float32
    h, resid, dy = (randn(g, T, d, dtype=f32) for _ in range(3))
    w1, w3 = (randn(g, d, f, dtype=f32, std=0.3).requires_grad_() for _ in range(2))
    w2 = randn(g, f, d, dtype=f32, std=0.3).requires_grad_()
    hh = h.clone().requires_grad_()
    gate = F.silu(hh @ w1) if activation == "silu" else F.gelu(hh @ w1, approximate="tanh")
    out_ref = resid + (gate * (hh @ w3)) @ w2
    gh, gw1, gw3, gw2 = torch.autograd.grad((out_ref * dy).sum(), [hh, w1, w3, w2])

    out, x1, x3 = o_ffn.ffn_fwd(h, w1.detach(), w3.detach(), w2.detach(), resid, activation)
    torch.testing.assert_close(out, out_ref.detach(), rtol=1e-5, atol=1e-5)
    g0 = [randn(g, *w.shape, dtype=f32) for w in (w1, w2, w3)]
    dx, g1, g2, g3 = o_ffn.ffn_bwd(dy, h, x1, x3, w1.detach(), w3.detach(), w2.detach(), g0[0], g0[1], g0[2], activation)
    torch.testing.assert_close(dx, gh, rtol=1e-4, atol=1e-5)
    torch.testing.assert_close(g1, g0[0] + gw1, rtol=1e-4, atol=1e-5)
    torch.testing.assert_close(g2, g0[1] + gw2, rtol=1e-4, atol=1e-5)
    torch.testing.assert_close(g3, g0[2] + gw3, rtol=1e-4, atol=1e-5)


def test_compute_cost_counts_three_gemms():
    from flextrain_amd.ffn_dense import SwiGLUConfig, SwiGLUFFN
    blk = SwiGLUFFN(SwiGLUConfig(d_model=8, expert_dim=20))
    c = blk.compute_cost([5, 7], max_tier=3)
    assert c.total_fwd_flops == 2 * 12 * 8 * 20 * 3
    assert c.avoided_recompute_flops == (0, 0, 0, 2 * 12 * 8 * 20 * 2)
    assert blk.compute_cost([5], max_tier=2).avoided_recompute_flops == (0, 0, 0)
    with pytest.raises(ValueError):
        SwiGLUFFN(SwiGLUConfig(d_model=8, expert_dim=20, activation="relu"))
