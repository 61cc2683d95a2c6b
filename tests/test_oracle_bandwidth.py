"""Pins the CPU oracle for RMSNorm, RoPE, gated activations and AdamW against
independent statements of the same mathematics (library routines, autograd,
closed forms, invariants).  CPU only."""
import math

import pytest
import torch
import torch.nn.functional as F

from oracle import adamw as o_adamw
from oracle import glu as o_glu
from oracle import rmsnorm as o_norm
from oracle import rope as o_rope
from util import gen, randn


# ---------------------------------------------------------------- RMSNorm
def test_rmsnorm_fwd_matches_library_rms_norm():
    g = gen(1)
    x = randn(g, 64, 256, dtype=torch.float32)
    w = randn(g, 256, dtype=torch.float32, std=0.02, mean=1.0)
    y, rstd = o_norm.rmsnorm_fwd(x, w, eps=1e-5)
    torch.testing.assert_close(y, F.rms_norm(x, (256,), w, eps=1e-5), rtol=1e-6, atol=1e-6)
    torch.testing.assert_close(rstd[:, 0], 1.0 / torch.sqrt((x * x).mean(-1) + 1e-5), rtol=1e-6, atol=0)


def test_rmsnorm_fwd_constant_rows_closed_form():
    c, eps = 3.0, 1e-5
    x = torch.full((4, 128), c)
    w = torch.linspace(0.5, 1.5, 128)
    y, rstd = o_norm.rmsnorm_fwd(x, w, eps=eps)
    torch.testing.assert_close(y, (c / math.sqrt(c * c + eps)) * w.expand(4, 128), rtol=1e-6, atol=0)
    assert rstd.shape == (4, 1)


def test_rmsnorm_bf16_rounds_before_weight():
    # reference-held formula: (x.float()*rstd).to(dtype) * w   (bench/parity.py:112-115)
    g = gen(2)
    x = randn(g, 32, 512)
    w = randn(g, 512, std=0.02, mean=1.0)
    y, _ = o_norm.rmsnorm_fwd(x, w, eps=1e-5)
    xf = x.float()
    ref = (xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + 1e-5)).to(x.dtype) * w
    assert torch.equal(y, ref)


def test_rmsnorm_per_head_equals_reshaped_rows():
    g = gen(3)
    x = randn(g, 16, 4 * 64)
    w = randn(g, 64, std=0.02, mean=1.0)
    y, rstd = o_norm.rmsnorm_fwd(x, w, head_dim=64)
    y2, rstd2 = o_norm.rmsnorm_fwd(x.reshape(64, 64), w)
    assert torch.equal(y.reshape(64, 64), y2) and torch.equal(rstd.reshape(-1), rstd2.reshape(-1))
    assert torch.equal(o_norm.rmsnorm_fwd_recompute(x, w, rstd, head_dim=64), y)


@pytest.mark.parametrize("head_dim", [None, 32])
def test_rmsnorm_bwd_matches_autograd(head_dim):
    g = gen(4)
    T, D = 24, 128
    x = randn(g, T, D, dtype=torch.float64).requires_grad_()
    w = randn(g, D if head_dim is None else head_dim, dtype=torch.float64, std=0.1, mean=1.0).requires_grad_()
    dy = randn(g, T, D, dtype=torch.float64)
    n = D if head_dim is None else head_dim
    xr = x.reshape(-1, n)
    y = (xr * torch.rsqrt(xr.pow(2).mean(-1, keepdim=True) + 1e-5) * w).reshape(T, D)
    gx, gw = torch.autograd.grad(y, (x, w), dy)
    _, rstd = o_norm.rmsnorm_fwd(x.detach().float(), None, 1e-5, head_dim)
    dx, dw, yr = o_norm.rmsnorm_bwd(dy.float(), x.detach().float(), w.detach().float(), rstd, head_dim,
                                    recompute_output=True)
    torch.testing.assert_close(dx.double(), gx, rtol=1e-4, atol=1e-5)
    torch.testing.assert_close(dw.double(), gw, rtol=1e-4, atol=1e-4)
    torch.testing.assert_close(yr.double(), y.detach(), rtol=1e-5, atol=1e-5)


def test_rmsnorm_bwd_accumulates_and_row_identity():
    g = gen(5)
    x = randn(g, 8, 64, dtype=torch.float32)
    w = randn(g, 64, dtype=torch.float32, mean=1.0, std=0.1)
    dy = randn(g, 8, 64, dtype=torch.float32)
    old = randn(g, 8, 64, dtype=torch.float32)
    dw_old = randn(g, 64, dtype=torch.float32)
    eps = 0.5  # large on purpose: makes the eps-proportional identity below visible in fp32
    _, rstd = o_norm.rmsnorm_fwd(x, w, eps)
    dx, dw, _ = o_norm.rmsnorm_bwd(dy, x, w, rstd)
    dx2, dw2, _ = o_norm.rmsnorm_bwd(dy, x, w, rstd, dx_old=old, dw_old=dw_old)
    torch.testing.assert_close(dx2, old + dx)
    torch.testing.assert_close(dw2, dw_old + dw)
    # sum_d dx*x = dot * eps / (var + eps), dot = sum x_hat * dy * w
    var = (x * x).mean(-1)
    dot = ((x * rstd) * dy * w).sum(-1)
    torch.testing.assert_close((dx * x).sum(-1), dot[:] * eps / (var + eps), rtol=1e-3, atol=1e-5)


# ------------------------------------------------------------------- RoPE
def _reference_held_rope(x, pos, inv):
    # flextrain/bench/parity.py:118-139, written here through complex multiplication
    T, H, D = x.shape
    ang = pos.view(-1, 1, 1).float() * inv
    z = torch.view_as_complex(x.float().reshape(T, H, D // 2, 2).contiguous())
    return torch.view_as_real(z * torch.polar(torch.ones_like(ang), ang)).reshape(T, H, D).to(x.dtype)


def test_rope_matches_complex_rotation():
    g = gen(6)
    x = randn(g, 50, 3, 64, dtype=torch.float32)
    pos = torch.randint(0, 8192, (50, 1), generator=g, dtype=torch.int32)
    inv = o_rope.vanilla_inv_freq(64, 500000.0)
    y = o_rope.rope(x, pos, inv)
    # same inv_freq bits on both sides: at pos ~8000 one ulp of inv_freq moves the angle by ~5e-4
    torch.testing.assert_close(y, _reference_held_rope(x, pos, inv), rtol=1e-4, atol=1e-4)
    held = 500000.0 ** (-(2.0 * torch.arange(0, 32).float() / 64))  # bench/parity.py:126-127
    torch.testing.assert_close(inv, held, rtol=1e-6, atol=0)
    # inverse, isometry, pos 0
    torch.testing.assert_close(o_rope.rope(y, pos, inv, backward=True), x, rtol=1e-4, atol=1e-4)
    n_in = x.reshape(50, 3, 32, 2).norm(dim=-1)
    n_out = y.reshape(50, 3, 32, 2).norm(dim=-1)
    torch.testing.assert_close(n_in, n_out, rtol=1e-5, atol=1e-5)
    assert torch.equal(o_rope.rope(x, torch.zeros(50, 1, dtype=torch.int32), inv), x)


def test_rope_backward_is_vjp_of_forward():
    g = gen(7)
    x = randn(g, 9, 2, 16, dtype=torch.float64).requires_grad_()
    pos = torch.arange(9, dtype=torch.int32).view(9, 1) * 37
    inv = o_rope.vanilla_inv_freq(16, 10000.0)
    dy = randn(g, 9, 2, 16, dtype=torch.float64)
    T, H, D = x.shape
    ang = pos.view(-1, 1, 1).double() * inv.double()
    e, o = x[..., 0::2], x[..., 1::2]
    y = torch.stack((e * ang.cos() - o * ang.sin(), e * ang.sin() + o * ang.cos()), -1).reshape(T, H, D)
    (gx,) = torch.autograd.grad(y, x, dy)
    torch.testing.assert_close(o_rope.rope(dy.float(), pos, inv, backward=True).double(), gx, rtol=1e-5, atol=1e-5)


def test_rope_partial_leaves_tail():
    g = gen(8)
    x = randn(g, 5, 2, 32, dtype=torch.float32)
    pos = torch.arange(5, dtype=torch.int32).view(5, 1) + 3
    inv = o_rope.vanilla_inv_freq(8, 10000.0)
    y = o_rope.rope(x, pos, inv, rot_dim=8)
    assert torch.equal(y[..., 8:], x[..., 8:])
    torch.testing.assert_close(y[..., :8], o_rope.rope(x[..., :8].contiguous(), pos, inv))


# -------------------------------------------------------------------- GLU
def test_swiglu_matches_library_and_autograd():
    g = gen(9)
    x1 = randn(g, 40, 96, dtype=torch.float64).requires_grad_()
    x3 = randn(g, 40, 96, dtype=torch.float64).requires_grad_()
    d = randn(g, 40, 96, dtype=torch.float64)
    out = F.silu(x1) * x3
    g1, g3 = torch.autograd.grad(out, (x1, x3), d)
    torch.testing.assert_close(o_glu.swiglu_fwd(x1.detach().float(), x3.detach().float()).double(), out.detach(), rtol=1e-5, atol=1e-6)
    dx1, dx3, act = o_glu.swiglu_bwd(x1.detach().float(), x3.detach().float(), d.float(), faithful=False)
    torch.testing.assert_close(dx1.double(), g1, rtol=1e-5, atol=1e-5)
    torch.testing.assert_close(dx3.double(), g3, rtol=1e-5, atol=1e-5)
    torch.testing.assert_close(act.double(), out.detach(), rtol=1e-5, atol=1e-6)


def test_swiglu_bf16_matches_reference_held_formula():
    g = gen(10)
    x1, x3 = randn(g, 64, 128), randn(g, 64, 128)
    ref = F.silu(x1.float()).to(x1.dtype) * x3  # bench/parity.py:208 (one extra rounding)
    torch.testing.assert_close(o_glu.swiglu_fwd(x1, x3).float(), ref.float(), rtol=1e-2, atol=1e-2)
    d = randn(g, 64, 128)
    f1 = o_glu.swiglu_bwd(x1, x3, d, faithful=True)[0].float()
    f0 = o_glu.swiglu_bwd(x1, x3, d, faithful=False)[0].float()
    torch.testing.assert_close(f1, f0, rtol=1e-2, atol=1e-2)


def test_gelu_tanh_gated_matches_library_and_autograd():
    # tests/test_gelu_tanh_gated_kernel.py:57-60,82-89
    g = gen(11)
    x1 = randn(g, 32, 1152, dtype=torch.float64).requires_grad_()
    x3 = randn(g, 32, 1152, dtype=torch.float64).requires_grad_()
    d = randn(g, 32, 1152, dtype=torch.float64)
    out = F.gelu(x1, approximate="tanh") * x3
    g1, g3 = torch.autograd.grad(out, (x1, x3), d)
    a, b = x1.detach().float(), x3.detach().float()
    torch.testing.assert_close(o_glu.gelu_tanh_gated_fwd(a, b).double(), out.detach(), rtol=1e-5, atol=1e-6)
    dx1, dx3, act = o_glu.gelu_tanh_gated_bwd(a, b, d.float())
    torch.testing.assert_close(dx1.double(), g1, rtol=1e-4, atol=1e-5)
    torch.testing.assert_close(dx3.double(), g3, rtol=1e-4, atol=1e-5)
    torch.testing.assert_close(act.double(), out.detach(), rtol=1e-5, atol=1e-6)


def test_silu_bwd_matches_autograd():
    g = gen(21)
    z = randn(g, 64, 33, std=3.0).double().requires_grad_()
    d = randn(g, 64, 33).double()
    (gz,) = torch.autograd.grad((F.silu(z) * d).sum(), z)
    torch.testing.assert_close(o_glu.silu_bwd(z.detach().float(), d.float()).double(), gz, rtol=1e-5, atol=1e-6)
    assert o_glu.silu_bwd(torch.zeros(4), torch.ones(4)).tolist() == [0.5] * 4      # silu'(0) = 1/2


def test_embedding_bwd_matches_autograd_and_loop():
    g = gen(22)
    T, D, V = 40, 6, 7
    go = randn(g, T, D, dtype=torch.float32)
    idx = torch.randint(0, V, (T,), generator=g)
    gw0 = randn(g, V, D, dtype=torch.float32)
    w = torch.zeros(V, D, requires_grad=True)
    (auto,) = torch.autograd.grad((F.embedding(idx, w) * go).sum(), w)
    out = o_glu.embedding_bwd(go, idx.int(), gw0, scale=0.25)
    torch.testing.assert_close(out, gw0 + 0.25 * auto, rtol=1e-6, atol=1e-6)
    loop = gw0.clone()
    for t in range(T):
        loop[idx[t]] += 0.25 * go[t]
    torch.testing.assert_close(out, loop, rtol=1e-5, atol=1e-6)
    assert o_glu.embedding_bwd(go, idx, gw0).dtype == gw0.dtype


# ------------------------------------------------------------------ AdamW
def test_adamw_matches_torch_optim_over_steps():
    g = gen(12)
    n = 4096
    p0 = randn(g, n, dtype=torch.float32, std=0.02)
    hp = dict(lr=3e-5, betas=(0.9, 0.95), eps=1e-8, weight_decay=0.1)
    tp = torch.nn.Parameter(p0.clone())
    opt = torch.optim.AdamW([tp], **hp)
    p, m, v = p0.clone(), torch.zeros(n), torch.zeros(n)
    for step in range(1, 5):
        grad = randn(g, n, dtype=torch.bfloat16, std=1e-3)
        tp.grad = grad.float()
        opt.step()
        p, m, v, pb = o_adamw.adamw_step(p, grad, m, v, lr=3e-5, beta1=0.9, beta2=0.95, eps=1e-8,
                                         weight_decay=0.1, step=step)
        torch.testing.assert_close(p, tp.detach(), rtol=1e-5, atol=1e-8)
        st = opt.state[tp]
        torch.testing.assert_close(m, st["exp_avg"], rtol=1e-5, atol=1e-10)
        torch.testing.assert_close(v, st["exp_avg_sq"], rtol=1e-5, atol=1e-14)
        assert torch.equal(pb, p.to(torch.bfloat16))


def test_adamw_step1_closed_form():
    g = gen(13)
    p0 = randn(g, 1000, dtype=torch.float32, std=0.02)
    grad = randn(g, 1000, dtype=torch.float32, std=1e-3)
    lr, wd, eps = 3e-5, 0.1, 1e-8
    p, m, v, _ = o_adamw.adamw_step(p0, grad, torch.zeros(1000), torch.zeros(1000), lr=lr, beta1=0.9,
                                    beta2=0.95, eps=eps, weight_decay=wd, step=1)
    torch.testing.assert_close(p, p0 * (1 - lr * wd) - lr * grad / (grad.abs() + eps), rtol=1e-5, atol=1e-9)
    torch.testing.assert_close(m, 0.1 * grad, rtol=1e-5, atol=0)
    torch.testing.assert_close(v, 0.05 * grad * grad, rtol=1e-4, atol=0)


def test_adamw_step_zero_is_step_one():
    p0 = torch.ones(8)
    g = torch.full((8,), 0.5)
    a = o_adamw.adamw_step(p0, g, torch.zeros(8), torch.zeros(8), step=0)
    b = o_adamw.adamw_step(p0, g, torch.zeros(8), torch.zeros(8), step=1)
    assert all(torch.equal(x, y) for x, y in zip(a, b))
