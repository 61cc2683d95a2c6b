"""Gated-activation oracle (CPU, fp32).  Test infrastructure — see
oracle/__init__.py.

``faithful=True`` keeps the one storage-dtype rounding the reference SwiGLU
backward has (dout*x3 is a bf16*bf16 product, flextrain/ops/_kernels/swiglu.py:92);
``faithful=False`` is the textbook fp32 formula.  Forward: swiglu.py:34-39,
gelu_tanh_gated.py:70-78; backward: swiglu.py:75-92, gelu_tanh_gated.py:111-137.
"""
from __future__ import annotations

import torch

_C = 0.7978845608028654
_A = 0.044715


def swiglu_fwd(x1, x3):
    a = x1.float()
    return (a * torch.sigmoid(a) * x3.float()).to(x1.dtype)


def swiglu_bwd(x1, x3, dout, faithful=True):
    """-> (dx1, dx3, act) in x1.dtype."""
    a, b, d = x1.float(), x3.float(), dout.float()
    s = torch.sigmoid(a)
    silu = a * s
    dx3 = d * silu
    db = (dout * x3).float() if faithful else d * b
    dx1 = db * (s * (1.0 + a * (1.0 - s)))
    return dx1.to(x1.dtype), dx3.to(x1.dtype), (silu * b).to(x1.dtype)


def _gelu_parts(a):
    u = _C * (a + _A * a * a * a)
    th = torch.tanh(u)
    return th, 0.5 * a * (1.0 + th)


def gelu_tanh_gated_fwd(x1, x3):
    _, g = _gelu_parts(x1.float())
    return (g * x3.float()).to(x1.dtype)


def gelu_tanh_gated_bwd(x1, x3, dout):
    a, b, d = x1.float(), x3.float(), dout.float()
    th, g = _gelu_parts(a)
    du = _C * (1.0 + 3.0 * _A * a * a)
    dg = 0.5 * (1.0 + th) + 0.5 * a * (1.0 - th * th) * du
    return (d * b * dg).to(x1.dtype), (d * g).to(x1.dtype), (g * b).to(x1.dtype)


def silu_bwd(z, dout):
    """din = dout * s * (1 + z * (1 - s)), s = sigmoid(z), in fp32, stored in z.dtype
    (flextrain/ops/_kernels/silu_bwd.py:26-35)."""
    zf, df = z.float(), dout.float()
    s = torch.sigmoid(zf)
    return (df * (s * (1.0 + zf * (1.0 - s)))).to(z.dtype)


def embedding_bwd(grad_output, indices, grad_weight, scale=1.0):
    """grad_weight[token] += scale * (fp32 sum of the grad_output rows of that token), stored in
    grad_weight.dtype (flextrain/ops/_kernels/embed.py:5-122).  Returns a new tensor."""
    acc = torch.zeros(grad_weight.shape, dtype=torch.float32)
    acc.index_add_(0, indices.long(), grad_output.float())
    return (grad_weight.float() + acc * scale).to(grad_weight.dtype)
