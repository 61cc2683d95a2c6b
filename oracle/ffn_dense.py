"""CPU restatement of the dense gated FFN block (flextrain/nn/blocks/ffn_dense.py:114-277).

Test infrastructure only.  Every tensor the reference stores between kernels in the compute dtype
(x1, x3, the gated activation, dx_up_act, dx1_up, dx3_up) is rounded to that dtype here as well;
GEMMs accumulate in fp32.
"""
import torch

from . import glu


def _mm(a, b, dtype):
    return (a.float() @ b.float()).to(dtype)


def ffn_fwd(h, w1, w3, w2, resid, activation="silu"):
    """Returns (out, x1, x3): x1 = h W1, x3 = h W3, out = resid + act(x1, x3) W2
    (ffn_dense.py:130-154)."""
    dt = h.dtype
    x1, x3 = _mm(h, w1, dt), _mm(h, w3, dt)
    act = glu.swiglu_fwd(x1, x3) if activation == "silu" else glu.gelu_tanh_gated_fwd(x1, x3)
    out = (resid.float() + act.float() @ w2.float()).to(dt)
    return out, x1, x3


def ffn_bwd(dy, h, x1, x3, w1, w3, w2, g1, g2, g3, activation="silu"):
    """Returns (dx_ffn_norm_up, g1', g2', g3') with the weight gradients accumulated onto the given
    ones (ffn_dense.py:193-267): dx_up_act = dy W2^T; gated-activation backward; g2 += act^T dy;
    dx = dx1 W1^T + dx3 W3^T (the second product added onto the rounded first); g1 += h^T dx1;
    g3 += h^T dx3."""
    dt = dy.dtype
    dx_up_act = _mm(dy, w2.t(), dt)
    bwd = glu.swiglu_bwd if activation == "silu" else glu.gelu_tanh_gated_bwd
    dx1, dx3, act = bwd(x1, x3, dx_up_act)
    g2n = (g2.float() + act.float().t() @ dy.float()).to(g2.dtype)
    dx = _mm(dx1, w1.t(), dt)
    dx = (dx.float() + dx3.float() @ w3.float().t()).to(dt)
    g1n = (g1.float() + h.float().t() @ dx1.float()).to(g1.dtype)
    g3n = (g3.float() + h.float().t() @ dx3.float()).to(g3.dtype)
    return dx, g1n, g2n, g3n
