"""Pair-interleaved rotary embedding oracle (CPU, fp32).  Test infrastructure —
see oracle/__init__.py.

Restates flextrain/ops/_kernels/rope.py:30-68 (forward) and :104-140
(backward): angle = float(pos) * inv_freq[i] in fp32; even/odd channels are the
real/imaginary parts; the result is rounded once to the tensor dtype.
``rot_dim`` < D leaves the tail channels untouched
(flextrain/ops/_kernels/rope_partial.py:52-76).
"""
from __future__ import annotations

import torch


def vanilla_inv_freq(rot_dim, theta):
    """flextrain/ops/_kernels/rope.py:174-177."""
    expo = torch.arange(0, rot_dim // 2, dtype=torch.float32) * 2.0 / rot_dim
    return 1.0 / (float(theta) ** expo)


def rope(x, pos, inv_freq, backward=False, rot_dim=None):
    """x (T,H,D) any float dtype; pos integer (T,) or (T,1); returns a new tensor."""
    T, H, D = x.shape
    rd = D if rot_dim is None else rot_dim
    ang = pos.reshape(T, -1)[:, 0].to(torch.float32).view(T, 1, 1) * inv_freq.float().view(1, 1, rd // 2)
    c, s = torch.cos(ang), torch.sin(ang)
    if backward:
        s = -s
    xf = x.float()
    e, o = xf[..., 0:rd:2], xf[..., 1:rd:2]
    out = xf.clone()
    out[..., 0:rd:2] = e * c - o * s
    out[..., 1:rd:2] = e * s + o * c
    return out.to(x.dtype)
