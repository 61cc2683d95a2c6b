"""RMSNorm oracle (CPU, fp32).  Test infrastructure — see oracle/__init__.py.

Restates flextrain/ops/_kernels/rmsnorm.py: forward :62-91 (x*rstd is rounded
to the input dtype before the weight multiply), recompute :134-155, backward dx
:224-274 (x_hat and dy*w stay fp32; y re-materialised as fp32 x_hat*w) and dW
:295-309 (sum over rows of UNSCALED dy times x_hat).
"""
from __future__ import annotations

import torch


def _rows(x, head_dim):
    T, D = x.shape
    n = D if head_dim is None else head_dim
    return x.reshape(-1, n), n


def rmsnorm_fwd(x, w=None, eps=1e-5, head_dim=None):
    """-> (y in x.dtype, rstd fp32 (T, H))."""
    T, D = x.shape
    xr, n = _rows(x, head_dim)
    xf = xr.float()
    var = (xf * xf).sum(-1, keepdim=True) / n
    rstd = torch.rsqrt(var + eps)
    xn = (xf * rstd).to(x.dtype)
    y = xn.float() * w.float() if w is not None else xn.float()
    return y.to(x.dtype).reshape(T, D), rstd.reshape(T, D // n)


def rmsnorm_fwd_recompute(x, w, rstd, head_dim=None):
    T, D = x.shape
    xr, n = _rows(x, head_dim)
    xn = (xr.float() * rstd.reshape(-1, 1).float()).to(x.dtype)
    y = xn.float() * w.float() if w is not None else xn.float()
    return y.to(x.dtype).reshape(T, D)


def rmsnorm_bwd(dy, x, w, rstd, head_dim=None, dx_old=None, dw_old=None, recompute_output=False):
    """-> (dx in x.dtype, dw fp32 or None, y or None)."""
    T, D = x.shape
    xr, n = _rows(x, head_dim)
    dyr, _ = _rows(dy, head_dim)
    xh = xr.float() * rstd.reshape(-1, 1).float()
    dys = dyr.float() * w.float() if w is not None else dyr.float()
    k = (xh * dys).sum(-1, keepdim=True) / n
    dx = rstd.reshape(-1, 1).float() * (dys - xh * k)
    dx = dx.reshape(T, D)
    if dx_old is not None:
        dx = dx_old.float() + dx
    dw = None
    if w is not None:
        dw = (dyr.float() * xh).sum(0)
        if dw_old is not None:
            dw = dw_old.float() + dw
    y = None
    if recompute_output:
        y = (xh * w.float() if w is not None else xh).to(x.dtype).reshape(T, D)
    return dx.to(x.dtype), dw, y
