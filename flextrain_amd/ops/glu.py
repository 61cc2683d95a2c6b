"""Gated activations behind the reference signatures
(flextrain/ops/_kernels/swiglu.py:103-182,
flextrain/ops/_kernels/gelu_tanh_gated.py:148-214).  ``x1`` is the gate,
``x3`` the up/value projection; non-contiguous inputs are copied first, as in
the reference."""
from __future__ import annotations

import torch

from .._lib import ACT_GELU_TANH, ACT_SILU, check, dtype_enum, lib, ptr, stream_ptr


def _fwd(x1, x3, out, act, name):
    assert x1.shape == x3.shape
    assert x1.is_cuda and x3.is_cuda
    if x1.dtype != x3.dtype:
        raise TypeError(f"{name}: x1 and x3 must share a dtype")
    if not x1.is_contiguous():
        x1 = x1.contiguous()
    if not x3.is_contiguous():
        x3 = x3.contiguous()
    if out is None:
        out = torch.empty_like(x1)
    elif out.numel() != x1.numel() or not out.is_contiguous():
        raise ValueError(f"{name}: out must be contiguous with {x1.numel()} elements")
    rc = lib().fx_glu_fwd(ptr(x1), ptr(x3), ptr(out), x1.numel(), dtype_enum(x1.dtype),
                          dtype_enum(out.dtype), act, stream_ptr(x1.device))
    check(rc, name)
    return out


def _bwd(x1, x3, dout, dx1, dx3, store_activations, activations, act, name):
    assert x1.shape == x3.shape == dout.shape
    assert x1.is_cuda and x3.is_cuda and dout.is_cuda
    if not (x1.dtype == x3.dtype == dout.dtype):
        raise TypeError(f"{name}: x1, x3 and dout must share a dtype")
    if not x1.is_contiguous():
        x1 = x1.contiguous()
    if not x3.is_contiguous():
        x3 = x3.contiguous()
    if not dout.is_contiguous():
        dout = dout.contiguous()
    if dx1 is None:
        dx1 = torch.empty_like(x1)
    if dx3 is None:
        dx3 = torch.empty_like(x3)
    if store_activations and activations is None:
        activations = torch.empty_like(x1)
    act_buf = activations if store_activations else None
    for t, nm in ((dx1, "dx1"), (dx3, "dx3"), (act_buf, "activations")):
        if t is not None and (t.numel() != x1.numel() or not t.is_contiguous() or t.dtype != x1.dtype):
            raise ValueError(f"{name}: {nm} must be contiguous, dtype {x1.dtype}, {x1.numel()} elements")
    rc = lib().fx_glu_bwd(ptr(x1), ptr(x3), ptr(dout), ptr(dx1), ptr(dx3), ptr(act_buf), x1.numel(),
                          dtype_enum(x1.dtype), act, stream_ptr(x1.device))
    check(rc, name)
    if store_activations:
        return dx1, dx3, activations
    return dx1, dx3


def flextrain_swiglu_fwd(x1, x3, out=None):
    """``silu(x1) * x3``; flextrain/ops/_kernels/swiglu.py:103-133."""
    return _fwd(x1, x3, out, ACT_SILU, "flextrain_swiglu_fwd")


def flextrain_swiglu_bwd(x1, x3, dout, dx1=None, dx3=None, store_activations=False, activations=None):
    """``(dx1, dx3[, act])``; flextrain/ops/_kernels/swiglu.py:136-182."""
    return _bwd(x1, x3, dout, dx1, dx3, store_activations, activations, ACT_SILU, "flextrain_swiglu_bwd")


def flextrain_gelu_tanh_gated_fwd(x1, x3, out=None):
    """``gelu_tanh(x1) * x3``; flextrain/ops/_kernels/gelu_tanh_gated.py:148-170."""
    return _fwd(x1, x3, out, ACT_GELU_TANH, "flextrain_gelu_tanh_gated_fwd")


def flextrain_gelu_tanh_gated_bwd(x1, x3, dout, dx1=None, dx3=None, store_activations=False,
                                  activations=None):
    """``(dx1, dx3[, act])``; flextrain/ops/_kernels/gelu_tanh_gated.py:173-214."""
    return _bwd(x1, x3, dout, dx1, dx3, store_activations, activations, ACT_GELU_TANH,
                "flextrain_gelu_tanh_gated_bwd")
