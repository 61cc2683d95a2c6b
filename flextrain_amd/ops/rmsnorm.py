"""RMSNorm forward / recompute / backward behind the reference signatures
(flextrain/ops/_kernels/rmsnorm.py:419-832).

Same argument names, shape/contiguity errors, return tuples and in-place
rules: ``output`` may be ``X``; a caller-provided ``dX``/``dW`` is accumulated
into, a missing one is allocated and overwritten.
"""
from __future__ import annotations

import torch

from .._lib import check, dtype_enum, lib, ptr, require_gpu, stream_ptr


def _norm_config(X, W, head_dim):
    # flextrain/ops/_kernels/rmsnorm.py:419-454
    if X.dim() != 2:
        raise ValueError(f"Input tensor X must be 2D, got {X.dim()} dims")
    T, D = X.shape
    if head_dim is None:
        n_cols, n_heads = D, 1
    else:
        if D % head_dim != 0:
            raise ValueError(f"Input dimension D ({D}) must be divisible by head_dim ({head_dim})")
        n_cols, n_heads = head_dim, D // head_dim
    if W is not None:
        expected = (n_cols,)
        if tuple(W.shape) != expected:
            raise ValueError(f"Weight tensor has incorrect shape. Expected {expected}, got {tuple(W.shape)}")
    if not X.is_contiguous():
        raise ValueError("Input tensor X must be contiguous")
    if W is not None and not W.is_contiguous():
        raise ValueError("Weight tensor W must be contiguous")
    return T, D, n_cols, n_heads


def _check_like(t, X, name):
    if t.shape != X.shape:
        raise ValueError(f"{name} shape {tuple(t.shape)} must match input shape {tuple(X.shape)}")
    if not t.is_contiguous():
        raise ValueError(f"{name} must be contiguous")
    if t.dtype != X.dtype:
        raise TypeError(f"{name} dtype {t.dtype} must match input dtype {X.dtype}")


def _fwd(X, W, head_dim, output, rstd, eps, saved):
    T, D, n_cols, n_heads = _norm_config(X, W, head_dim)
    require_gpu(X, W, output, rstd, op="flextrain_rmsnorm_fwd")
    if output is None:
        Y = torch.empty_like(X)
    else:
        _check_like(output, X, "Output tensor")
        Y = output
    if rstd is None:
        if saved:
            raise ValueError("rstd is required")
        rstd = torch.empty(T, n_heads, dtype=torch.float32, device=X.device)
    else:
        if tuple(rstd.shape) != (T, n_heads):
            raise ValueError(f"rstd tensor shape {tuple(rstd.shape)} must match (T, N_HEADS) {(T, n_heads)}")
        if not rstd.is_contiguous():
            raise ValueError("rstd tensor must be contiguous")
        if rstd.dtype != torch.float32:
            raise TypeError("rstd tensor must be float32")
    rc = lib().fx_rmsnorm_fwd(
        ptr(X), ptr(W), ptr(Y), ptr(rstd), T * n_heads, n_cols, float(eps),
        dtype_enum(X.dtype), dtype_enum(W.dtype) if W is not None else 0, 1 if saved else 0,
        stream_ptr(X.device))
    check(rc, "fx_rmsnorm_fwd")
    return Y, rstd


def flextrain_rmsnorm_fwd(X, W=None, head_dim=None, output=None, rstd=None, rms_norm_eps=1e-5):
    """``(Y, rstd)``; flextrain/ops/_kernels/rmsnorm.py:456-530."""
    return _fwd(X, W, head_dim, output, rstd, rms_norm_eps, saved=False)


def flextrain_rmsnorm_fwd_recompute(X, W, rstd, head_dim=None, output=None):
    """``Y`` from the saved ``rstd``; flextrain/ops/_kernels/rmsnorm.py:532-583."""
    Y, _ = _fwd(X, W, head_dim, output, rstd, 0.0, saved=True)
    return Y


def flextrain_rmsnorm_bwd(dY, X, W, rstd, head_dim=None, dX=None, dW=None,
                          recompute_output=False, recomputed_output_tensor=None):
    """``(dX, dW, Y_or_None)``; flextrain/ops/_kernels/rmsnorm.py:585-832.

    ``dW`` is None when ``W`` is None; with ``W`` given and ``dW=None`` a fresh
    fp32 gradient is returned (the reference computes it in that case too,
    rmsnorm.py:690-704).  Unlike the reference's atomics the reduction order is
    fixed, so results are reproducible run to run.
    """
    T, D, n_cols, n_heads = _norm_config(X, W, head_dim)
    require_gpu(dY, X, W, rstd, dX, dW, recomputed_output_tensor, op="flextrain_rmsnorm_bwd")
    _check_like(dY, X, "dY")
    if tuple(rstd.shape) != (T, n_heads) or not rstd.is_contiguous() or rstd.dtype != torch.float32:
        raise ValueError(f"rstd must be a contiguous float32 tensor of shape {(T, n_heads)}")
    y_out = None
    if recompute_output:
        if recomputed_output_tensor is None:
            y_out = torch.empty_like(X)
        else:
            _check_like(recomputed_output_tensor, X, "recomputed_output_tensor")
            y_out = recomputed_output_tensor
    if dX is None:
        dX = torch.empty_like(X)
        acc_dx = 0
    else:
        _check_like(dX, X, "dX")
        acc_dx = 1
    dw_buf, acc_dw = None, 0
    if W is not None:
        if dW is None:
            dw_buf = torch.empty((n_cols,), dtype=torch.float32, device=X.device)
        else:
            if tuple(dW.shape) != (n_cols,):
                raise ValueError(f"dW shape {tuple(dW.shape)} mismatch. Expected {(n_cols,)}")
            if not dW.is_contiguous():
                raise ValueError("dW tensor must be contiguous")
            dw_buf, acc_dw = dW, 1
    rows = T * n_heads
    L = lib()
    ws, ws_bytes = None, 0
    if dw_buf is not None:
        ws_bytes = int(L.fx_rmsnorm_bwd_ws_bytes(rows, n_cols))
        if ws_bytes:
            ws = torch.empty(ws_bytes // 4, dtype=torch.float32, device=X.device)
    rc = L.fx_rmsnorm_bwd(
        ptr(dY), ptr(X), ptr(W), ptr(rstd), ptr(dX), acc_dx, ptr(dw_buf),
        dtype_enum(dw_buf.dtype) if dw_buf is not None else 0, acc_dw, ptr(y_out), rows, n_cols,
        dtype_enum(X.dtype), dtype_enum(W.dtype) if W is not None else 0, ptr(ws), ws_bytes,
        stream_ptr(X.device))
    check(rc, "fx_rmsnorm_bwd")
    return dX, dw_buf, y_out
