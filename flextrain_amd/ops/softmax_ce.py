"""Softmax and cross-entropy ops behind the reference signatures
(flextrain/ops/_kernels/softmax.py:111-215,
flextrain/ops/_kernels/cross_entropy.py:61-134) plus the fused
logits -> (loss, dZ) op the LM head uses."""
from __future__ import annotations

import torch

from .._lib import check, dtype_enum, lib, ptr, stream_ptr

_FLOATS = (torch.float32, torch.float16, torch.bfloat16)


def flextrain_softmax(x, out=None, max_idx_out=None, max_val_out=None, temperature=1.0):
    """``(out, max_idx_out, max_val_out)``: ``out = softmax(x / temperature)`` per
    row; the optional outputs receive the argmax (int64) and the maximum
    probability (fp32).  flextrain/ops/_kernels/softmax.py:111-215."""
    if x.dim() != 2:
        raise ValueError(f"Input tensor 'x' must be 2D, but got {x.dim()} dims.")
    M, N = x.shape
    if not x.is_contiguous():
        raise ValueError("Input tensor 'x' must be contiguous.")
    if x.dtype not in _FLOATS:
        raise TypeError(f"Input dtype {x.dtype} not supported. Supported: {_FLOATS}")
    if temperature <= 0:
        raise ValueError(f"Temperature must be positive, but got {temperature}.")
    if out is None:
        out = torch.empty_like(x)
    else:
        if not out.is_contiguous():
            raise ValueError("Output tensor 'out' must be contiguous.")
        if out.shape != x.shape:
            raise ValueError("Output tensor 'out' must have the same shape as 'x'.")
        if out.dtype not in _FLOATS:
            raise TypeError(f"Output dtype {out.dtype} not supported. Supported: {_FLOATS}")
    if max_val_out is not None:
        if tuple(max_val_out.shape) != (M,):
            raise ValueError(f"Output tensor 'max_val_out' must have shape ({M},), got {tuple(max_val_out.shape)}.")
        if max_val_out.dtype != torch.float32:
            raise ValueError(f"Output tensor 'max_val_out' must have dtype torch.float32, got {max_val_out.dtype}.")
        if not max_val_out.is_contiguous():
            raise ValueError("Output tensor 'max_val_out' must be contiguous.")
    if max_idx_out is not None:
        if tuple(max_idx_out.shape) != (M,):
            raise ValueError(f"Output tensor 'max_idx_out' must have shape ({M},), got {tuple(max_idx_out.shape)}.")
        if max_idx_out.dtype != torch.int64:
            raise ValueError(f"Output tensor 'max_idx_out' must have dtype torch.int64, got {max_idx_out.dtype}.")
        if not max_idx_out.is_contiguous():
            raise ValueError("Output tensor 'max_idx_out' must be contiguous.")
    rc = lib().fx_softmax(ptr(x), ptr(out), ptr(max_idx_out), ptr(max_val_out), M, N, x.stride(0), out.stride(0),
                          float(temperature), dtype_enum(x.dtype), dtype_enum(out.dtype), stream_ptr(x.device))
    check(rc, "fx_softmax")
    return out, max_idx_out, max_val_out


def _labels_flag(labels):
    if labels.dtype == torch.int64:
        return 1
    if labels.dtype == torch.int32:
        return 0
    raise TypeError(f"labels must be int32 or int64, got {labels.dtype}")


def flextrain_cross_entropy_loss(P_in, labels, L=None, Valid_Count_out=None, max_loss=100.0):
    """``(dZ, L)``: ``P_in`` is overwritten with ``P - onehot(label)``;
    ``L = min(-log P[label], max_loss)``.  flextrain/ops/_kernels/cross_entropy.py:61-134."""
    if P_in.dim() != 2:
        raise ValueError(f"Input tensor 'P_in' must be 2D, but got {P_in.dim()} dims.")
    T, V = P_in.shape
    if not P_in.is_contiguous():
        raise ValueError("Input tensor 'P_in' must be contiguous.")
    if P_in.dtype not in _FLOATS:
        raise TypeError(f"Input dtype {P_in.dtype} not supported. Supported: {_FLOATS}")
    if labels.dim() != 1:
        raise ValueError(f"Input tensor 'labels' must be 1D, but got {labels.dim()} dims.")
    if labels.shape[0] != T:
        raise ValueError(f"labels.shape[0] ({labels.shape[0]}) must match P_in.shape[0] ({T}).")
    outs = []
    for t, name in ((L, "L"), (Valid_Count_out, "Valid_Count_out")):
        if t is None:
            t = torch.empty((T,), dtype=torch.float32, device=P_in.device)
        else:
            if tuple(t.shape) != (T,):
                raise ValueError(f"Output tensor '{name}' must have shape ({T},), got {tuple(t.shape)}.")
            if t.dtype != torch.float32:
                raise ValueError(f"Output tensor '{name}' must have dtype torch.float32, got {t.dtype}.")
            if not t.is_contiguous():
                raise ValueError(f"Output tensor '{name}' must be contiguous.")
        outs.append(t)
    L, Valid_Count_out = outs
    labels = labels.contiguous()
    rc = lib().fx_cross_entropy(ptr(P_in), ptr(labels), _labels_flag(labels), ptr(L), ptr(Valid_Count_out), T, V,
                                P_in.stride(0), P_in.stride(1), float(max_loss), dtype_enum(P_in.dtype),
                                stream_ptr(P_in.device))
    check(rc, "fx_cross_entropy")
    return P_in, L


def flextrain_softmax_cross_entropy_loss(X, labels, L=None, Valid_Count=None):
    """The reference's summary wrapper (flextrain/ops/_kernels/cross_entropy.py:215-268): runs the
    probability cross-entropy kernel on ``X`` in place (``X`` becomes ``P - onehot``, rows with a
    negative label become zero), then reduces on the device and returns
    ``(X, L, total_loss, avg_loss, num_valid_labels)`` with the three scalars as Python floats
    (this synchronises with the host, as the reference's ``.item()`` calls do)."""
    T, V = X.shape
    assert X.is_contiguous(), "Input tensor X must be contiguous"
    assert labels.shape == (T,), f"Labels tensor must have shape ({T},), but got {labels.shape}"
    if L is not None:
        assert L.shape == (T,), f"L must have shape {(T,)}, but got {L.shape}"
        assert L.device == X.device, "L must be on the same device as X"
        assert L.dtype == torch.float32, "L must be dtype torch.float32"
    if Valid_Count is None:
        Valid_Count = torch.empty((T,), dtype=torch.float32, device=X.device)
    else:
        assert Valid_Count.shape == (T,), f"Valid_Count must have shape {(T,)}, but got {Valid_Count.shape}"
        assert Valid_Count.device == X.device, "Valid_Count must be on the same device as X"
        assert Valid_Count.dtype == torch.float32, "Valid_Count must be dtype torch.float32"
    X, L = flextrain_cross_entropy_loss(X, labels, L=L, Valid_Count_out=Valid_Count)
    total_loss = torch.sum(L)
    num_valid_labels = torch.sum(Valid_Count)
    avg_loss = total_loss / (num_valid_labels + 1e-8)
    return X, L, total_loss.item(), avg_loss.item(), num_valid_labels.item()


def flextrain_softmax_cross_entropy(logits, labels, L=None, dZ=None, loss_mask=None, max_idx_out=None,
                                    max_val_out=None, ignore_index=-100, max_loss=100.0, logit_softcap=None):
    """Fused row softmax + cross-entropy + dZ.  ``dZ`` defaults to ``logits`` (in
    place).  Per-row fp32 loss ``lse - logit[label]`` goes to ``L``; rows whose
    label is ``ignore_index`` or whose ``loss_mask`` is False get loss 0 and a zero
    dZ row.  No host synchronisation.  Returns ``(dZ, L)``.

    ``logit_softcap`` (Gemma's final-logit soft cap, flextrain/nn/head.py:273-298): loss,
    argmax and probabilities are taken from ``cap * tanh(logits / cap)`` and ``dZ`` is the
    gradient at the uncapped logits; the capped logits are never written."""
    if logits.dim() != 2 or not logits.is_cuda:
        raise ValueError("logits must be a 2-D CUDA tensor")
    T, V = logits.shape
    if logits.stride(1) != 1:
        raise ValueError("logits must have unit column stride")
    if logits.dtype not in _FLOATS:
        raise TypeError(f"Input dtype {logits.dtype} not supported. Supported: {_FLOATS}")
    if tuple(labels.shape) != (T,):
        raise ValueError(f"labels must have shape ({T},), got {tuple(labels.shape)}")
    if dZ is None:
        dZ = logits
    elif dZ.shape != logits.shape or dZ.dtype != logits.dtype or dZ.stride(1) != 1:
        raise ValueError("dZ must match logits in shape and dtype with unit column stride")
    if L is None:
        L = torch.empty((T,), dtype=torch.float32, device=logits.device)
    elif tuple(L.shape) != (T,) or L.dtype != torch.float32 or not L.is_contiguous():
        raise ValueError(f"L must be a contiguous float32 tensor of shape ({T},)")
    mask = None
    if loss_mask is not None:
        if tuple(loss_mask.shape) != (T,):
            raise ValueError(f"loss_mask must have shape ({T},)")
        mask = loss_mask.to(torch.uint8).contiguous() if loss_mask.dtype != torch.uint8 else loss_mask.contiguous()
    for t, nm, dt in ((max_idx_out, "max_idx_out", torch.int64), (max_val_out, "max_val_out", torch.float32)):
        if t is not None and (tuple(t.shape) != (T,) or t.dtype != dt or not t.is_contiguous()):
            raise ValueError(f"{nm} must be a contiguous {dt} tensor of shape ({T},)")
    cap = 0.0
    if logit_softcap is not None:
        cap = float(logit_softcap)
        if not cap > 0.0:
            raise ValueError(f"logit_softcap must be positive, got {logit_softcap}")
    labels = labels.contiguous()
    rc = lib().fx_softmax_ce(ptr(logits), ptr(dZ), ptr(labels), _labels_flag(labels), ptr(mask), ptr(L),
                             ptr(max_idx_out), ptr(max_val_out), T, V, logits.stride(0), dZ.stride(0),
                             int(ignore_index), float(max_loss), cap, dtype_enum(logits.dtype),
                             stream_ptr(logits.device))
    check(rc, "fx_softmax_ce")
    return dZ, L


def _softcap_args(t, name):
    if t.dim() != 2 or not t.is_cuda or t.stride(1) != 1:
        raise ValueError(f"{name} must be a 2-D CUDA tensor with unit column stride")
    if t.dtype not in _FLOATS:
        raise TypeError(f"{name} dtype {t.dtype} not supported. Supported: {_FLOATS}")


def flextrain_logit_softcap_fwd(logits, cap, gate_out=None):
    """In place ``logits = cap * tanh(logits / cap)``; returns the gate
    ``1 - (logits_capped / cap)^2`` in the logits' dtype (flextrain/nn/head.py:276-282)."""
    _softcap_args(logits, "logits")
    if not float(cap) > 0.0:
        raise ValueError(f"cap must be positive, got {cap}")
    if gate_out is None:
        gate_out = torch.empty_like(logits)
    elif gate_out.shape != logits.shape or gate_out.dtype != logits.dtype or gate_out.stride(1) != 1:
        raise ValueError("gate_out must match logits in shape and dtype with unit column stride")
    T, V = logits.shape
    rc = lib().fx_softcap_fwd(ptr(logits), ptr(gate_out), T, V, logits.stride(0), gate_out.stride(0), float(cap),
                              dtype_enum(logits.dtype), stream_ptr(logits.device))
    check(rc, "fx_softcap_fwd")
    return gate_out


def flextrain_logit_softcap_bwd(dZ, gate):
    """In place ``dZ *= gate`` (flextrain/nn/head.py:295-297)."""
    _softcap_args(dZ, "dZ")
    if gate.shape != dZ.shape or gate.dtype != dZ.dtype or gate.stride(1) != 1 or not gate.is_cuda:
        raise ValueError("gate must match dZ in shape and dtype with unit column stride")
    T, V = dZ.shape
    rc = lib().fx_softcap_bwd(ptr(dZ), ptr(gate), T, V, dZ.stride(0), gate.stride(0), dtype_enum(dZ.dtype),
                              stream_ptr(dZ.device))
    check(rc, "fx_softcap_bwd")
    return dZ
