"""In-place pair-interleaved rotary embedding behind the reference signatures
(flextrain/ops/_kernels/rope.py:163-307) plus the ``inv_freq`` builders that
feed it (flextrain/nn/blocks/rope.py:28-104).

Differences from the reference, both deliberate: a list of more than two
tensors is rotated completely (the reference's recursion on ``[2:]`` with
``has_k`` false skips the second tensor, rope.py:226-259), and
``flextrain_rope_bwd`` returns its list (the reference returns None).
"""
from __future__ import annotations

import ctypes
import math
import warnings
from typing import Mapping

import torch

from .._lib import check, dtype_enum, lib, ptr, stream_ptr

_INV_FREQ_CACHE: dict = {}


def _vanilla_inv_freq(head_dim, base, device, dtype=torch.float32):
    """``inv_freq[i] = base ** (-2i / head_dim)`` in fp32, cached per
    (head_dim, base, device); flextrain/ops/_kernels/rope.py:165-178."""
    key = (head_dim, float(base), str(device), dtype)
    hit = _INV_FREQ_CACHE.get(key)
    if hit is None:
        exponents = torch.arange(0, head_dim // 2, dtype=torch.float32) * 2.0 / head_dim
        hit = (1.0 / (float(base) ** exponents)).to(dtype).to(device)
        _INV_FREQ_CACHE[key] = hit
    return hit


def _resolve_freqs(freqs_arg, rot_dim, device):
    """``freqs`` is either the (rot_dim/2,) inv_freq array or a 1-element tensor
    holding the base θ; flextrain/ops/_kernels/rope.py:181-204."""
    half = rot_dim // 2
    if freqs_arg.numel() == half:
        f = freqs_arg
        if f.dtype != torch.float32:
            f = f.to(torch.float32)
        if f.device != device:
            f = f.to(device)
        return f.contiguous()
    if freqs_arg.numel() == 1:
        return _vanilla_inv_freq(rot_dim, float(freqs_arg.item()), device)
    raise ValueError(
        f"flextrain_rope: expected freqs of length {half} (inv_freq) or 1 "
        f"(scalar base θ), got numel={freqs_arg.numel()}")


def _strides(t):
    return (ctypes.c_int64 * 3)(*t.stride())


def _apply(tensors_list, pos_ids, freqs, backward, rot_dim=None):
    if not tensors_list:
        return tensors_list
    first = tensors_list[0]
    if first.dim() != 3:
        raise ValueError("flextrain_rope: tensors must be (T, H, D)")
    T, _, D = first.shape
    assert first.is_cuda and pos_ids.is_cuda
    rd = D if rot_dim is None else int(rot_dim)
    if rd <= 0 or rd > D or rd % 2:
        raise ValueError(f"flextrain_rope: rot_dim {rd} invalid for head dim {D}")
    inv_freq = _resolve_freqs(freqs, rd, first.device)
    if pos_ids.dtype != torch.int32:
        pos_ids = pos_ids.to(torch.int32)
    if pos_ids.shape[0] != T:
        raise ValueError(f"flextrain_rope: pos_ids has {pos_ids.shape[0]} rows for {T} tokens")
    L = lib()
    s = stream_ptr(first.device)
    for i in range(0, len(tensors_list), 2):
        q = tensors_list[i]
        k = tensors_list[i + 1] if i + 1 < len(tensors_list) else None
        for t in (q, k):
            if t is None:
                continue
            assert t.dim() == 3 and t.shape[0] == T and t.shape[2] == D and t.is_cuda
            if t.dtype != first.dtype:
                raise TypeError("flextrain_rope: all tensors must share a dtype")
        rc = L.fx_rope(ptr(q), ptr(k), ptr(pos_ids), pos_ids.stride(0), ptr(inv_freq),
                       inv_freq.stride(0), T, q.shape[1], k.shape[1] if k is not None else 0, D, rd,
                       _strides(q), _strides(k) if k is not None else None,
                       dtype_enum(first.dtype), 1 if backward else 0, s)
        check(rc, "fx_rope")
    return tensors_list


def flextrain_rope_fwd(tensors_list, pos_ids, freqs):
    """Rotate every ``(T, H, D)`` tensor of the list in place (Q and K fused in
    one launch) and return the list; flextrain/ops/_kernels/rope.py:207-261."""
    return _apply(tensors_list, pos_ids, freqs, backward=False)


def flextrain_rope_bwd(grad_tensors_list, pos_ids, freqs):
    """Inverse rotation of the gradients, in place;
    flextrain/ops/_kernels/rope.py:264-307."""
    return _apply(grad_tensors_list, pos_ids, freqs, backward=True)


def flextrain_rope_partial_fwd(tensors_list, pos_ids, freqs, rot_dim):
    """Rotate only the first ``rot_dim`` channels of each head
    (flextrain/ops/_kernels/rope_partial.py:29-147)."""
    return _apply(tensors_list, pos_ids, freqs, backward=False, rot_dim=rot_dim)


def flextrain_rope_partial_bwd(grad_tensors_list, pos_ids, freqs, rot_dim):
    return _apply(grad_tensors_list, pos_ids, freqs, backward=True, rot_dim=rot_dim)


def build_rope_inv_freq(head_dim: int, rope_base: float, rope_scaling: Mapping | None = None):
    """fp32 CPU ``inv_freq`` of length ``head_dim/2`` for the HF ``rope_scaling``
    kinds the reference handles: None/"default", "linear" (divide by factor) and
    "llama3" (three wavelength bands); flextrain/nn/blocks/rope.py:28-104."""
    idx = torch.arange(0, head_dim // 2, dtype=torch.float32)
    base_freq = 1.0 / (rope_base ** (idx * 2.0 / head_dim))
    if rope_scaling is None:
        return base_freq
    kind = rope_scaling.get("rope_type") or rope_scaling.get("type") or "default"
    if kind == "default":
        return base_freq
    if kind == "linear":
        return base_freq / float(rope_scaling.get("factor", 1.0))
    if kind == "llama3":
        factor = float(rope_scaling.get("factor", 8.0))
        lo = float(rope_scaling.get("low_freq_factor", 1.0))
        hi = float(rope_scaling.get("high_freq_factor", 4.0))
        orig = int(rope_scaling.get("original_max_position_embeddings", 8192))
        wavelen = 2.0 * math.pi / base_freq
        blend = (orig / wavelen - lo) / max(1e-12, hi - lo)
        mid = (1.0 - blend) * (base_freq / factor) + blend * base_freq
        out = torch.where(wavelen < orig / hi, base_freq, mid)
        return torch.where(wavelen > orig / lo, base_freq / factor, out)
    warnings.warn(f"flextrain RoPE: unknown rope_type {kind!r}; falling back to vanilla.", stacklevel=2)
    return base_freq
