"""SiLU backward and embedding backward behind the reference signatures
(flextrain/ops/_kernels/silu_bwd.py:38-67, flextrain/ops/_kernels/embed.py:79-122)."""
from __future__ import annotations

import torch

from .._lib import check, dtype_enum, lib, ptr, stream_ptr


def flextrain_silu_bwd(z, dout, din=None):
    """``din = dout * d/dz silu(z)`` element-wise; inputs and output share a dtype."""
    assert z.shape == dout.shape, f"shape mismatch: z={tuple(z.shape)}, dout={tuple(dout.shape)}"
    assert z.is_cuda and dout.is_cuda
    if z.dtype != dout.dtype:
        raise TypeError("z and dout must share a dtype")
    if not z.is_contiguous():
        z = z.contiguous()
    if not dout.is_contiguous():
        dout = dout.contiguous()
    if din is None:
        din = torch.empty_like(z)
    elif din.shape != z.shape or din.dtype != z.dtype or not din.is_contiguous():
        raise ValueError("din must be contiguous with the shape and dtype of z")
    check(lib().fx_silu_bwd(ptr(z), ptr(dout), ptr(din), z.numel(), dtype_enum(z.dtype), stream_ptr(z.device)),
          "fx_silu_bwd")
    return din


def flextrain_embedding_bwd(grad_output, indices, grad_weight, scale=1.0):
    """``grad_weight[indices[t]] += scale * grad_output[t]`` summed per token id in fp32; returns
    ``grad_weight``.  The ids are sorted with a stable sort, so the summation order — and with it
    the result — is reproducible."""
    assert grad_output.dim() == 2
    assert indices.dim() == 1
    assert grad_weight.dim() == 2
    T, D = grad_output.shape
    if indices.shape[0] != T or grad_weight.shape[1] != D:
        raise ValueError(f"shape mismatch: grad_output {tuple(grad_output.shape)}, indices {tuple(indices.shape)}, "
                         f"grad_weight {tuple(grad_weight.shape)}")
    if not (grad_output.is_cuda and indices.is_cuda and grad_weight.is_cuda):
        raise ValueError("flextrain_embedding_bwd: tensors must be on the GPU")
    if indices.dtype not in (torch.int32, torch.int64):
        raise TypeError(f"indices must be int32 or int64, got {indices.dtype}")
    if T == 0:
        return grad_weight
    sorted_tokens, sorted_pos = torch.sort(indices, stable=True)
    sorted_pos = sorted_pos.to(indices.dtype)
    rc = lib().fx_embedding_bwd(ptr(grad_output), ptr(sorted_pos), ptr(sorted_tokens),
                                1 if indices.dtype == torch.int64 else 0, ptr(grad_weight), T, D,
                                grad_weight.shape[0], grad_output.stride(0), grad_output.stride(1),
                                grad_weight.stride(0), grad_weight.stride(1), float(scale),
                                dtype_enum(grad_output.dtype), dtype_enum(grad_weight.dtype),
                                stream_ptr(grad_output.device))
    check(rc, "fx_embedding_bwd")
    return grad_weight
