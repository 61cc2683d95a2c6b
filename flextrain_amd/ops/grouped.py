"""Expert-grouped GEMMs: every per-expert matmul of the reference's Python expert
loop (flextrain/ops/full_moe.py:428-466, :545-626) as one launch that reads the
per-expert row counts on the device.  These ops have no single counterpart in
``flextrain.ops``; ``flextrain_amd.full_moe`` composes them behind the
reference's ``swiglu_expert_loop_*`` functions."""
from __future__ import annotations

import torch

from .._lib import check, dtype_enum, lib, ptr, stream_ptr


def _counts_ptr(counts: torch.Tensor, E: int) -> int:
    if counts.dtype != torch.int32 or counts.numel() != E or not counts.is_contiguous():
        raise ValueError(f"expert counts must be a contiguous int32 tensor with {E} elements")
    if not (counts.is_cuda or counts.is_pinned()):
        raise ValueError("expert counts must live on the GPU or in pinned host memory")
    return counts.data_ptr()


def _workspace(E, total_rows, device):
    nbytes = int(lib().fx_grouped_ws_bytes(E, total_rows))
    return torch.empty(nbytes // 4, dtype=torch.int32, device=device), nbytes


def _rowmajor(t, name):
    if t.dim() != 2 or t.stride(1) != 1:
        raise ValueError(f"{name} must be 2-D with unit column stride")


def flextrain_grouped_gemm_rows(A, B, counts, D, C=None, alpha=1.0, beta=0.0):
    """``D[rows_e] = alpha * A[rows_e] @ B[e] + beta * C[rows_e]`` for every expert.

    ``A (TK, K)``, ``D``/``C (TK, N)`` are expert-sorted; ``B`` is ``(E, K, N)``
    in either memory order: pass ``w.transpose(1, 2)`` of an ``(E, N, K)``
    weight for ``x @ w[e].T`` — no copy is made."""
    _rowmajor(A, "A"), _rowmajor(D, "D")
    if B.dim() != 3:
        raise ValueError("B must be (E, K, N)")
    E, K, N = B.shape
    TK = A.shape[0]
    if A.shape[1] != K or tuple(D.shape) != (TK, N):
        raise ValueError(f"shape mismatch: A {tuple(A.shape)}, B {tuple(B.shape)}, D {tuple(D.shape)}")
    if B.stride(2) == 1:
        trans_b, ldb = 0, B.stride(1)
    elif B.stride(1) == 1:
        trans_b, ldb = 1, B.stride(2)
    else:
        raise ValueError("B[e] must be row-major or column-major")
    if not (A.dtype == B.dtype == D.dtype) or (C is not None and C.dtype != D.dtype):
        raise TypeError("A, B, C, D must share a dtype")
    if C is not None:
        _rowmajor(C, "C")
    ws, nbytes = _workspace(E, TK, A.device)
    rc = lib().fx_grouped_gemm_rows(ptr(A), A.stride(0), ptr(B), ldb, B.stride(0), trans_b, ptr(C),
                                    C.stride(0) if C is not None else 0, ptr(D), D.stride(0),
                                    _counts_ptr(counts, E), E, TK, N, K, alpha, beta, dtype_enum(A.dtype),
                                    ptr(ws), nbytes, stream_ptr(A.device))
    check(rc, "fx_grouped_gemm_rows")
    return D


def flextrain_grouped_gemm_wgrad(A, B, G, counts, alpha=1.0, beta=1.0):
    """``G[e] = alpha * A[rows_e].T @ B[rows_e] + beta * G[e]`` for every expert;
    ``A (TK, M)``, ``B (TK, N)`` expert-sorted, ``G (E, M, N)`` (bf16/fp16, or fp32
    for bf16 inputs)."""
    _rowmajor(A, "A"), _rowmajor(B, "B")
    if G.dim() != 3 or G.stride(2) != 1:
        raise ValueError("G must be (E, M, N) with unit last stride")
    E, M, N = G.shape
    TK = A.shape[0]
    if A.shape[1] != M or B.shape[1] != N or B.shape[0] != TK:
        raise ValueError(f"shape mismatch: A {tuple(A.shape)}, B {tuple(B.shape)}, G {tuple(G.shape)}")
    if A.dtype != B.dtype:
        raise TypeError("A and B must share a dtype")
    ws, nbytes = _workspace(E, TK, A.device)
    rc = lib().fx_grouped_gemm_wgrad(ptr(A), A.stride(0), ptr(B), B.stride(0), ptr(G), G.stride(1), G.stride(0),
                                     dtype_enum(G.dtype), _counts_ptr(counts, E), E, TK, M, N, alpha, beta,
                                     dtype_enum(A.dtype), ptr(ws), nbytes, stream_ptr(A.device))
    check(rc, "fx_grouped_gemm_wgrad")
    return G
