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


class GroupedPlan:
    """Row offsets and tile list of one routing (``fx_grouped_plan``), made once and passed as
    ``plan=`` to several grouped launches of the same ``(counts, E, total_rows)``.  The plan is
    written on the stream that is current when it is made: launches that use it must be ordered
    after that point (same stream, or an event), and it must outlive them."""

    def __init__(self, counts: torch.Tensor, E: int, total_rows: int, device):
        self.E, self.total_rows = E, total_rows
        self.ws, self.nbytes = _workspace(E, total_rows, device)
        rc = lib().fx_grouped_plan(_counts_ptr(counts, E), E, total_rows, ptr(self.ws), self.nbytes, stream_ptr(device))
        check(rc, "fx_grouped_plan")


def _plan_or_workspace(plan, counts, E, total_rows, device):
    """(counts pointer or None, workspace tensor, bytes): with a plan the counts are not read again."""
    if plan is not None:
        if plan.E != E or plan.total_rows != total_rows:
            raise ValueError(f"the plan was made for E={plan.E}, rows={plan.total_rows}; this call has E={E}, rows={total_rows}")
        return None, plan.ws, plan.nbytes
    if counts is None:
        raise ValueError("expert counts are required when no plan is given")
    ws, nbytes = _workspace(E, total_rows, device)
    return _counts_ptr(counts, E), ws, nbytes


def _rowmajor(t, name):
    if t.dim() != 2 or t.stride(1) != 1:
        raise ValueError(f"{name} must be 2-D with unit column stride")


def flextrain_grouped_gemm_rows(A, B, counts, D, C=None, alpha=1.0, beta=0.0, plan=None):
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
    cptr, ws, nbytes = _plan_or_workspace(plan, counts, E, TK, A.device)
    rc = lib().fx_grouped_gemm_rows(ptr(A), A.stride(0), ptr(B), ldb, B.stride(0), trans_b, ptr(C),
                                    C.stride(0) if C is not None else 0, ptr(D), D.stride(0),
                                    cptr, E, TK, N, K, alpha, beta, dtype_enum(A.dtype),
                                    ptr(ws), nbytes, stream_ptr(A.device))
    check(rc, "fx_grouped_gemm_rows")
    return D


def _row_sources_ok(row_sources, TK):
    return (row_sources.dtype == torch.int32 and row_sources.numel() == TK and row_sources.is_contiguous()
            and row_sources.is_cuda)


def gathered_operand_supported(src):
    """Whether an unsorted activation matrix can stand in for its expert-sorted copy in the grouped
    launches that take ``row_sources`` (16-byte rows below 4 GB in all)."""
    return (src.dim() == 2 and src.stride(1) == 1 and src.stride(0) % 8 == 0 and src.data_ptr() % 16 == 0
            and src.dtype in (torch.bfloat16, torch.float16)
            and src.shape[0] * src.stride(0) * src.element_size() < (1 << 32))


def flextrain_grouped_gemm_wgrad(A, B, G, counts, alpha=1.0, beta=1.0, plan=None, a_row_sources=None,
                                 b_row_sources=None):
    """``G[e] = alpha * A[rows_e].T @ B[rows_e] + beta * G[e]`` for every expert;
    ``A (TK, M)``, ``B (TK, N)`` expert-sorted, ``G (E, M, N)`` (bf16/fp16, or fp32
    for bf16 inputs).

    ``a_row_sources`` / ``b_row_sources`` (at most one; int32, one entry per expert-sorted row, from
    ``flextrain_moe_row_sources``): that operand is then the UNSORTED ``(T, M)`` / ``(T, N)`` matrix and
    sorted row ``r`` of it is row ``row_sources[r]``, gathered by the kernel's own tile loads."""
    _rowmajor(A, "A"), _rowmajor(B, "B")
    if G.dim() != 3 or G.stride(2) != 1:
        raise ValueError("G must be (E, M, N) with unit last stride")
    E, M, N = G.shape
    if a_row_sources is not None and b_row_sources is not None:
        raise ValueError("at most one operand may be gathered")
    TK = B.shape[0] if a_row_sources is not None else A.shape[0]
    for t, src, name in ((A, a_row_sources, "A"), (B, b_row_sources, "B")):
        if src is None:
            if t.shape[0] != TK:
                raise ValueError(f"shape mismatch: A {tuple(A.shape)}, B {tuple(B.shape)}, G {tuple(G.shape)}")
        elif not _row_sources_ok(src, TK) or not gathered_operand_supported(t):
            raise ValueError(f"{name}: row sources must be a contiguous int32 CUDA tensor with {TK} elements and the "
                             f"unsorted matrix must have 16-byte rows below 4 GB")
    if A.shape[1] != M or B.shape[1] != N:
        raise ValueError(f"shape mismatch: A {tuple(A.shape)}, B {tuple(B.shape)}, G {tuple(G.shape)}")
    if A.dtype != B.dtype:
        raise TypeError("A and B must share a dtype")
    cptr, ws, nbytes = _plan_or_workspace(plan, counts, E, TK, A.device)
    rc = lib().fx_grouped_gemm_wgrad(ptr(A), A.stride(0), ptr(B), B.stride(0), ptr(G), G.stride(1), G.stride(0),
                                     dtype_enum(G.dtype), cptr, E, TK, M, N, alpha, beta,
                                     dtype_enum(A.dtype), ptr(ws), nbytes, ptr(a_row_sources), A.shape[0],
                                     ptr(b_row_sources), B.shape[0], stream_ptr(A.device))
    check(rc, "fx_grouped_gemm_wgrad")
    return G



def _b_layout(B):
    if B.stride(-1) == 1:
        return 0, B.stride(-2)
    if B.stride(-2) == 1:
        return 1, B.stride(-1)
    raise ValueError("the weight must be row-major or column-major")


def grouped_glu_supported(A, w_up, pre, act):
    """Whether :func:`flextrain_grouped_gemm_rows_glu` can take these tensors (else the caller
    runs the GEMM and the activation kernel separately)."""
    F = act.shape[1]
    K = A.shape[1]
    return (A.dtype in (torch.bfloat16, torch.float16) and A.dtype == w_up.dtype == pre.dtype == act.dtype
            and K % 64 == 0 and F % 8 == 0 and A.stride(1) == 1 and pre.stride(1) == 1 and act.stride(1) == 1
            and A.stride(0) % 8 == 0 and pre.stride(0) % 8 == 0 and act.stride(0) % 8 == 0
            and w_up.is_contiguous() and all(t.data_ptr() % 16 == 0 for t in (A, w_up, pre, act)))


def flextrain_grouped_gemm_rows_glu(A, w_up, counts, pre, act, row_sources=None, plan=None):
    """Expert up-projection and SwiGLU in one launch: ``pre[rows_e] = A[rows_e] @ w_up[e].T``
    (packed ``[value (F) | gate (F)]`` like ``w_up (E, 2F, K)``) and ``act = silu(gate) * value``,
    the activation evaluated from the rounded ``pre`` as the separate kernel would.

    ``row_sources`` (int32, one entry per expert-sorted row, from ``flextrain_moe_row_sources``):
    ``A`` is then the UNSORTED ``(T, K)`` activation matrix and sorted row ``r`` is
    ``A[row_sources[r]]``, gathered by the kernel's own tile loads (no expert-sorted copy)."""
    _rowmajor(A, "A"), _rowmajor(pre, "pre"), _rowmajor(act, "act")
    if w_up.dim() != 3 or not w_up.is_contiguous():
        raise ValueError("w_up must be a contiguous (E, 2F, K) tensor")
    E, F2, K = w_up.shape
    F = F2 // 2
    TK = pre.shape[0]
    if A.shape[1] != K or tuple(pre.shape) != (TK, F2) or tuple(act.shape) != (TK, F):
        raise ValueError(f"shape mismatch: A {tuple(A.shape)}, w_up {tuple(w_up.shape)}, pre {tuple(pre.shape)}, "
                         f"act {tuple(act.shape)}")
    if row_sources is None:
        if A.shape[0] != TK:
            raise ValueError(f"A has {A.shape[0]} rows, the outputs {TK}")
    elif (row_sources.dtype != torch.int32 or row_sources.numel() != TK or not row_sources.is_contiguous()
          or not row_sources.is_cuda):
        raise ValueError(f"row_sources must be a contiguous int32 CUDA tensor with {TK} elements")
    cptr, ws, nbytes = _plan_or_workspace(plan, counts, E, TK, A.device)
    es = pre.element_size()
    rc = lib().fx_grouped_gemm_rows_glu(ptr(A), A.stride(0), ptr(w_up), K, w_up.stride(0), 1, F * K, ptr(pre),
                                        pre.data_ptr() + F * es, pre.stride(0), ptr(act), act.stride(0),
                                        cptr, E, TK, F, K, 0, dtype_enum(A.dtype), ptr(ws), nbytes,
                                        ptr(row_sources), A.shape[0], stream_ptr(A.device))
    check(rc, "fx_grouped_gemm_rows_glu")
    return pre, act


def grouped_swiglu_bwd_supported(dy, w_down, x_up, srw, dx_up, fwd_act, dprob, dy_is_unsorted=False):
    """Whether :func:`flextrain_grouped_gemm_rows_swiglu_bwd` can take these tensors (else the
    caller runs the dgrad GEMM and ``flextrain_swiglu_moe_bwd`` separately).  ``dy_is_unsorted``:
    ``dy`` is the ``(T, d)`` upstream gradient, to be gathered through row sources."""
    if dy.dtype not in (torch.bfloat16, torch.float16) or w_down.dim() != 3 or not w_down.is_contiguous():
        return False
    E, d, F = w_down.shape
    TK = x_up.shape[0]
    if dy_is_unsorted and not gathered_operand_supported(dy):
        return False
    if any(t.dtype != dy.dtype for t in (w_down, x_up, dx_up)) or (fwd_act is not None and fwd_act.dtype != dy.dtype):
        return False
    if srw.dtype not in (dy.dtype, torch.float32) or dprob.dtype not in (dy.dtype, torch.float32):
        return False
    if not (srw.is_contiguous() and dprob.is_contiguous() and srw.numel() == TK and dprob.numel() == TK):
        return False
    two_d = [x_up, dx_up] + ([fwd_act] if fwd_act is not None else []) + ([] if dy_is_unsorted else [dy])
    if any(t.dim() != 2 or t.stride(1) != 1 or t.stride(0) % 8 or t.data_ptr() % 16 or t.shape[0] != TK for t in two_d):
        return False
    if dy.dim() != 2 or dy.stride(1) != 1 or dy.stride(0) % 8 or dy.data_ptr() % 16:
        return False
    if dy.shape[1] != d or x_up.shape[1] != 2 * F or dx_up.shape[1] != 2 * F or (fwd_act is not None and fwd_act.shape[1] != F):
        return False
    return (d % 8 == 0 and F % 8 == 0 and w_down.data_ptr() % 16 == 0
            and int(lib().fx_grouped_rows_tile_height(E, TK)) == 256)


def flextrain_grouped_gemm_rows_swiglu_bwd(dy, w_down, counts, x_up, srw, dx_up, dprob, fwd_act=None, plan=None,
                                           row_sources=None):
    """Expert dgrad through ``w_down (E, d, F)`` with the weighted SwiGLU backward in its epilogue:
    ``dx_act = dy[rows_e] @ w_down[e]`` is rounded and consumed in registers;
    ``dx_up (TK, 2F)``, ``fwd_act (TK, F) = act * w`` and ``dprob (TK,) = sum_F dx_act * act`` are
    written.  ``x_up (TK, 2F)`` is the saved pre-activation ``[value | gate]``, ``srw`` the
    expert-sorted router weights.  ``dx_up`` / ``fwd_act`` equal, bit for bit, what
    ``flextrain_grouped_gemm_rows`` + ``flextrain_swiglu_moe_bwd`` give.

    ``row_sources``: ``dy`` is then the UNSORTED ``(T, d)`` upstream gradient and sorted row ``r`` is
    ``dy[row_sources[r]]`` (no expert-sorted copy of it is read)."""
    if not grouped_swiglu_bwd_supported(dy, w_down, x_up, srw, dx_up, fwd_act, dprob, dy_is_unsorted=row_sources is not None):
        raise ValueError("unsupported operands for the fused dgrad + SwiGLU backward (see grouped_swiglu_bwd_supported)")
    E, d, F = w_down.shape
    TK = x_up.shape[0]
    if row_sources is not None and not _row_sources_ok(row_sources, TK):
        raise ValueError(f"row_sources must be a contiguous int32 CUDA tensor with {TK} elements")
    cptr, ws, nbytes = _plan_or_workspace(plan, counts, E, TK, dy.device)
    part_bytes = int(lib().fx_grouped_swiglu_bwd_ws_bytes(TK, F))
    part = torch.empty(part_bytes // 4, dtype=torch.float32, device=dy.device)
    rc = lib().fx_grouped_gemm_rows_swiglu_bwd(
        ptr(dy), dy.stride(0), ptr(w_down), F, w_down.stride(0), 0, ptr(x_up), x_up.stride(0), ptr(srw),
        dtype_enum(srw.dtype), ptr(dx_up), dx_up.stride(0), ptr(fwd_act), fwd_act.stride(0) if fwd_act is not None else 0,
        ptr(dprob), dtype_enum(dprob.dtype), cptr, E, TK, F, d, dtype_enum(dy.dtype), ptr(ws), nbytes, ptr(part),
        part_bytes, ptr(row_sources), dy.shape[0], stream_ptr(dy.device))
    check(rc, "fx_grouped_gemm_rows_swiglu_bwd")
    return dx_up, dprob, fwd_act


_ACT_ENUM = {"silu": 0, "gelu_tanh": 1}


def dual_glu_supported(A, B1, B2, P1, P2, act):
    """Whether :func:`flextrain_gemm_dual_glu` can take these tensors."""
    if A.dtype not in (torch.bfloat16, torch.float16) or any(t.dtype != A.dtype for t in (B1, B2, P1, P2, act)):
        return False
    if A.dim() != 2 or B1.dim() != 2 or B1.shape != B2.shape or B1.stride() != B2.stride():
        return False
    if not (B1.stride(1) == 1 or B1.stride(0) == 1):
        return False
    K, N = B1.shape
    ldb = B1.stride(0) if B1.stride(1) == 1 else B1.stride(1)
    return (K % 64 == 0 and N % 8 == 0 and ldb % 8 == 0 and A.stride(1) == 1 and A.stride(0) % 8 == 0
            and all(t.stride(1) == 1 and t.stride(0) % 8 == 0 for t in (P1, P2, act)) and P1.stride(0) == P2.stride(0)
            and all(t.data_ptr() % 16 == 0 for t in (A, B1, B2, P1, P2, act)))


def flextrain_gemm_dual_glu(A, B1, B2, P1, P2, act, activation="silu", gate_first=True):
    """``P1 = A @ B1``, ``P2 = A @ B2`` and ``act = f(gate) * value`` in one launch, where
    ``(gate, value) = (P1, P2)`` when ``gate_first``; ``B1`` / ``B2`` are ``(K, N)`` in either memory
    order (the same for both)."""
    M, K = A.shape
    N = B1.shape[1]
    if B1.shape[0] != K or tuple(P1.shape) != (M, N) or tuple(P2.shape) != (M, N) or tuple(act.shape) != (M, N):
        raise ValueError("shape mismatch")
    trans_b, ldb = _b_layout(B1)
    rc = lib().fx_gemm_dual_glu(ptr(A), A.stride(0), ptr(B1), ptr(B2), ldb, trans_b, ptr(P1), ptr(P2), P1.stride(0),
                                ptr(act), act.stride(0), M, N, K, 1 if gate_first else 0, _ACT_ENUM[activation],
                                dtype_enum(A.dtype), stream_ptr(A.device))
    check(rc, "fx_gemm_dual_glu")
    return act
