"""MoE routing, permutation and expert-activation ops behind the reference
signatures (flextrain/ops/_kernels/moe.py:645-1745).  Same argument names,
validation errors, allocation-when-None behaviour and return values."""
from __future__ import annotations

import torch

from .._lib import check, dtype_enum, lib, ptr, stream_ptr

_MODE_TOPK_THEN_SOFTMAX = 0
_MODE_SOFTMAX_THEN_TOPK = 1


def _routing_mode_id(mode: str) -> int:
    if mode == "topk_then_softmax":
        return _MODE_TOPK_THEN_SOFTMAX
    if mode == "softmax_then_topk":
        return _MODE_SOFTMAX_THEN_TOPK
    raise ValueError(f"unknown routing mode: {mode!r}")


def _is64(t: torch.Tensor) -> int:
    if t.dtype == torch.int64:
        return 1
    if t.dtype == torch.int32:
        return 0
    raise TypeError(f"index tensors must be int32 or int64, got {t.dtype}")


def flextrain_fused_topk_softmax(gate_logits, top_k, topk_ids_out=None, topk_weights_out=None,
                                 mode="topk_then_softmax"):
    """-> ``(topk_weights [T,K], topk_ids [T,K] int32)``;
    flextrain/ops/_kernels/moe.py:848-943."""
    if not gate_logits.is_cuda:
        raise ValueError("gate_logits must be a CUDA tensor")
    if not gate_logits.is_contiguous():
        raise ValueError("gate_logits must be contiguous")
    if gate_logits.dim() != 2:
        raise ValueError(f"gate_logits must be 2D, got {gate_logits.dim()}D")
    T, E = gate_logits.shape
    K = top_k
    if K > E:
        raise ValueError(f"top_k ({K}) cannot exceed num_experts ({E})")
    mode_id = _routing_mode_id(mode)
    if topk_ids_out is None:
        topk_ids_out = torch.empty((T, K), dtype=torch.int32, device=gate_logits.device)
    else:
        if tuple(topk_ids_out.shape) != (T, K):
            raise ValueError(f"topk_ids_out shape {tuple(topk_ids_out.shape)} must be [{T}, {K}]")
        if not topk_ids_out.is_contiguous():
            raise ValueError("topk_ids_out must be contiguous")
        if topk_ids_out.dtype != torch.int32:
            raise TypeError("topk_ids_out must be int32")
    if topk_weights_out is None:
        topk_weights_out = torch.empty((T, K), dtype=gate_logits.dtype, device=gate_logits.device)
    else:
        if tuple(topk_weights_out.shape) != (T, K):
            raise ValueError(f"topk_weights_out shape {tuple(topk_weights_out.shape)} must be [{T}, {K}]")
        if not topk_weights_out.is_contiguous():
            raise ValueError("topk_weights_out must be contiguous")
    rc = lib().fx_topk_softmax(ptr(gate_logits), ptr(topk_ids_out), ptr(topk_weights_out), T, E, K,
                               dtype_enum(gate_logits.dtype), dtype_enum(topk_weights_out.dtype), mode_id,
                               stream_ptr(gate_logits.device))
    check(rc, "fx_topk_softmax")
    return topk_weights_out, topk_ids_out


def flextrain_moe_sort(topk_ids, num_experts, indices=None, expert_counts_gpu=None, block_size=256,
                       expert_counts_pinned=None):
    """-> ``(index_mapping [T,K], expert_counts [E] int32)``;
    flextrain/ops/_kernels/moe.py:649-783.  ``block_size`` is accepted for
    signature compatibility and ignored.  ``expert_counts_pinned`` (extension):
    a pinned int32 host tensor that the sort fills directly, which saves the
    separate :func:`flextrain_copy_expert_counts` launch."""
    if not topk_ids.is_cuda:
        raise ValueError("topk_ids must be a CUDA tensor")
    flat_ids = topk_ids.flatten()
    if not flat_ids.is_contiguous():
        flat_ids = flat_ids.contiguous()
    n = flat_ids.numel()
    dev = topk_ids.device
    if indices is None:
        indices_flat = torch.empty_like(flat_ids)
        result = indices_flat.view(topk_ids.shape)
    else:
        if indices.shape != topk_ids.shape:
            raise ValueError(f"indices shape {indices.shape} must match topk_ids shape {topk_ids.shape}")
        if not indices.is_cuda:
            raise ValueError("indices must be a CUDA tensor")
        if not indices.is_contiguous():
            raise ValueError("indices must be contiguous")
        indices_flat = indices
        result = indices
    total_counts = torch.empty(num_experts, dtype=torch.int32, device=dev)
    host_ptr = None
    if expert_counts_pinned is not None:
        if not expert_counts_pinned.is_pinned() or expert_counts_pinned.dtype != torch.int32 \
                or expert_counts_pinned.numel() != num_experts:
            raise ValueError("expert_counts_pinned must be a pinned int32 tensor with num_experts elements")
        host_ptr = expert_counts_pinned.data_ptr()
    L = lib()
    ws_bytes = int(L.fx_moe_sort_ws_bytes(max(n, 1), num_experts))
    ws = torch.empty(ws_bytes // 4, dtype=torch.int32, device=dev)
    rc = L.fx_moe_sort(ptr(flat_ids), _is64(flat_ids), n, num_experts, ptr(indices_flat), _is64(indices_flat),
                       ptr(total_counts), host_ptr, ptr(ws), ws_bytes, stream_ptr(dev))
    check(rc, "fx_moe_sort")
    if expert_counts_gpu is not None:
        expert_counts_gpu.copy_(total_counts)
    return result, total_counts


def flextrain_copy_expert_counts(gpu_counts, cpu_buffer) -> None:
    """Kernel-side store of the counts into pinned host memory; the caller
    synchronises before reading.  flextrain/ops/_kernels/moe.py:787-834."""
    if not gpu_counts.is_cuda:
        raise ValueError("gpu_counts must be a CUDA tensor")
    if not cpu_buffer.is_pinned():
        raise ValueError("cpu_buffer must be pinned memory (use pin_memory=True)")
    if gpu_counts.shape != cpu_buffer.shape:
        raise ValueError(f"Shape mismatch: gpu_counts {gpu_counts.shape} vs cpu_buffer {cpu_buffer.shape}")
    if gpu_counts.dtype != torch.int32 or cpu_buffer.dtype != torch.int32:
        raise TypeError("expert counts must be int32")
    rc = lib().fx_copy_i32(ptr(gpu_counts), cpu_buffer.data_ptr(), gpu_counts.numel(),
                           stream_ptr(gpu_counts.device))
    check(rc, "fx_copy_i32")


def flextrain_moe_scatter(x, indices, scales=None, out=None):
    """``out[indices[t,k]] = x[t] (* scales[t,k])``; flextrain/ops/_kernels/moe.py:946-1050."""
    if not x.is_cuda:
        raise ValueError("x must be a CUDA tensor")
    if not indices.is_cuda:
        raise ValueError("indices must be a CUDA tensor")
    if not x.is_contiguous():
        raise ValueError("x must be contiguous")
    if not indices.is_contiguous():
        raise ValueError("indices must be contiguous")
    T, D = x.shape
    T_idx, K = indices.shape
    if T_idx != T:
        raise ValueError(f"indices first dim {T_idx} must match x first dim {T}")
    if scales is not None:
        if not scales.is_cuda:
            raise ValueError("scales must be a CUDA tensor")
        if not scales.is_contiguous():
            raise ValueError("scales must be contiguous")
        if scales.numel() != T * K:
            raise ValueError(
                f"scales must have T*K={T*K} elements, got {scales.numel()}. "
                f"Expected shape [T={T}, K={K}] in ORIGINAL order (not sorted).")
    if out is None:
        out = torch.empty((T * K, D), dtype=x.dtype, device=x.device)
    else:
        if tuple(out.shape) != (T * K, D):
            raise ValueError(f"out shape {tuple(out.shape)} must be [{T * K}, {D}]")
        if out.dtype != x.dtype or out.stride(1) != 1:
            raise ValueError("out must have x's dtype and unit column stride")
    rc = lib().fx_moe_scatter(ptr(x), ptr(indices), _is64(indices), ptr(scales),
                              dtype_enum(scales.dtype) if scales is not None else 0, ptr(out), T, D, K,
                              out.stride(0), dtype_enum(x.dtype), stream_ptr(x.device))
    check(rc, "fx_moe_scatter")
    return out


def flextrain_moe_scatter_routing_weights(weights, indices, out=None):
    """``out[indices[i]] = weights[i]``; flextrain/ops/_kernels/moe.py:1053-1127."""
    if not weights.is_cuda:
        raise ValueError("weights must be a CUDA tensor")
    if not indices.is_cuda:
        raise ValueError("indices must be a CUDA tensor")
    if weights.shape != indices.shape:
        raise ValueError(f"weights shape {weights.shape} must match indices shape {indices.shape}")
    w_flat = weights.flatten()
    idx_flat = indices.flatten()
    if not w_flat.is_contiguous():
        raise ValueError("weights must be contiguous")
    if not idx_flat.is_contiguous():
        raise ValueError("indices must be contiguous")
    N = w_flat.numel()
    if out is None:
        out = torch.empty_like(w_flat)
    else:
        if out.numel() != N:
            raise ValueError(f"out must have {N} elements, got {out.numel()}")
        if out.dtype != w_flat.dtype or not out.is_contiguous():
            raise ValueError("out must be contiguous with the weights' dtype")
    rc = lib().fx_moe_scatter_weights(ptr(w_flat), ptr(idx_flat), _is64(idx_flat), ptr(out), N,
                                      dtype_enum(w_flat.dtype), stream_ptr(weights.device))
    check(rc, "fx_moe_scatter_weights")
    return out


def flextrain_moe_row_sources(indices, out=None):
    """``out[indices[t, k]] = t``: the token each expert-sorted row was routed from (int32,
    ``T*K`` entries).  No counterpart in the reference, which always scatters the activations into
    an expert-sorted copy (flextrain/ops/full_moe.py:131-141); with this map the grouped
    up-projection reads the token rows in place (``flextrain_grouped_gemm_rows_glu(row_sources=)``)."""
    if not indices.is_cuda or indices.dim() != 2 or not indices.is_contiguous():
        raise ValueError("indices must be a contiguous (T, K) CUDA tensor")
    if indices.dtype not in (torch.int32, torch.int64):
        raise ValueError("indices must be int32 or int64")
    T, K = indices.shape
    if out is None:
        out = torch.empty(T * K, dtype=torch.int32, device=indices.device)
    elif out.dtype != torch.int32 or out.numel() != T * K or not out.is_contiguous() or not out.is_cuda:
        raise ValueError(f"out must be a contiguous int32 CUDA tensor with {T * K} elements")
    rc = lib().fx_moe_row_sources(ptr(indices), _is64(indices), T, K, ptr(out), stream_ptr(indices.device))
    check(rc, "fx_moe_row_sources")
    return out


def flextrain_moe_gather(expert_out, indices, weights=None, residual=None, out=None):
    """``out[t] = residual[t] + sum_k weights[t,k] * expert_out[indices[t,k]]``
    with an fp32 accumulator; flextrain/ops/_kernels/moe.py:1130-1271."""
    if not expert_out.is_cuda:
        raise ValueError("expert_out must be a CUDA tensor")
    if not indices.is_cuda:
        raise ValueError("indices must be a CUDA tensor")
    if not expert_out.is_contiguous():
        raise ValueError("expert_out must be contiguous")
    if not indices.is_contiguous():
        raise ValueError("indices must be contiguous")
    T, K = indices.shape
    _, D = expert_out.shape
    if expert_out.shape[0] != T * K:
        raise ValueError(
            f"expert_out has {expert_out.shape[0]} rows but expected T*K={T * K} for T={T}, K={K}")
    if residual is not None:
        if not residual.is_cuda:
            raise ValueError("residual must be a CUDA tensor")
        if not residual.is_contiguous():
            raise ValueError("residual must be contiguous")
        if tuple(residual.shape) != (T, D):
            raise ValueError(f"residual shape {tuple(residual.shape)} must be [{T}, {D}]")
    if weights is not None:
        if not weights.is_cuda:
            raise ValueError("weights must be a CUDA tensor")
        if not weights.is_contiguous():
            raise ValueError("weights must be contiguous")
        if tuple(weights.shape) != (T, K):
            raise ValueError(
                f"weights shape {tuple(weights.shape)} must be [{T}, {K}] in ORIGINAL order. "
                f"Do NOT pass router_weights_sorted here - use the original router_weights.")
    if out is None:
        out_dtype = residual.dtype if residual is not None else expert_out.dtype
        out = torch.empty((T, D), dtype=out_dtype, device=expert_out.device)
    else:
        if not out.is_contiguous():
            raise ValueError("out must be contiguous")
        if tuple(out.shape) != (T, D):
            raise ValueError(f"out shape {tuple(out.shape)} must be [{T}, {D}]")
    rc = lib().fx_moe_gather(ptr(expert_out), ptr(indices), _is64(indices), ptr(weights),
                             dtype_enum(weights.dtype) if weights is not None else 0, ptr(residual),
                             dtype_enum(residual.dtype) if residual is not None else 0, ptr(out),
                             dtype_enum(out.dtype), T, D, K, dtype_enum(expert_out.dtype),
                             stream_ptr(expert_out.device))
    check(rc, "fx_moe_gather")
    return out


def _row_major(t, name):
    if t.dim() != 2 or t.stride(1) != 1:
        raise ValueError(f"{name} must be 2-D with unit column stride")


def flextrain_swiglu_moe_fwd(x, w=None, out=None):
    """``silu(x[:, F:]) * x[:, :F] (* w)``; flextrain/ops/_kernels/moe.py:1274-1320."""
    if not x.is_cuda:
        raise ValueError("x must be a CUDA tensor")
    if w is not None and not w.is_cuda:
        raise ValueError("w must be a CUDA tensor")
    T, F2 = x.shape
    if F2 % 2 != 0:
        raise ValueError(f"x last dimension must be even (got {F2}), as it contains packed [value, gate]")
    F = F2 // 2
    _row_major(x, "x")
    if out is None:
        out = torch.empty((T, F), device=x.device, dtype=x.dtype)
    else:
        if tuple(out.shape) != (T, F):
            raise ValueError(f"out shape {tuple(out.shape)} must be [{T}, {F}]")
        _row_major(out, "out")
    if w is not None:
        if w.numel() != T:
            raise ValueError(f"w must have {T} elements, got {w.numel()}")
        w = w.reshape(-1)
        if not w.is_contiguous():
            w = w.contiguous()
    rc = lib().fx_swiglu_moe_fwd(ptr(x), ptr(w), dtype_enum(w.dtype) if w is not None else 0, ptr(out),
                                 dtype_enum(out.dtype), T, F, x.stride(0), out.stride(0), dtype_enum(x.dtype),
                                 stream_ptr(x.device))
    check(rc, "fx_swiglu_moe_fwd")
    return out


def _swiglu_moe_bwd(dout, x, w, dx, dw, fwd_act, prescaled, dname):
    if not dout.is_cuda:
        raise ValueError(f"{dname} must be a CUDA tensor")
    if not x.is_cuda:
        raise ValueError("x must be a CUDA tensor")
    if not w.is_cuda:
        raise ValueError("w must be a CUDA tensor")
    T, F = dout.shape
    if x.shape[0] != T:
        raise ValueError(f"x first dim {x.shape[0]} must match {dname} first dim {T}")
    if x.shape[1] != 2 * F:
        raise ValueError(f"x second dim {x.shape[1]} must be 2*F={2*F}")
    if w.numel() != T:
        raise ValueError(f"w must have {T} elements, got {w.numel()}")
    if dx is None:
        dx = torch.empty_like(x)
    elif dx.shape != x.shape:
        raise ValueError(f"dx shape {dx.shape} must match x shape {x.shape}")
    if dw is None:
        dw = torch.empty((T,), device=x.device, dtype=torch.float32)
    elif dw.numel() != T:
        raise ValueError(f"dw must have {T} elements, got {dw.numel()}")
    if fwd_act is not None and tuple(fwd_act.shape) != (T, F):
        raise ValueError(f"fwd_act shape {tuple(fwd_act.shape)} must be [{T}, {F}]")
    for t, nm in ((dout, dname), (x, "x"), (dx, "dx"), (fwd_act, "fwd_act")):
        if t is not None:
            _row_major(t, nm)
            if t.dtype != x.dtype:
                raise TypeError(f"{nm} must have x's dtype")
    w_flat = w.reshape(-1)
    dw_flat = dw.reshape(-1)
    if not w_flat.is_contiguous() or not dw_flat.is_contiguous():
        raise ValueError("w and dw must be contiguous")
    rc = lib().fx_swiglu_moe_bwd(ptr(dx), ptr(dw_flat), dtype_enum(dw.dtype), ptr(dout), ptr(x), ptr(w_flat),
                                 dtype_enum(w.dtype), ptr(fwd_act), T, F, dx.stride(0), dout.stride(0),
                                 x.stride(0), fwd_act.stride(0) if fwd_act is not None else 0,
                                 dtype_enum(x.dtype), 1 if prescaled else 0, stream_ptr(x.device))
    check(rc, "fx_swiglu_moe_bwd")
    return dx, dw


def flextrain_swiglu_moe_bwd(dout, x, w, dx=None, dw=None, fwd_act=None):
    """-> ``(dx packed [d value | d gate], dw = sum_F dout * act)``; ``fwd_act``
    receives ``act * w``.  flextrain/ops/_kernels/moe.py:1323-1392."""
    return _swiglu_moe_bwd(dout, x, w, dx, dw, fwd_act, False, "dout")


def flextrain_swiglu_moe_bwd_prescaled(dout_scaled, x, w, dx=None, dw=None, fwd_act=None):
    """Variant for an upstream gradient already multiplied by ``w``;
    flextrain/ops/_kernels/moe.py:1395-1524."""
    return _swiglu_moe_bwd(dout_scaled, x, w, dx, dw, fwd_act, True, "dout_scaled")


def flextrain_moe_router_gate_bwd(probs, dprobs, indices, chosen_experts, dlogits=None, num_experts=None,
                                  mode="topk_then_softmax", logits=None):
    """Accumulate the router softmax Jacobian into ``dlogits``;
    flextrain/ops/_kernels/moe.py:1527-1655."""
    if not probs.is_contiguous():
        raise ValueError("probs must be contiguous")
    if not dprobs.is_contiguous():
        raise ValueError("dprobs must be contiguous")
    if not indices.is_contiguous():
        raise ValueError("indices must be contiguous")
    if not chosen_experts.is_contiguous():
        raise ValueError("chosen_experts must be contiguous")
    T, K = probs.shape
    if dprobs.numel() != T * K:
        raise ValueError(f"dprobs must have T*K={T*K} elements, got {dprobs.numel()}")
    if tuple(indices.shape) != (T, K):
        raise ValueError(f"indices shape {tuple(indices.shape)} must be [{T}, {K}]")
    if tuple(chosen_experts.shape) != (T, K):
        raise ValueError(f"chosen_experts shape {tuple(chosen_experts.shape)} must be [{T}, {K}]")
    if dlogits is None:
        if num_experts is None:
            raise ValueError("num_experts must be provided if dlogits is not passed")
        dlogits = torch.zeros((T, num_experts), device=probs.device, dtype=probs.dtype)
    else:
        if dlogits.shape[0] != T:
            raise ValueError(f"dlogits first dim {dlogits.shape[0]} must be T={T}")
        if not dlogits.is_contiguous():
            raise ValueError("dlogits must be contiguous")
    E = dlogits.shape[1]
    mode_id = _routing_mode_id(mode)
    if mode_id == _MODE_SOFTMAX_THEN_TOPK:
        if logits is None:
            raise ValueError("softmax_then_topk backward requires ``logits`` (the original router "
                             "logits, shape [T, E])")
        if tuple(logits.shape) != (T, E):
            raise ValueError(f"logits shape {tuple(logits.shape)} must be [{T}, {E}]")
        if not logits.is_contiguous():
            raise ValueError("logits must be contiguous")
        if logits.dtype != dlogits.dtype:
            raise TypeError("logits and dlogits must share a dtype")
    if probs.dtype != dlogits.dtype:
        raise TypeError("probs and dlogits must share a dtype")
    if chosen_experts.dtype != torch.int32:
        chosen_experts = chosen_experts.to(torch.int32)
    rc = lib().fx_router_gate_bwd(ptr(dlogits), ptr(dprobs), ptr(probs), ptr(indices), _is64(indices),
                                  ptr(chosen_experts), ptr(logits), T, K, E, dtype_enum(dlogits.dtype),
                                  dtype_enum(dprobs.dtype), mode_id, stream_ptr(probs.device))
    check(rc, "fx_router_gate_bwd")
    return dlogits


def flextrain_load_balance_bwd(logits, expert_counts, num_experts, top_k, alpha=0.01, tokens_per_step=0,
                               dlogits=None):
    """``dlogits += (alpha*E/tokens_per_step) * p * (f - <f,p>)``;
    flextrain/ops/_kernels/moe.py:1658-1745."""
    if not logits.is_cuda:
        raise ValueError("logits must be a CUDA tensor")
    if not expert_counts.is_cuda:
        raise ValueError("expert_counts must be a CUDA tensor")
    T, E = logits.shape
    if E != num_experts:
        raise ValueError(f"logits has {E} experts but num_experts={num_experts}")
    if expert_counts.numel() != E:
        raise ValueError(f"expert_counts must have {E} elements, got {expert_counts.numel()}")
    if dlogits is None:
        dlogits = torch.zeros_like(logits)
    elif tuple(dlogits.shape) != (T, E):
        raise ValueError(f"dlogits shape {tuple(dlogits.shape)} must be [{T}, {E}]")
    if not logits.is_contiguous() or not dlogits.is_contiguous():
        raise ValueError("logits and dlogits must be contiguous")
    if tokens_per_step == 0:
        tokens_per_step = T
    scale = alpha * E / tokens_per_step
    counts = expert_counts if expert_counts.dtype == torch.int32 else expert_counts.to(torch.int32)
    rc = lib().fx_load_balance_bwd(ptr(logits), ptr(counts.contiguous()), ptr(dlogits), T, E, top_k, scale,
                                   dtype_enum(logits.dtype), dtype_enum(dlogits.dtype),
                                   stream_ptr(logits.device))
    check(rc, "fx_load_balance_bwd")
    return dlogits
