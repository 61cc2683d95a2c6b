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


def _on_gpu(**tensors) -> None:
    """ValueError for a given tensor that is not on the GPU (None entries are optional arguments not given)."""
    for name, t in tensors.items():
        if t is not None and not t.is_cuda:
            raise ValueError(f"{name} must be a CUDA tensor")


def _dense(**tensors) -> None:
    for name, t in tensors.items():
        if t is not None and not t.is_contiguous():
            raise ValueError(f"{name} must be contiguous")


def _shaped(t, name, *shape) -> None:
    if tuple(t.shape) != shape:
        raise ValueError(f"{name} is {tuple(t.shape)}, expected {shape}")


def _counted(t, name, n, what="") -> None:
    if t.numel() != n:
        raise ValueError(f"{name} holds {t.numel()} elements, expected {n}{what}")


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
    _on_gpu(gate_logits=gate_logits)
    _dense(gate_logits=gate_logits)
    if gate_logits.dim() != 2:
        raise ValueError(f"gate_logits must be (tokens, experts), got {gate_logits.dim()} dimensions")
    T, E = gate_logits.shape
    K = top_k
    if K > E:
        raise ValueError(f"top_k = {K} with only {E} experts")
    mode_id = _routing_mode_id(mode)
    if topk_ids_out is None:
        topk_ids_out = torch.empty((T, K), dtype=torch.int32, device=gate_logits.device)
    else:
        _shaped(topk_ids_out, "topk_ids_out", T, K)
        _dense(topk_ids_out=topk_ids_out)
        if topk_ids_out.dtype != torch.int32:
            raise TypeError("topk_ids_out must be int32")
    if topk_weights_out is None:
        topk_weights_out = torch.empty((T, K), dtype=gate_logits.dtype, device=gate_logits.device)
    else:
        _shaped(topk_weights_out, "topk_weights_out", T, K)
        _dense(topk_weights_out=topk_weights_out)
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
    _on_gpu(topk_ids=topk_ids)
    flat_ids = topk_ids.flatten()
    if not flat_ids.is_contiguous():
        flat_ids = flat_ids.contiguous()
    n = flat_ids.numel()
    dev = topk_ids.device
    if indices is None:
        indices_flat = torch.empty_like(flat_ids)
        result = indices_flat.view(topk_ids.shape)
    else:
        _shaped(indices, "indices", *topk_ids.shape)
        _on_gpu(indices=indices)
        _dense(indices=indices)
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
    _on_gpu(gpu_counts=gpu_counts)
    if not cpu_buffer.is_pinned():
        raise ValueError("cpu_buffer must be pinned host memory: the kernel stores into it directly")
    _shaped(cpu_buffer, "cpu_buffer", *gpu_counts.shape)
    if gpu_counts.dtype != torch.int32 or cpu_buffer.dtype != torch.int32:
        raise TypeError("expert counts must be int32")
    rc = lib().fx_copy_i32(ptr(gpu_counts), cpu_buffer.data_ptr(), gpu_counts.numel(),
                           stream_ptr(gpu_counts.device))
    check(rc, "fx_copy_i32")


def flextrain_moe_scatter(x, indices, scales=None, out=None):
    """``out[indices[t,k]] = x[t] (* scales[t,k])``; flextrain/ops/_kernels/moe.py:946-1050."""
    _on_gpu(x=x, indices=indices, scales=scales)
    _dense(x=x, indices=indices, scales=scales)
    T, D = x.shape
    T_idx, K = indices.shape
    if T_idx != T:
        raise ValueError(f"indices cover {T_idx} tokens, x has {T}")
    if scales is not None:
        _counted(scales, "scales", T * K, f" (one per (token, slot) pair in token order: [{T}, {K}])")
    if out is None:
        out = torch.empty((T * K, D), dtype=x.dtype, device=x.device)
    else:
        _shaped(out, "out", T * K, D)
        if out.dtype != x.dtype or out.stride(1) != 1:
            raise ValueError("out must have x's dtype and unit column stride")
    rc = lib().fx_moe_scatter(ptr(x), ptr(indices), _is64(indices), ptr(scales),
                              dtype_enum(scales.dtype) if scales is not None else 0, ptr(out), T, D, K,
                              out.stride(0), dtype_enum(x.dtype), stream_ptr(x.device))
    check(rc, "fx_moe_scatter")
    return out


def flextrain_moe_scatter_routing_weights(weights, indices, out=None):
    """``out[indices[i]] = weights[i]``; flextrain/ops/_kernels/moe.py:1053-1127."""
    _on_gpu(weights=weights, indices=indices)
    _shaped(weights, "weights", *indices.shape)
    w_flat = weights.flatten()
    idx_flat = indices.flatten()
    _dense(weights=w_flat, indices=idx_flat)
    N = w_flat.numel()
    if out is None:
        out = torch.empty_like(w_flat)
    else:
        _counted(out, "out", N)
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
    _on_gpu(expert_out=expert_out, indices=indices, residual=residual, weights=weights)
    _dense(expert_out=expert_out, indices=indices, residual=residual, weights=weights)
    T, K = indices.shape
    rows, D = expert_out.shape
    if rows != T * K:
        raise ValueError(f"expert_out has {rows} rows, the mapping routes {T} x {K} = {T * K}")
    if residual is not None:
        _shaped(residual, "residual", T, D)
    if weights is not None:
        # one weight per (token, slot) pair in TOKEN order, not the expert-sorted copy
        _shaped(weights, "weights", T, K)
    if out is None:
        out_dtype = residual.dtype if residual is not None else expert_out.dtype
        out = torch.empty((T, D), dtype=out_dtype, device=expert_out.device)
    else:
        _dense(out=out)
        _shaped(out, "out", T, D)
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
    _on_gpu(x=x, w=w)
    T, F2 = x.shape
    if F2 % 2 != 0:
        raise ValueError(f"x rows are packed [value | gate] halves; {F2} columns do not split")
    F = F2 // 2
    _row_major(x, "x")
    if out is None:
        out = torch.empty((T, F), device=x.device, dtype=x.dtype)
    else:
        _shaped(out, "out", T, F)
        _row_major(out, "out")
    if w is not None:
        _counted(w, "w", T)
        w = w.reshape(-1)
        if not w.is_contiguous():
            w = w.contiguous()
    rc = lib().fx_swiglu_moe_fwd(ptr(x), ptr(w), dtype_enum(w.dtype) if w is not None else 0, ptr(out),
                                 dtype_enum(out.dtype), T, F, x.stride(0), out.stride(0), dtype_enum(x.dtype),
                                 stream_ptr(x.device))
    check(rc, "fx_swiglu_moe_fwd")
    return out


def _swiglu_moe_bwd(dout, x, w, dx, dw, fwd_act, prescaled, dname):
    _on_gpu(**{dname: dout, "x": x, "w": w})
    T, F = dout.shape
    _shaped(x, "x", T, 2 * F)
    _counted(w, "w", T)
    if dx is None:
        dx = torch.empty_like(x)
    else:
        _shaped(dx, "dx", *x.shape)
    if dw is None:
        dw = torch.empty((T,), device=x.device, dtype=torch.float32)
    else:
        _counted(dw, "dw", T)
    if fwd_act is not None:
        _shaped(fwd_act, "fwd_act", T, F)
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
    _dense(probs=probs, dprobs=dprobs, indices=indices, chosen_experts=chosen_experts)
    T, K = probs.shape
    _counted(dprobs, "dprobs", T * K)
    _shaped(indices, "indices", T, K)
    _shaped(chosen_experts, "chosen_experts", T, K)
    if dlogits is None:
        if num_experts is None:
            raise ValueError("without dlogits the expert count must be given (num_experts)")
        dlogits = torch.zeros((T, num_experts), device=probs.device, dtype=probs.dtype)
    else:
        if dlogits.shape[0] != T:
            raise ValueError(f"dlogits has {dlogits.shape[0]} rows for {T} tokens")
        _dense(dlogits=dlogits)
    E = dlogits.shape[1]
    mode_id = _routing_mode_id(mode)
    if mode_id == _MODE_SOFTMAX_THEN_TOPK:
        if logits is None:
            raise ValueError("softmax_then_topk recomputes the full softmax: pass the router logits (T, E)")
        _shaped(logits, "logits", T, E)
        _dense(logits=logits)
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
    _on_gpu(logits=logits, expert_counts=expert_counts)
    T, E = logits.shape
    if E != num_experts:
        raise ValueError(f"logits have {E} columns for num_experts = {num_experts}")
    _counted(expert_counts, "expert_counts", E)
    if dlogits is None:
        dlogits = torch.zeros_like(logits)
    else:
        _shaped(dlogits, "dlogits", T, E)
    _dense(logits=logits, dlogits=dlogits)
    if tokens_per_step == 0:
        tokens_per_step = T
    scale = alpha * E / tokens_per_step
    counts = expert_counts if expert_counts.dtype == torch.int32 else expert_counts.to(torch.int32)
    rc = lib().fx_load_balance_bwd(ptr(logits), ptr(counts.contiguous()), ptr(dlogits), T, E, top_k, scale,
                                   dtype_enum(logits.dtype), dtype_enum(dlogits.dtype),
                                   stream_ptr(logits.device))
    check(rc, "fx_load_balance_bwd")
    return dlogits
