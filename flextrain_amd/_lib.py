"""ctypes binding of ``libflexhip.so`` (declared in ``include/flexhip.h``).

The library is the only compute path: when it is missing or fails to load,
``lib()`` raises — there is no PyTorch or CPU fallback behind the ops.
"""
from __future__ import annotations

import ctypes
import os
from ctypes import c_char_p, c_double, c_float, c_int, c_int32, c_int64, c_size_t, c_uint64, c_void_p, POINTER

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libflexhip.so")

DT_F32, DT_F16, DT_BF16 = 0, 1, 2
ACT_SILU, ACT_GELU_TANH = 0, 1

_DTYPE_ENUM = {torch.float32: DT_F32, torch.float16: DT_F16, torch.bfloat16: DT_BF16}


def dtype_enum(dtype: torch.dtype) -> int:
    """0 fp32 / 1 fp16 / 2 bf16 (helpers/matmul_dispatcher/matmul_dispatcher/__init__.py:40-49)."""
    try:
        return _DTYPE_ENUM[dtype]
    except KeyError:
        raise TypeError(f"dtype {dtype} not supported; supported: {list(_DTYPE_ENUM)}") from None


# name -> (restype, argtypes); one entry per declaration in include/flexhip.h
_SIGNATURES = {
    "fx_version": (c_char_p, []),
    "fx_rmsnorm_fwd": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int, c_float,
                               c_int, c_int, c_int, c_void_p]),
    "fx_rmsnorm_bwd_ws_bytes": (c_size_t, [c_int64, c_int]),
    "fx_rmsnorm_bwd": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_void_p,
                               c_int, c_int, c_void_p, c_int64, c_int, c_int, c_int, c_void_p,
                               c_size_t, c_void_p]),
    "fx_rope": (c_int, [c_void_p, c_void_p, c_void_p, c_int64, c_void_p, c_int64, c_int64, c_int,
                        c_int, c_int, c_int, POINTER(c_int64), POINTER(c_int64), c_int, c_int,
                        c_void_p]),
    "fx_glu_fwd": (c_int, [c_void_p, c_void_p, c_void_p, c_int64, c_int, c_int, c_int, c_void_p]),
    "fx_glu_bwd": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int64,
                           c_int, c_int, c_void_p]),
    "fx_silu_bwd": (c_int, [c_void_p, c_void_p, c_void_p, c_int64, c_int, c_void_p]),
    "fx_embedding_bwd": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_int64, c_int, c_int64, c_int64,
                                 c_int64, c_int64, c_int64, c_float, c_int, c_int, c_void_p]),
    "fx_adamw_step": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int,
                              c_int, c_int, c_float, c_float, c_float, c_float, c_float, c_float,
                              c_float, c_void_p]),
    "fx_nonfinite_flag": (c_int, [c_void_p, c_int64, c_int, c_void_p, c_void_p]),
    "fx_topk_softmax": (c_int, [c_void_p, c_void_p, c_void_p, c_int64, c_int, c_int, c_int, c_int, c_int,
                                c_void_p]),
    "fx_moe_sort_ws_bytes": (c_size_t, [c_int64, c_int]),
    "fx_moe_sort": (c_int, [c_void_p, c_int, c_int64, c_int, c_void_p, c_int, c_void_p, c_void_p, c_void_p,
                            c_size_t, c_void_p]),
    "fx_moe_sort_noalloc": (c_int, [c_void_p, c_int, c_int64, c_int, c_void_p, c_int, c_void_p, c_void_p, c_void_p]),
    "fx_moe_sort_noalloc_init": (c_int, []),
    "fx_moe_sort_noalloc_max_words": (c_size_t, []),
    "fx_copy_i32": (c_int, [c_void_p, c_void_p, c_int, c_void_p]),
    "fx_router_gate_bwd": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p,
                                   c_int64, c_int, c_int, c_int, c_int, c_int, c_void_p]),
    "fx_load_balance_bwd": (c_int, [c_void_p, c_void_p, c_void_p, c_int64, c_int, c_int, c_float, c_int,
                                    c_int, c_void_p]),
    "fx_moe_scatter": (c_int, [c_void_p, c_void_p, c_int, c_void_p, c_int, c_void_p, c_int64, c_int, c_int,
                               c_int64, c_int, c_void_p]),
    "fx_moe_scatter_weights": (c_int, [c_void_p, c_void_p, c_int, c_void_p, c_int64, c_int, c_void_p]),
    "fx_grouped_plan": (c_int, [c_void_p, c_int, c_int64, c_void_p, c_size_t, c_void_p]),
    "fx_moe_row_sources": (c_int, [c_void_p, c_int, c_int64, c_int, c_void_p, c_void_p]),
    "fx_moe_gather": (c_int, [c_void_p, c_void_p, c_int, c_void_p, c_int, c_void_p, c_int, c_void_p, c_int,
                              c_int64, c_int, c_int, c_int, c_void_p]),
    "fx_swiglu_moe_fwd": (c_int, [c_void_p, c_void_p, c_int, c_void_p, c_int, c_int64, c_int, c_int64,
                                  c_int64, c_int, c_void_p]),
    "fx_softmax": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int, c_int64, c_int64, c_float,
                           c_int, c_int, c_void_p]),
    "fx_cross_entropy": (c_int, [c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_int64, c_int, c_int64, c_int64,
                                 c_float, c_int, c_void_p]),
    "fx_softmax_ce": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_void_p,
                              c_int64, c_int, c_int64, c_int64, c_int64, c_float, c_float, c_int, c_void_p]),
    "fx_softcap_fwd": (c_int, [c_void_p, c_void_p, c_int64, c_int, c_int64, c_int64, c_float, c_int, c_void_p]),
    "fx_softcap_bwd": (c_int, [c_void_p, c_void_p, c_int64, c_int, c_int64, c_int64, c_int, c_void_p]),
    "fx_grouped_rows_tile_height": (c_int, [c_int, c_int64]),
    "fx_grouped_swiglu_bwd_ws_bytes": (c_size_t, [c_int64, c_int]),
    "fx_grouped_gemm_rows_swiglu_bwd": (c_int, [c_void_p, c_int64, c_void_p, c_int64, c_int64, c_int, c_void_p, c_int64,
                                                c_void_p, c_int, c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_int,
                                                c_void_p, c_int, c_int64, c_int, c_int, c_int, c_void_p, c_size_t,
                                                c_void_p, c_size_t, c_void_p, c_int64, c_void_p]),
    "fx_grouped_ws_bytes": (c_size_t, [c_int, c_int64]),
    "fx_grouped_gemm_rows": (c_int, [c_void_p, c_int64, c_void_p, c_int64, c_int64, c_int, c_void_p, c_int64,
                                     c_void_p, c_int64, c_void_p, c_int, c_int64, c_int, c_int, c_float, c_float,
                                     c_int, c_void_p, c_size_t, c_void_p]),
    "fx_grouped_gemm_wgrad": (c_int, [c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_int64, c_int64, c_int,
                                      c_void_p, c_int, c_int64, c_int, c_int, c_float, c_float, c_int, c_void_p,
                                      c_size_t, c_void_p, c_int64, c_void_p, c_int64, c_void_p]),
    "fx_grouped_gemm_rows_glu": (c_int, [c_void_p, c_int64, c_void_p, c_int64, c_int64, c_int, c_int64, c_void_p,
                                         c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_int, c_int64, c_int,
                                         c_int, c_int, c_int, c_void_p, c_size_t, c_void_p, c_int64, c_void_p]),
    "fx_gemm_dual_glu": (c_int, [c_void_p, c_int64, c_void_p, c_void_p, c_int64, c_int, c_void_p, c_void_p, c_int64,
                                 c_void_p, c_int64, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p]),
    "fx_gemm_segments": (c_int, [c_void_p, c_int64, c_int, c_int, POINTER(c_void_p), POINTER(c_int64), c_int,
                                 POINTER(c_void_p), POINTER(c_int64), POINTER(c_void_p), POINTER(c_int64), c_int,
                                 POINTER(c_int), c_int, c_float, c_float, c_int, c_void_p]),
    "fx_gemm_ksum": (c_int, [c_int, POINTER(c_void_p), POINTER(c_int64), c_int, POINTER(c_void_p), POINTER(c_int64),
                             c_int, POINTER(c_int), c_void_p, c_int64, c_void_p, c_int64, c_int, c_int, c_float,
                             c_float, c_int, c_int, c_void_p]),
    "fx_copy_fields": (c_int, [c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_void_p]),
    "create_dispatcher": (c_void_p, [c_int, c_int]),
    "destroy_dispatcher": (None, [c_void_p]),
    "get_stats": (None, [c_void_p, POINTER(c_uint64)]),
    "dispatch_matmul": (c_int, [c_void_p, c_void_p, c_int, c_int, c_int, c_void_p, c_int, c_void_p, c_int,
                                c_void_p, c_int, c_void_p, c_int, c_void_p, c_size_t, c_int, c_int, c_int,
                                c_int, c_int, c_float, c_float, c_int, c_int]),
    "fx_host_alloc": (c_int, [c_size_t, POINTER(c_void_p)]),
    "fx_host_free": (c_int, [c_void_p]),
    "fx_stream_ring_create": (c_int, [c_int, POINTER(c_void_p)]),
    "fx_stream_ring_destroy": (c_int, [c_void_p]),
    "fx_adamw_stream_ws_bytes": (c_size_t, [c_int64, c_int, c_int, c_int, c_int, c_int]),
    "fx_adamw_stream_chunk": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int64, c_int,
                                      c_int, c_int, c_float, c_float, c_float, c_float, c_float, c_float,
                                      c_float, c_void_p, c_size_t, c_int64, c_int, c_void_p, c_void_p,
                                      c_void_p, c_void_p]),
    "fx_probe_ws_bytes": (c_size_t, []),
    "fx_probe_mfma_rate": (c_int, [c_int, c_int, c_void_p, c_size_t, POINTER(c_double), c_void_p]),
    "solve_scheduler": (c_double, [c_int, c_int, c_int, c_void_p, c_void_p, c_void_p, c_double, c_int, c_int,
                                   c_void_p]),
    "compute_buf_size": (c_int, [c_int, c_int, c_int, c_void_p, c_void_p, c_double, c_int]),
    "fx_swiglu_moe_bwd": (c_int, [c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int, c_void_p,
                                  c_int64, c_int, c_int64, c_int64, c_int64, c_int64, c_int, c_int,
                                  c_void_p]),
}

_lib = None


def exported_symbols() -> list[str]:
    """Names every build of the library must export."""
    return sorted(_SIGNATURES)


def lib() -> ctypes.CDLL:
    """Load (once) and return the native library; raise if it is not built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: build it with `make -C flextrain_amd/csrc` "
                "(or `python -c 'import __graft_entry__ as g; g.build()'`). "
                "There is no fallback compute path."
            )
        handle = ctypes.CDLL(LIB_PATH)
        for name, (restype, argtypes) in _SIGNATURES.items():
            fn = getattr(handle, name)  # AttributeError if the build lacks a symbol
            fn.restype = restype
            fn.argtypes = argtypes
        _lib = handle
    return _lib


def ptr(t: torch.Tensor | None):
    """Raw address of a tensor's first element, or NULL."""
    return None if t is None else t.data_ptr()


def stream_ptr(device=None) -> int:
    """The current torch stream of ``device`` as a raw ``hipStream_t``."""
    return torch.cuda.current_stream(device).cuda_stream


def check(rc: int, what: str) -> None:
    if rc != 0:
        raise RuntimeError(f"{what} failed (rc={rc}); see stderr for the reason")


def require_gpu(*tensors: torch.Tensor, op: str) -> None:
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise ValueError(f"{op}: tensors must be on the GPU (got device {t.device})")
