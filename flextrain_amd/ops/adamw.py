"""AdamW step on a flat chunk behind the reference signature
(flextrain/ops/_kernels/adamw.py:62-102)."""
from __future__ import annotations

import torch

from .._lib import check, dtype_enum, lib, ptr, stream_ptr


def flextrain_adamw_step(params, grads, exp_avgs, exp_avg_sqs, lr=1e-4, beta1=0.9, beta2=0.95,
                         eps=1e-8, weight_decay=0.001, step=1, check_error=False,
                         params_bf16_out=None):
    """Update ``params``, ``exp_avgs``, ``exp_avg_sqs`` in place; return 0, or
    -1 (and leave everything untouched) when ``check_error`` is set and a
    gradient is NaN/Inf.  ``params_bf16_out`` (extension, default off) also
    receives the updated parameters rounded to bf16."""
    if not params.is_cuda:
        raise ValueError("Parameters must be on CUDA")
    n = params.numel()
    for t, name in ((grads, "grads"), (exp_avgs, "exp_avgs"), (exp_avg_sqs, "exp_avg_sqs"),
                    (params_bf16_out, "params_bf16_out")):
        if t is None:
            continue
        if not t.is_cuda or t.numel() != n:
            raise ValueError(f"{name} must be a CUDA tensor with {n} elements")
    for t, name in ((params, "params"), (grads, "grads"), (exp_avgs, "exp_avgs"),
                    (exp_avg_sqs, "exp_avg_sqs"), (params_bf16_out, "params_bf16_out")):
        if t is not None and not t.is_contiguous():
            raise ValueError(f"{name} must be contiguous")
    if exp_avgs.dtype != exp_avg_sqs.dtype:
        raise TypeError("exp_avgs and exp_avg_sqs must share a dtype")
    if params_bf16_out is not None and params_bf16_out.dtype != torch.bfloat16:
        raise TypeError("params_bf16_out must be bfloat16")
    step = max(1, step)
    bc1 = 1.0 - (beta1 ** step)
    bc2 = 1.0 - (beta2 ** step)
    L = lib()
    s = stream_ptr(params.device)
    if check_error:
        flag = torch.zeros(1, dtype=torch.int32, device=params.device)
        check(L.fx_nonfinite_flag(ptr(grads), n, dtype_enum(grads.dtype), ptr(flag), s), "fx_nonfinite_flag")
        if int(flag.item()) != 0:
            print("Grad is inf or nan")
            return -1
    rc = L.fx_adamw_step(ptr(params), ptr(grads), ptr(exp_avgs), ptr(exp_avg_sqs),
                         ptr(params_bf16_out), n, dtype_enum(params.dtype), dtype_enum(grads.dtype),
                         dtype_enum(exp_avgs.dtype), lr, beta1, beta2, eps, weight_decay, bc1, bc2, s)
    check(rc, "fx_adamw_step")
    return 0
