"""AdamW behind the reference optimizer interface (flextrain/optim/adamw.py:28-154)
and the streamed step of one host-offloaded chunk (the per-layer part of
``ActiveModel.step``, flextrain/engine/active_model.py:486-655)."""
from __future__ import annotations

from dataclasses import dataclass
from typing import Mapping, MutableMapping

import torch

from ._lib import check, dtype_enum, lib
from .ops.adamw import flextrain_adamw_step
from .streams import StreamBundle


@dataclass(frozen=True)
class AdamWHyperparams:
    """flextrain/optim/adamw.py:28-42."""
    lr: float = 1e-4
    beta1: float = 0.9
    beta2: float = 0.95
    eps: float = 1e-8
    weight_decay: float = 0.001
    check_error: bool = False


def state_key(state_name: str, param_name: str) -> str:
    """``o_adam_m`` + ``w_q`` -> ``o_adam_m_q``: the leading ``w_`` of the parameter name
    is dropped (flextrain/optim/base.py:78-88)."""
    stripped = param_name[2:] if param_name.startswith("w_") else param_name
    return f"{state_name}_{stripped}"


class AdamW:
    """``step(param_spec, master, grads, state, step_num=...)`` loops over the
    non-frozen tensors of ``param_spec`` (objects with ``.name`` and ``.frozen``) and
    calls :func:`flextrain_adamw_step` on each; returns 0, or the first non-zero
    kernel status.  flextrain/optim/adamw.py:98-154."""

    def __init__(self, hp: AdamWHyperparams | None = None, *, state_dtype: torch.dtype = torch.bfloat16) -> None:
        self.hp = hp or AdamWHyperparams()
        self.state_dtype = state_dtype

    def step(self, param_spec, master: Mapping[str, torch.Tensor], grads: Mapping[str, torch.Tensor],
             state: MutableMapping[str, torch.Tensor], *, step_num: int) -> int:
        for p in param_spec.tensors:
            if p.frozen:
                continue
            grad_key = "g_" + p.name[2:] if p.name.startswith("w_") else "g_" + p.name
            ret = flextrain_adamw_step(master[p.name], grads[grad_key], state[state_key("o_adam_m", p.name)],
                                       state[state_key("o_adam_v", p.name)], lr=self.hp.lr, beta1=self.hp.beta1,
                                       beta2=self.hp.beta2, eps=self.hp.eps, weight_decay=self.hp.weight_decay,
                                       step=step_num, check_error=self.hp.check_error)
            if ret != 0:
                return ret
        return 0


class AdamWStreamWorkspace:
    """Device staging memory for :func:`flextrain_adamw_step_streamed` together with the
    per-slot events that order one call after the previous one on the same memory, so
    calls for successive chunks / layers may follow each other without synchronising."""

    def __init__(self, sub_elems, n_slots, p_dtype, g_dtype, state_dtype, stage_bf16_copy, device):
        import ctypes

        self.sub_elems, self.n_slots = int(sub_elems), int(n_slots)
        nbytes = int(lib().fx_adamw_stream_ws_bytes(self.sub_elems, self.n_slots, dtype_enum(p_dtype),
                                                    dtype_enum(g_dtype), dtype_enum(state_dtype),
                                                    1 if stage_bf16_copy else 0))
        self.buffer = torch.empty(nbytes, dtype=torch.uint8, device=device)
        # the allocating stream may still own the block's previous life: order every stream after it
        self.alloc_event = torch.cuda.current_stream(device).record_event()
        handle = ctypes.c_void_p()
        check(lib().fx_stream_ring_create(self.n_slots, ctypes.byref(handle)), "fx_stream_ring_create")
        self._ring = handle

    def numel(self) -> int:
        return self.buffer.numel()

    def data_ptr(self) -> int:
        return self.buffer.data_ptr()

    def close(self) -> None:
        if self._ring is not None:
            lib().fx_stream_ring_destroy(self._ring)
            self._ring = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


def adamw_stream_workspace(sub_elems, n_slots, p_dtype, g_dtype, state_dtype, stage_bf16_copy, device):
    """Device staging workspace for :func:`flextrain_adamw_step_streamed`."""
    return AdamWStreamWorkspace(sub_elems, n_slots, p_dtype, g_dtype, state_dtype, stage_bf16_copy, device)


def flextrain_adamw_step_streamed(params, grads, exp_avgs, exp_avg_sqs, *, streams: StreamBundle, lr=1e-4, beta1=0.9,
                                  beta2=0.95, eps=1e-8, weight_decay=0.001, step=1, params_bf16_out=None,
                                  workspace=None, sub_elems=4 * 1024 * 1024, n_slots=3):
    """AdamW on one flat chunk whose ``params`` / ``grads`` / moments live in PINNED HOST
    memory: sub-chunks are copied in on ``streams.inbound``, updated on
    ``streams.compute`` and copied back on ``streams.outbound`` with all three
    overlapping.  ``params_bf16_out`` (optional, bf16, pinned host or device) receives the
    updated parameters rounded to bf16.  Enqueues only; the host tensors hold the result
    after ``streams.outbound.synchronize()``.  Returns 0.

    ``workspace`` (:func:`adamw_stream_workspace`) may be passed to successive calls
    without any synchronisation between them: its slot events order each call's copies
    after the previous call's kernels and copies on the same staging memory.  A raw
    ``torch.uint8`` tensor is accepted too; its first copies then wait for everything
    enqueued so far on ``compute`` and ``outbound``.  The caller still orders the three
    streams after whatever PRODUCED the host tensors (e.g. a gradient offload)."""
    n = params.numel()
    for t, name in ((params, "params"), (grads, "grads"), (exp_avgs, "exp_avgs"), (exp_avg_sqs, "exp_avg_sqs")):
        if t.is_cuda or not t.is_pinned():
            raise ValueError(f"{name} must be a pinned host tensor")
        if t.numel() != n or not t.is_contiguous():
            raise ValueError(f"{name} must be contiguous with {n} elements")
    if exp_avgs.dtype != exp_avg_sqs.dtype:
        raise TypeError("exp_avgs and exp_avg_sqs must share a dtype")
    out_on_device = 0
    if params_bf16_out is not None:
        if params_bf16_out.dtype != torch.bfloat16 or params_bf16_out.numel() != n or not params_bf16_out.is_contiguous():
            raise ValueError(f"params_bf16_out must be contiguous bfloat16 with {n} elements")
        if params_bf16_out.is_cuda:
            out_on_device = 1
        elif not params_bf16_out.is_pinned():
            raise ValueError("params_bf16_out must be on the GPU or in pinned host memory")
    if n == 0:
        return 0
    device = streams.compute.device
    stage = params_bf16_out is not None and not out_on_device
    ring = None
    if workspace is None:
        sub_elems = max(8, min(int(sub_elems), (n + 7) // 8 * 8))
        workspace = AdamWStreamWorkspace(sub_elems, n_slots, params.dtype, grads.dtype, exp_avgs.dtype, stage, device)
    if isinstance(workspace, AdamWStreamWorkspace):
        sub_elems, n_slots, ring, buf = workspace.sub_elems, workspace.n_slots, workspace._ring, workspace.buffer
        if workspace.alloc_event is not None:
            for s in (streams.inbound, streams.compute, streams.outbound):
                s.wait_event(workspace.alloc_event)
            workspace.alloc_event = None
    else:
        sub_elems = max(8, min(int(sub_elems), (n + 7) // 8 * 8))
        buf = workspace
    step = max(1, step)
    rc = lib().fx_adamw_stream_chunk(
        params.data_ptr(), grads.data_ptr(), exp_avgs.data_ptr(), exp_avg_sqs.data_ptr(),
        params_bf16_out.data_ptr() if params_bf16_out is not None else None, out_on_device, n,
        dtype_enum(params.dtype), dtype_enum(grads.dtype), dtype_enum(exp_avgs.dtype), lr, beta1, beta2, eps,
        weight_decay, 1.0 - beta1 ** step, 1.0 - beta2 ** step, buf.data_ptr(), buf.numel(), sub_elems,
        n_slots, streams.inbound.cuda_stream, streams.compute.cuda_stream, streams.outbound.cuda_stream, ring)
    check(rc, "fx_adamw_stream_chunk")
    # the staging buffer must outlive the enqueued work
    buf.record_stream(streams.inbound)
    buf.record_stream(streams.compute)
    buf.record_stream(streams.outbound)
    return 0
