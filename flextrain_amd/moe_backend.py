"""The MoE expert-compute backend protocol of the reference
(flextrain/ops/moe_backend.py:41-197) and its in-tree implementation
(:205-520) on top of the grouped kernels.

A backend owns scatter + per-expert MLP + gather.  Slot fields, the
``slot.aux["moe_dprobs"]`` hand-off, the ``lora_capture`` dictionary keys and the
pinned host counts kept in ``chunk_extra`` follow the reference.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Callable, Mapping, MutableMapping, Protocol, runtime_checkable

import torch

from . import full_moe
from .ops.moe import flextrain_moe_gather, flextrain_moe_row_sources, flextrain_moe_scatter


@dataclass(frozen=True)
class ActivationField:
    """Stand-in for ``flextrain.core.activation_schema.ActivationField`` (the
    planner type the reference backend returns from ``activation_fields``):
    name, shape function of (num_tokens, d_model), dtype, save tier, token axis."""
    name: str
    shape_fn: Callable[[int, int], tuple]
    dtype: torch.dtype
    tier: int = 0
    token_axis: int | None = 0


@runtime_checkable
class MoEExpertCompute(Protocol):
    """flextrain/ops/moe_backend.py:41-197."""

    name: str

    @property
    def supports_residual_in_gather(self) -> bool: ...

    @property
    def supported_tiers(self) -> frozenset: ...

    def activation_fields(self, num_experts, top_k, expert_dim, d_model, compute_dtype) -> tuple: ...

    def fwd(self, x, router_weights, chosen_experts, weights, *, out, residual, slot, chunk_extra, layer_id,
            primary_stream, secondary_stream, scratch_fn) -> None: ...

    def fwd_recompute(self, x, weights, *, slot, chunk_extra, layer_id, primary_stream, secondary_stream,
                      scratch_fn) -> Any: ...

    def expert_counts_gpu(self, slot) -> torch.Tensor: ...

    def bwd(self, dy, x, weights, grads, *, slot, chunk_extra, layer_id, primary_stream, secondary_stream,
            scratch_fn, dx=None, recompute_handoff=None, lora_capture=None) -> torch.Tensor: ...


class FlextrainMoEExpertCompute:
    """flextrain/ops/moe_backend.py:205-520.  Backend-private slot fields:
    ``index_mapping (T,K) int32``, ``expert_counts (E,) int32``,
    ``scattered_router_weights (TK,1)``; shared: ``x_up (TK,2F)``."""

    name = "flextrain"
    _CHUNK_EXTRA_HOST_COUNTS = "flextrain.moe.expert_counts_host"

    @property
    def supports_residual_in_gather(self) -> bool:
        return True

    @property
    def supported_tiers(self) -> frozenset:
        return frozenset({0, 1, 2, 3})

    def activation_fields(self, num_experts, top_k, expert_dim, d_model, compute_dtype):
        return (
            ActivationField("expert_counts", lambda n, d: (num_experts,), torch.int32, tier=0, token_axis=None),
            ActivationField("index_mapping", lambda n, d: (n, top_k), torch.int32, tier=0),
            ActivationField("scattered_router_weights", lambda n, d: (n * top_k, 1), compute_dtype, tier=0,
                            token_axis=None),
        )

    def expert_counts_gpu(self, slot):
        return slot.expert_counts

    @classmethod
    def _host_counts(cls, chunk_extra, layer_id, num_experts):
        per_layer = chunk_extra.setdefault(cls._CHUNK_EXTRA_HOST_COUNTS, {})
        buf = per_layer.get(layer_id)
        if buf is None:
            buf = torch.zeros(num_experts, dtype=torch.int32, pin_memory=True)
            per_layer[layer_id] = buf
        return buf

    def fwd(self, x, router_weights, chosen_experts, weights, *, out, residual, slot, chunk_extra, layer_id,
            primary_stream, secondary_stream, scratch_fn):
        num_experts = weights["w_up"].shape[0]
        expert_dim = weights["w_down"].shape[2]
        num_tokens, d_model = x.shape
        TK = num_tokens * router_weights.shape[1]
        host_counts = self._host_counts(chunk_extra, layer_id, num_experts)
        scattered_x = scratch_fn((TK, d_model), x.dtype)
        srw = slot.scattered_router_weights[:TK, :]
        # When the fused up-projection can take the operands it reads the token rows of x in place
        # through the row map, and the expert-sorted copy of x (one write and one read of TK x d) is
        # never made; scattered_x then only receives the down-projection's result.
        gathered = full_moe.gathered_up_projection_supported(x, weights["w_up"], slot.x_up[:TK], expert_dim)
        indices, _ = full_moe.dispatch_scatter(
            x, router_weights, chosen_experts, num_experts=num_experts, index_mapping=slot.index_mapping,
            expert_counts_gpu=slot.expert_counts, expert_counts_cpu=host_counts,
            scattered_x_out=None if gathered else scattered_x,
            scattered_router_weights_out=srw, sync=False)   # nothing below reads the counts on the host
        row_sources = flextrain_moe_row_sources(indices, out=scratch_fn((TK,), torch.int32)) if gathered else None
        x_act = scratch_fn((TK, expert_dim), x.dtype)
        full_moe.swiglu_expert_loop_fwd(
            scattered_x=scattered_x, x_preact_buf=slot.x_up, w_up=weights["w_up"], w_down=weights["w_down"],
            expert_counts_cpu=host_counts, primary_stream=primary_stream, secondary_stream=secondary_stream,
            x_act_even=x_act, x_act_odd=x_act, expert_counts_gpu=slot.expert_counts,
            gather_from=x if gathered else None, row_sources=row_sources)
        full_moe.combine_gather(scattered_x, indices, router_weights=router_weights,
                                residual=residual.view(-1, d_model) if residual is not None else None,
                                out_tensor=out)

    def fwd_recompute(self, x, weights, *, slot, chunk_extra, layer_id, primary_stream, secondary_stream,
                      scratch_fn):
        num_tokens, d_model = x.shape
        TK = num_tokens * slot.index_mapping.shape[1]
        host_counts = self._host_counts(chunk_extra, layer_id, weights["w_up"].shape[0])
        scattered_x = scratch_fn((TK, d_model), x.dtype)
        flextrain_moe_scatter(x, slot.index_mapping, out=scattered_x)
        full_moe.swiglu_expert_loop_recompute_x_up(
            scattered_x=scattered_x, x_preact_buf=slot.x_up, w_up=weights["w_up"], expert_counts_cpu=host_counts,
            primary_stream=primary_stream, secondary_stream=secondary_stream,
            expert_counts_gpu=slot.expert_counts)
        return scattered_x

    def bwd(self, dy, x, weights, grads, *, slot, chunk_extra, layer_id, primary_stream, secondary_stream,
            scratch_fn, dx=None, recompute_handoff=None, lora_capture=None):
        num_tokens, d_model = dy.shape
        top_k = slot.index_mapping.shape[1]
        TK = num_tokens * top_k
        num_experts = weights["w_up"].shape[0]
        expert_dim = weights["w_down"].shape[2]
        host_counts = self._host_counts(chunk_extra, layer_id, num_experts)
        srw = slot.scattered_router_weights[:TK, :]
        dprobs = torch.zeros_like(srw)
        dx_up_up_grouped = scratch_fn((TK, 2 * expert_dim), dy.dtype)
        dx_pre_grouped = scratch_fn((TK, d_model), dy.dtype)
        # When the fused launches can take the operands they read the token rows of dy and x in place
        # through the row map, and neither expert-sorted copy (one write and two reads of TK x d each) is
        # made.  The LoRA capture hands the sorted copies on and a recompute hand-off already is one, so
        # those two cases keep the scatter launches.
        gathered = (lora_capture is None and recompute_handoff is None
                    and full_moe.gathered_backward_supported(dy, x, weights["w_down"], slot.x_up[:TK], srw,
                                                             dx_up_up_grouped, dprobs))
        scattered_upstream = scattered_x = row_sources = None
        if gathered:
            row_sources = flextrain_moe_row_sources(slot.index_mapping, out=scratch_fn((TK,), torch.int32))
        else:
            scattered_upstream = scratch_fn((TK, d_model), dy.dtype)
            flextrain_moe_scatter(dy, slot.index_mapping, out=scattered_upstream)
            if recompute_handoff is not None:
                scattered_x = recompute_handoff
            else:
                scattered_x = scratch_fn((TK, d_model), dy.dtype)
                flextrain_moe_scatter(x, slot.index_mapping, out=scattered_x)
        full_moe.swiglu_expert_loop_bwd(
            scattered_upstream=scattered_upstream, scattered_x=scattered_x, x_preact_buf=slot.x_up[:TK], srw=srw,
            dprobs=dprobs, w_up=weights["w_up"], w_down=weights["w_down"], grads=grads,
            expert_counts_cpu=host_counts, dx_up_up_grouped=dx_up_up_grouped, dx_pre_grouped=dx_pre_grouped,
            expert_dim=expert_dim, primary_stream=primary_stream, secondary_stream=secondary_stream,
            expert_counts_gpu=slot.expert_counts, gather_dy=dy if gathered else None,
            gather_x=x if gathered else None, row_sources=row_sources)
        if lora_capture is not None:
            lora_capture["scattered_x_grouped"] = scattered_x
            lora_capture["dx_up_up_grouped"] = dx_up_up_grouped
            lora_capture["scattered_upstream_grouped"] = scattered_upstream
            lora_capture["x_up_grouped"] = slot.x_up[:TK]
            lora_capture["expert_offsets"] = self.expert_counts_gpu(slot).cumsum(0).to(torch.int32)
            lora_capture["TK"] = TK
        if dx is None:
            dx = torch.empty_like(dy)
        flextrain_moe_gather(dx_pre_grouped, slot.index_mapping, out=dx)
        slot.aux["moe_dprobs"] = dprobs
        return dx
