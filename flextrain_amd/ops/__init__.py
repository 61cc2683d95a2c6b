"""The ``flextrain_*`` op surface (flextrain/ops/__init__.py:14-120) for the
ops on the per-layer training compute path, backed by libflexhip.so."""
from __future__ import annotations

from .adamw import flextrain_adamw_step
from .glu import (
    flextrain_gelu_tanh_gated_bwd,
    flextrain_gelu_tanh_gated_fwd,
    flextrain_swiglu_bwd,
    flextrain_swiglu_fwd,
)
from .misc import flextrain_embedding_bwd, flextrain_silu_bwd
from .moe import (
    flextrain_copy_expert_counts,
    flextrain_fused_topk_softmax,
    flextrain_load_balance_bwd,
    flextrain_moe_gather,
    flextrain_moe_row_sources,
    flextrain_moe_router_gate_bwd,
    flextrain_moe_scatter,
    flextrain_moe_scatter_routing_weights,
    flextrain_moe_sort,
    flextrain_swiglu_moe_bwd,
    flextrain_swiglu_moe_bwd_prescaled,
    flextrain_swiglu_moe_fwd,
)
from .rmsnorm import (
    flextrain_rmsnorm_bwd,
    flextrain_rmsnorm_fwd,
    flextrain_rmsnorm_fwd_recompute,
)
from .softmax_ce import (
    flextrain_cross_entropy_loss,
    flextrain_logit_softcap_bwd,
    flextrain_logit_softcap_fwd,
    flextrain_softmax,
    flextrain_softmax_cross_entropy,
    flextrain_softmax_cross_entropy_loss,
)
from .rope import (
    build_rope_inv_freq,
    flextrain_rope_bwd,
    flextrain_rope_fwd,
    flextrain_rope_partial_bwd,
    flextrain_rope_partial_fwd,
)

from ..host_memory import destroy_pinned_tensor, pin_tensor

_dispatchers = {}


def __getattr__(name):
    """``dispatcher`` / ``dispatcher_secondary``: the two module-level GEMM dispatchers of the
    reference (flextrain/ops/_kernels/_matmul_dispatchers.py:3-4), created on first access instead
    of at import."""
    if name in ("dispatcher", "dispatcher_secondary"):
        if name not in _dispatchers:
            from ..matmul_dispatcher import CublasLtDispatcher
            _dispatchers[name] = CublasLtDispatcher(round_multiple=32)
        return _dispatchers[name]
    raise AttributeError(f"module {__name__!r} has no attribute {name!r}")


__all__ = [
    "build_rope_inv_freq",
    "destroy_pinned_tensor",
    "dispatcher",
    "dispatcher_secondary",
    "flextrain_embedding_bwd",
    "flextrain_silu_bwd",
    "pin_tensor",
    "flextrain_adamw_step",
    "flextrain_copy_expert_counts",
    "flextrain_cross_entropy_loss",
    "flextrain_fused_topk_softmax",
    "flextrain_load_balance_bwd",
    "flextrain_moe_gather",
    "flextrain_moe_row_sources",
    "flextrain_moe_router_gate_bwd",
    "flextrain_moe_scatter",
    "flextrain_moe_scatter_routing_weights",
    "flextrain_moe_sort",
    "flextrain_swiglu_moe_bwd",
    "flextrain_swiglu_moe_bwd_prescaled",
    "flextrain_swiglu_moe_fwd",
    "flextrain_gelu_tanh_gated_bwd",
    "flextrain_gelu_tanh_gated_fwd",
    "flextrain_rmsnorm_bwd",
    "flextrain_rmsnorm_fwd",
    "flextrain_rmsnorm_fwd_recompute",
    "flextrain_rope_bwd",
    "flextrain_rope_fwd",
    "flextrain_rope_partial_bwd",
    "flextrain_rope_partial_fwd",
    "flextrain_logit_softcap_bwd",
    "flextrain_logit_softcap_fwd",
    "flextrain_softmax",
    "flextrain_softmax_cross_entropy",
    "flextrain_softmax_cross_entropy_loss",
    "flextrain_swiglu_bwd",
    "flextrain_swiglu_fwd",
]
