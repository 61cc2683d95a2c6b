"""Dense gated FFN block: ``out = resid + W_2 @ act(W_1 @ h) * (W_3 @ h)``.

Host-side mirror of the reference block (flextrain/nn/blocks/ffn_dense.py:57-301): the same
method names, argument meaning, saved activations (``slot.x1`` / ``slot.x3``), the
``skip_grads`` / ``capture_xy`` contract and the hand-off of ``dx1_up`` / ``dx3_up`` through
``slot.aux``.  Every GEMM goes through the MFMA dispatcher (`dispatch_matmul`), with the residual
add folded into the down projection (``beta = 1`` on the residual operand), the gate and up projections run as one launch with the
activation in its epilogue when the shapes allow (``fuse_gate_up``), and the weight
gradients accumulated in place (``beta = 1`` on the gradient itself); the gated activation and
its backward are the SwiGLU / GELU-tanh kernels of :mod:`flextrain_amd.ops`.

``slot`` is any object with ``x1``, ``x3`` tensors ``(T, expert_dim)`` and an ``aux`` dict;
``ctx`` is anything with ``scratch(shape, dtype)`` or ``None`` (a fresh tensor is allocated).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Mapping, MutableMapping, Sequence

import torch

from . import ops
from .ops.grouped import dual_glu_supported, flextrain_gemm_dual_glu


@dataclass(frozen=True)
class SwiGLUConfig:
    d_model: int
    expert_dim: int
    compute_dtype: torch.dtype = torch.bfloat16
    master_dtype: torch.dtype | None = None
    grad_dtype: torch.dtype | None = None
    activation: str = "silu"          # "silu" (Llama / Qwen / Mistral) or "gelu_tanh" (Gemma 2 / 3)


@dataclass(frozen=True)
class ComputeCost:
    total_fwd_flops: int
    avoided_recompute_flops: tuple


def _stream_ptr(t):
    return torch.cuda.current_stream(t.device).cuda_stream


class SwiGLUFFN:
    """Gate / up / down projections around the gated activation."""

    def __init__(self, cfg: SwiGLUConfig, dispatcher=None, fuse_gate_up: bool = True):
        if cfg.activation not in ("silu", "gelu_tanh"):
            raise ValueError(f"SwiGLUFFN: unsupported activation {cfg.activation!r}")
        self.cfg = cfg
        self._dispatcher = dispatcher
        self.fuse_gate_up = fuse_gate_up

    @property
    def dispatcher(self):
        return self._dispatcher if self._dispatcher is not None else ops.dispatcher

    def _mm(self, A, B, D, C=None, beta=0.0):
        return self.dispatcher.matmul(_stream_ptr(A), A=A, B=B, C=C, D=D, alpha=1.0, beta=beta)

    def _act_fwd(self, x1, x3, out):
        if self.cfg.activation == "silu":
            return ops.flextrain_swiglu_fwd(x1, x3, out=out)
        return ops.flextrain_gelu_tanh_gated_fwd(x1, x3, out=out)

    def _act_bwd(self, x1, x3, dout):
        if self.cfg.activation == "silu":
            return ops.flextrain_swiglu_bwd(x1, x3, dout, store_activations=True)
        return ops.flextrain_gelu_tanh_gated_bwd(x1, x3, dout, store_activations=True)

    # -------------------------------------------------------------- forward
    def fwd(self, ffn_norm_output, weights: Mapping[str, torch.Tensor], attn_output_with_residual, out_tensor, slot,
            ctx=None):
        """Writes ``slot.x1``, ``slot.x3`` and returns ``out_tensor`` (which may be the residual
        tensor itself: the down projection reads each residual element before writing it)."""
        scratch = ctx.scratch(slot.x1.shape, slot.x1.dtype) if ctx is not None else torch.empty_like(slot.x1)
        w1, w3 = weights["w_1"], weights["w_3"]
        if self.fuse_gate_up and dual_glu_supported(ffn_norm_output, w1, w3, slot.x1, slot.x3, scratch):
            # one launch: both projections and the activation from their rounded results
            act = flextrain_gemm_dual_glu(ffn_norm_output, w1, w3, slot.x1, slot.x3, scratch,
                                          activation=self.cfg.activation, gate_first=True)
        else:
            self._mm(ffn_norm_output, w1, slot.x1)
            self._mm(ffn_norm_output, w3, slot.x3)
            act = self._act_fwd(slot.x1, slot.x3, scratch)
        return self._mm(act, weights["w_2"], out_tensor, C=attn_output_with_residual, beta=1.0)

    def fwd_recompute_x1x3(self, ffn_norm_output, weights, slot, *, recompute_x1: bool, recompute_x3: bool) -> None:
        if recompute_x1:
            self._mm(ffn_norm_output, weights["w_1"], slot.x1)
        if recompute_x3:
            self._mm(ffn_norm_output, weights["w_3"], slot.x3)

    # ------------------------------------------------------------- backward
    def bwd(self, dy_resid, weights, grads: MutableMapping[str, torch.Tensor], slot, *,
            skip_grads: frozenset = frozenset(), capture_xy: dict | None = None):
        """Accumulates ``g_2`` and returns the gradient with respect to the FFN-norm output;
        ``dx1_up`` / ``dx3_up`` are left in ``slot.aux`` for :meth:`bwd_accumulate_w1_w3_grads`."""
        T = dy_resid.shape[0]
        dx_up_act = torch.empty((T, self.cfg.expert_dim), dtype=dy_resid.dtype, device=dy_resid.device)
        self._mm(dy_resid, weights["w_2"].T, dx_up_act)
        dx1_up, dx3_up, fwd_act = self._act_bwd(slot.x1, slot.x3, dx_up_act)
        if "g_2" in skip_grads:
            if capture_xy is not None:
                capture_xy["g_2"] = (fwd_act.clone(), dy_resid.clone())
        else:
            self._mm(fwd_act.T, dy_resid, grads["g_2"], C=grads["g_2"], beta=1.0)
        dx_ffn_norm_up = torch.empty_like(dy_resid)
        fused = getattr(self.dispatcher, "matmul_sum", None)
        if fused is not None:    # both products in one launch, summed in fp32 and rounded once
            fused(_stream_ptr(dx1_up), [dx1_up, dx3_up], [weights["w_1"].T, weights["w_3"].T], D=dx_ffn_norm_up)
        else:
            self._mm(dx1_up, weights["w_1"].T, dx_ffn_norm_up)
            self._mm(dx3_up, weights["w_3"].T, dx_ffn_norm_up, C=dx_ffn_norm_up, beta=1.0)
        slot.aux["bwd_dx1_up"] = dx1_up
        slot.aux["bwd_dx3_up"] = dx3_up
        return dx_ffn_norm_up

    def bwd_accumulate_w1_w3_grads(self, ffn_norm_output, grads, slot, *, skip_grads: frozenset = frozenset(),
                                   capture_xy: dict | None = None) -> None:
        todo = []
        for name, dy_key in (("g_1", "bwd_dx1_up"), ("g_3", "bwd_dx3_up")):
            dy = slot.aux[dy_key]
            if name in skip_grads:
                if capture_xy is not None:
                    capture_xy[name] = (ffn_norm_output, dy)
            else:
                todo.append((name, dy))
        shared = getattr(self.dispatcher, "matmul_shared_a", None)
        if len(todo) == 2 and shared is not None:
            # one grid for both: 2 x 3.5 rounds of workgroups (Llama-3.1-8B shapes) become 7 full ones
            g = [grads[n] for n, _ in todo]
            shared(_stream_ptr(ffn_norm_output), ffn_norm_output.T, [dy for _, dy in todo], g, Cs=g, alpha=1.0, beta=1.0)
            todo = []
        for name, dy in todo:
            self._mm(ffn_norm_output.T, dy, grads[name], C=grads[name], beta=1.0)
        del slot.aux["bwd_dx1_up"]
        del slot.aux["bwd_dx3_up"]

    # ------------------------------------------------------- FLOP accounting
    def compute_cost(self, seq_lens_host: Sequence[int], max_tier: int) -> ComputeCost:
        """Forward FLOPs of the block for the chunk's sequences, and per save tier the FLOPs a
        backward pass no longer has to recompute (flextrain/nn/blocks/ffn_dense.py:280-301)."""
        cfg = self.cfg
        avoided = [0] * (max_tier + 1)
        total = 0
        for seq_len in seq_lens_host:
            up_gate = 2 * seq_len * cfg.d_model * cfg.expert_dim * 2
            total += up_gate
            if max_tier >= 3:
                avoided[3] += up_gate
            total += 2 * seq_len * cfg.expert_dim * cfg.d_model
        return ComputeCost(total_fwd_flops=total, avoided_recompute_flops=tuple(avoided))
