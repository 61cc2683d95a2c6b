"""Everything of the grouped-query attention block except the attention core itself.

Mirror of the GEMM / norm / RoPE / epilogue work in ``GQAAttentionBlock``
(flextrain/nn/blocks/attention.py:392-823): the Q/K/V projections with the Qwen2 biases, the
Qwen3 per-head QK-norm, in-place RoPE, the output projection with the residual folded into the
GEMM epilogue (``beta = 1`` on the residual operand, attention.py:493-500), and the matching
backward halves (attention.py:614-629 and :712-775) plus the deferred weight gradients
(:777-823).  The attention core (flash-attn in the reference, a third-party kernel) sits between
the two halves and is the caller's: ``fwd`` / ``bwd`` take it as a callable.

Names and argument meaning follow the reference: ``weights`` holds ``w_q w_k w_v w_o`` stored
``(in, out)`` (and ``b_q b_k b_v``, ``w_q_norm w_k_norm`` when configured), ``grads`` holds
``g_q g_k g_v g_o`` (``g_b_*``, ``g_q_norm``, ``g_k_norm``) and is accumulated into, ``slot`` is any
object with ``xq (T, n_heads, head_dim)``, ``xk`` / ``xv (T, n_kv_heads, head_dim)``,
``attn_result (T, n_heads, head_dim)``, ``xo (T, d_model)``, ``q_norm_rstd`` / ``k_norm_rstd`` and
an ``aux`` dict.  Every GEMM goes through the MFMA dispatcher.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Callable, Mapping, MutableMapping

import torch

from . import ops


@dataclass(frozen=True)
class GQAProjectionConfig:
    d_model: int
    n_heads: int
    n_kv_heads: int
    head_dim: int
    rope_theta: float = 500000.0
    rope_scaling: Mapping | None = None
    qkv_bias: bool = False            # Qwen2: biases added after the projections
    qk_norm: bool = False             # Qwen3: per-head RMSNorm on Q and K before RoPE
    rms_norm_eps: float = 1e-6

    @property
    def attn_dim(self) -> int:
        return self.n_heads * self.head_dim

    @property
    def kv_dim(self) -> int:
        return self.n_kv_heads * self.head_dim


def _stream_ptr(t: torch.Tensor) -> int:
    return torch.cuda.current_stream(t.device).cuda_stream


class GQAAttentionProjections:
    """The two halves of the attention block around its core."""

    q_rstd_name = "q_norm_rstd"
    k_rstd_name = "k_norm_rstd"

    def __init__(self, cfg: GQAProjectionConfig, dispatcher=None):
        if cfg.n_heads % cfg.n_kv_heads:
            raise ValueError("n_heads must be a multiple of n_kv_heads")
        self.cfg = cfg
        self._dispatcher = dispatcher
        self._inv_freq: torch.Tensor | None = None

    @property
    def dispatcher(self):
        return self._dispatcher if self._dispatcher is not None else ops.dispatcher

    def _mm(self, A, B, D, C=None, beta=0.0):
        return self.dispatcher.matmul(_stream_ptr(A), A=A, B=B, C=C, D=D, alpha=1.0, beta=beta)

    def _mm_shared(self, A, Bs, Ds, Cs=None, beta=0.0):
        """Products that share ``A`` (key / value projections, their weight gradients): one launch
        where the dispatcher offers it, since each alone is too small to fill the GPU."""
        shared = getattr(self.dispatcher, "matmul_shared_a", None)
        if shared is not None:
            return shared(_stream_ptr(A), A, Bs, Ds, Cs=Cs, alpha=1.0, beta=beta)
        for i, B in enumerate(Bs):
            self._mm(A, B, Ds[i], C=None if Cs is None else Cs[i], beta=beta)
        return Ds

    def _mm_sum(self, As, Bs, D):
        """``D = sum_i As[i] @ Bs[i]``: one launch with a single rounding where the dispatcher offers
        it, else the reference's chain of accumulating calls (attention.py:760-775)."""
        fused = getattr(self.dispatcher, "matmul_sum", None)
        if fused is not None:
            return fused(_stream_ptr(As[0]), As, Bs, D=D)
        self._mm(As[0], Bs[0], D)
        for A, B in zip(As[1:], Bs[1:]):
            self._mm(A, B, D, C=D, beta=1.0)
        return D

    def _rope_freqs(self, device) -> torch.Tensor:
        """inv_freq of the configured RoPE, built once (attention.py:373-390)."""
        if self._inv_freq is None or self._inv_freq.device != device:
            self._inv_freq = ops.build_rope_inv_freq(self.cfg.head_dim, self.cfg.rope_theta,
                                                     self.cfg.rope_scaling).to(device)
        return self._inv_freq

    # -------------------------------------------------------------- forward
    def fwd_qkv(self, attn_norm_output, seq_positions, weights: Mapping[str, torch.Tensor], slot):
        """Projections, biases, QK-norm and RoPE into ``slot.xq / xk / xv`` (attention.py:424-463)."""
        cfg = self.cfg
        xq2d, xk2d, xv2d = slot.xq.view(-1, cfg.attn_dim), slot.xk.view(-1, cfg.kv_dim), slot.xv.view(-1, cfg.kv_dim)
        self._mm(attn_norm_output, weights["w_q"], xq2d)
        self._mm_shared(attn_norm_output, [weights["w_k"], weights["w_v"]], [xk2d, xv2d])
        if cfg.qkv_bias:
            xq2d.add_(weights["b_q"])
            xk2d.add_(weights["b_k"])
            xv2d.add_(weights["b_v"])
        if cfg.qk_norm:
            ops.flextrain_rmsnorm_fwd(xq2d, weights["w_q_norm"], head_dim=cfg.head_dim, output=xq2d,
                                      rstd=getattr(slot, self.q_rstd_name), rms_norm_eps=cfg.rms_norm_eps)
            ops.flextrain_rmsnorm_fwd(xk2d, weights["w_k_norm"], head_dim=cfg.head_dim, output=xk2d,
                                      rstd=getattr(slot, self.k_rstd_name), rms_norm_eps=cfg.rms_norm_eps)
        ops.flextrain_rope_fwd([slot.xq, slot.xk], seq_positions, self._rope_freqs(attn_norm_output.device))
        return slot.xq, slot.xk, slot.xv

    def fwd_recompute_q(self, attn_norm_output, seq_positions, weights, slot):
        """Q again from the norm output and the saved rstd (attention.py:502-536)."""
        cfg = self.cfg
        xq2d = slot.xq.view(-1, cfg.attn_dim)
        self._mm(attn_norm_output, weights["w_q"], xq2d)
        if cfg.qkv_bias:
            xq2d.add_(weights["b_q"])
        if cfg.qk_norm:
            ops.flextrain_rmsnorm_fwd_recompute(xq2d, weights["w_q_norm"], getattr(slot, self.q_rstd_name),
                                                head_dim=cfg.head_dim, output=xq2d)
        ops.flextrain_rope_fwd([slot.xq], seq_positions, self._rope_freqs(attn_norm_output.device))
        return slot.xq

    def fwd_o(self, x_resid, weights, slot):
        """``slot.xo = x_resid + attn_result @ w_o`` in one GEMM (attention.py:493-500, :567-581)."""
        return self._mm(slot.attn_result.view(-1, self.cfg.attn_dim), weights["w_o"], slot.xo, C=x_resid, beta=1.0)

    def fwd(self, x_resid, attn_norm_output, seq_positions, weights, slot, attention_fwd: Callable):
        """Whole block; ``attention_fwd(q, k, v, out)`` writes ``slot.attn_result``."""
        q, k, v = self.fwd_qkv(attn_norm_output, seq_positions, weights, slot)
        attention_fwd(q, k, v, slot.attn_result)
        return self.fwd_o(x_resid, weights, slot)

    # ------------------------------------------------------------- backward
    def bwd_o(self, dx_resid, weights, grads: MutableMapping[str, torch.Tensor], slot, *,
              skip_grads: frozenset = frozenset(), capture_xy: dict | None = None):
        """``g_o += attn_result^T dx_resid`` and the gradient entering the attention core,
        ``(T, n_heads, head_dim)`` (attention.py:614-629)."""
        cfg = self.cfg
        T = dx_resid.shape[0]
        attn_result = slot.attn_result.view(T, cfg.attn_dim)
        if "g_o" in skip_grads:
            if capture_xy is not None:
                capture_xy["g_o"] = (attn_result, dx_resid.clone())
        else:
            self._mm(attn_result.T, dx_resid, grads["g_o"], C=grads["g_o"], beta=1.0)
        dx_up_attn = torch.empty((T, cfg.attn_dim), dtype=dx_resid.dtype, device=dx_resid.device)
        self._mm(dx_resid, weights["w_o"].T, dx_up_attn)
        return dx_up_attn.view(T, cfg.n_heads, cfg.head_dim)

    def bwd_qkv(self, dq, local_dk, local_dv, seq_positions, weights, grads, slot, attn_norm_output=None):
        """From the core's ``dq / dk / dv`` (modified in place) to the gradient with respect to the
        attention-norm output: RoPE backward, QK-norm backward on recomputed pre-norm Q / K, bias
        gradients, three accumulating GEMMs (attention.py:712-775).  The projections' own
        gradients are left in ``slot.aux`` for :meth:`bwd_accumulate_qkv_grads`."""
        cfg = self.cfg
        T = dq.shape[0]
        dq_view, dk_view = ops.flextrain_rope_bwd(
            [dq.view(T, cfg.n_heads, cfg.head_dim), local_dk.view(T, cfg.n_kv_heads, cfg.head_dim)],
            seq_positions, self._rope_freqs(dq.device))
        dq2d, dk2d, dv2d = dq_view.view(T, cfg.attn_dim), dk_view.view(T, cfg.kv_dim), local_dv.view(T, cfg.kv_dim)
        if cfg.qk_norm:
            if attn_norm_output is None:
                raise ValueError("bwd_qkv requires attn_norm_output when cfg.qk_norm=True "
                                 "(the pre-norm Q / K are recomputed from it)")
            xq_pre = torch.empty((T, cfg.attn_dim), dtype=attn_norm_output.dtype, device=dq.device)
            xk_pre = torch.empty((T, cfg.kv_dim), dtype=attn_norm_output.dtype, device=dq.device)
            self._mm(attn_norm_output, weights["w_q"], xq_pre)
            self._mm(attn_norm_output, weights["w_k"], xk_pre)
            if cfg.qkv_bias:
                xq_pre.add_(weights["b_q"])
                xk_pre.add_(weights["b_k"])
            dq2d, _, _ = ops.flextrain_rmsnorm_bwd(dq2d, xq_pre, weights["w_q_norm"], getattr(slot, self.q_rstd_name),
                                                   head_dim=cfg.head_dim, dW=grads.get("g_q_norm"))
            dk2d, _, _ = ops.flextrain_rmsnorm_bwd(dk2d, xk_pre, weights["w_k_norm"], getattr(slot, self.k_rstd_name),
                                                   head_dim=cfg.head_dim, dW=grads.get("g_k_norm"))
        if cfg.qkv_bias:
            grads["g_b_q"].add_(dq2d.sum(dim=0))
            grads["g_b_k"].add_(dk2d.sum(dim=0))
            grads["g_b_v"].add_(dv2d.sum(dim=0))
        dx = torch.empty((T, cfg.d_model), dtype=dq2d.dtype, device=dq.device)
        self._mm_sum([dq2d, dk2d, dv2d], [weights["w_q"].T, weights["w_k"].T, weights["w_v"].T], dx)
        slot.aux["bwd_dq"] = dq2d
        slot.aux["bwd_local_dk"] = dk2d
        slot.aux["bwd_local_dv"] = dv2d
        return dx

    def bwd_accumulate_qkv_grads(self, attn_norm_output, grads, slot, *, skip_grads: frozenset = frozenset(),
                                 capture_xy: dict | None = None) -> None:
        """``g_v, g_k, g_q += attn_norm_output^T d{v,k,q}`` (attention.py:777-823)."""
        todo = []
        for name, dy_key in (("g_v", "bwd_local_dv"), ("g_k", "bwd_local_dk"), ("g_q", "bwd_dq")):
            dy = slot.aux[dy_key]
            if name in skip_grads:
                if capture_xy is not None:
                    capture_xy[name] = (attn_norm_output, dy)
            else:
                todo.append((name, dy))
        kv = [(n, dy) for n, dy in todo if n in ("g_v", "g_k")]
        if len(kv) == 2:     # the two small products as one launch
            g = [grads[n] for n, _ in kv]
            self._mm_shared(attn_norm_output.T, [dy for _, dy in kv], g, Cs=g, beta=1.0)
            todo = [t for t in todo if t[0] == "g_q"]
        for name, dy in todo:
            self._mm(attn_norm_output.T, dy, grads[name], C=grads[name], beta=1.0)
        del slot.aux["bwd_dq"]
        del slot.aux["bwd_local_dk"]
        del slot.aux["bwd_local_dv"]

    def bwd(self, dx_resid, seq_positions, weights, grads, slot, attn_norm_output, attention_bwd: Callable, *,
            skip_grads: frozenset = frozenset(), capture_xy: dict | None = None):
        """Whole backward; ``attention_bwd(d_out, q, k, v, out) -> (dq, dk, dv)`` is the core's."""
        d_out = self.bwd_o(dx_resid, weights, grads, slot, skip_grads=skip_grads, capture_xy=capture_xy)
        dq, dk, dv = attention_bwd(d_out, slot.xq, slot.xk, slot.xv, slot.attn_result)
        return self.bwd_qkv(dq, dk, dv, seq_positions, weights, grads, slot, attn_norm_output)

    # ------------------------------------------------------- FLOP accounting
    def projection_flops(self, tokens: int) -> int:
        """Forward FLOPs of the four projections (attention.py:825-862 without the core's term)."""
        cfg = self.cfg
        return 2 * tokens * cfg.d_model * (2 * cfg.attn_dim + 2 * cfg.kv_dim)
