"""The LM head's fused forward + loss + backward over token micro-chunks, with the
interface of flextrain/nn/head.py:60-393 (``LMHeadConfig``, ``LMHead.forward_backward``)
and ``LossStats`` (flextrain/core/layer.py:1060-1088).

Per group of micro-chunks: RMSNorm fwd -> logits GEMM -> loss fn (dZ in place) -> head
weight-gradient GEMM (``beta = 1``, ``alpha = loss_scale``) -> dX GEMM -> RMSNorm
bwd -> dx written over x.  The GEMMs go through the MFMA dispatcher; the
weight may be stored ``(d_model, vocab)`` (reference) or be the transposed view
of a ``(vocab, d_model)`` tensor (Hugging Face layout) without a copy.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Mapping, MutableMapping

import torch

from .loss import CrossEntropyLoss, LossFn, TokenContext
from .matmul_dispatcher import CublasLtDispatcher
from .ops.rmsnorm import flextrain_rmsnorm_bwd, flextrain_rmsnorm_fwd
from .ops.softmax_ce import flextrain_logit_softcap_bwd, flextrain_logit_softcap_fwd


@dataclass(frozen=True)
class LMHeadConfig:
    """flextrain/nn/head.py:60-95 (the dtype-role fields feed the parameter
    planner, which is outside this package, and are kept for signature parity)."""
    d_model: int
    vocab_size: int
    rms_norm_eps: float = 1e-5
    head_chunk_size: int = 1024
    # Micro-chunks handled by one GEMM group.  1 (default) is the reference's schedule: one logits
    # buffer of head_chunk_size rows (263 MB at a 128256-entry vocabulary).  Larger groups are an
    # opt-in trade of memory for time (not in the reference): fewer read-modify-write passes over the
    # head weight gradient and better-filled GEMMs; the result differs only in accumulation order.
    # Measured at 8192 tokens x 128256: 2 chunks (525 MB) are no faster than 1, because the buffer no
    # longer fits the 256 MB last-level cache between the GEMMs and the loss kernel; 8 chunks (2.1 GB)
    # are a fifth faster.  None: as many chunks as keep the buffer under ``logits_buffer_bytes``.
    fuse_chunks: int | None = 1
    logits_buffer_bytes: int = 4 << 30
    final_logit_softcap: float | None = None
    compute_dtype: torch.dtype = torch.bfloat16
    master_dtype: torch.dtype | None = None
    grad_dtype: torch.dtype | None = None
    norm_grad_dtype: torch.dtype = torch.float32
    norm_master_dtype: torch.dtype = torch.float32
    norm_compute_dtype: torch.dtype = torch.float32


@dataclass
class LossStats:
    """flextrain/core/layer.py:1060-1088."""
    per_token_loss: torch.Tensor
    next_prediction: torch.Tensor
    next_prediction_prob: torch.Tensor
    token_count: int


class LMHead:
    layer_id: int = -2

    def __init__(self, cfg: LMHeadConfig) -> None:
        self.cfg = cfg
        self._disp = None

    def _dispatcher(self) -> CublasLtDispatcher:
        if self._disp is None:
            self._disp = CublasLtDispatcher(round_multiple=32)
        return self._disp

    def forward_backward(self, x, token_ctx: TokenContext, chunk, weights: Mapping[str, torch.Tensor],
                         grads: MutableMapping[str, torch.Tensor], ctx, *, loss_scale: float = 1.0,
                         loss_fn: LossFn | None = None):
        """Returns ``(dx, stats)`` with ``dx is x`` (x is overwritten micro-chunk by
        micro-chunk).  Gradients accumulate in place into ``grads["g_head_proj"]``
        and ``grads["g_final_norm"]``; a missing/None entry skips that gradient.
        flextrain/nn/head.py:155-393."""
        if loss_fn is None:
            loss_fn = CrossEntropyLoss()
        num_tokens, d_model = x.shape
        cfg = self.cfg
        assert d_model == cfg.d_model, f"x has d_model={d_model}, head expects {cfg.d_model}"
        if token_ctx.total_tokens != num_tokens:
            raise ValueError(f"token_ctx covers {token_ctx.total_tokens} tokens, x has {num_tokens}")
        device, dtype = x.device, x.dtype
        per_token_loss = torch.empty(num_tokens, dtype=torch.float32, device=device)
        next_prediction = torch.empty(num_tokens, dtype=torch.int64, device=device)
        next_prediction_prob = torch.empty(num_tokens, dtype=torch.float32, device=device)
        any_next_prediction = False
        w_final_norm = weights["w_final_norm"]
        w_head_proj = weights["w_head_proj"]                  # logical (d_model, vocab)
        g_final_norm = grads.get("g_final_norm")
        g_head_proj = grads.get("g_head_proj")
        V = w_head_proj.shape[1]
        disp = self._dispatcher()
        stream = torch.cuda.current_stream(device).cuda_stream
        aux_chunks = []
        fuse = cfg.fuse_chunks
        if fuse is None:
            per_chunk = cfg.head_chunk_size * V * x.element_size()
            fuse = max(1, cfg.logits_buffer_bytes // max(1, per_chunk))
        group_rows = cfg.head_chunk_size * max(1, int(fuse))
        chunk_rows = min(group_rows, num_tokens)
        logits_buf = torch.empty((chunk_rows, V), dtype=dtype, device=device)
        dx_head_buf = torch.empty((chunk_rows, d_model), dtype=dtype, device=device)

        offset = 0
        while offset < num_tokens:
            t_prime = min(group_rows, num_tokens - offset)
            x_slice = x[offset:offset + t_prime]
            head_in, rstd = flextrain_rmsnorm_fwd(x_slice, W=w_final_norm, rms_norm_eps=cfg.rms_norm_eps)
            logits = logits_buf[:t_prime]
            disp.matmul(stream, A=head_in, B=w_head_proj, D=logits)

            # Gemma's final-logit soft cap (flextrain/nn/head.py:273-298): a loss object that caps inside
            # its own kernel gets the cap as an argument; for any other one the logits are capped in
            # place first and dZ is multiplied by the saved gate afterwards, as the reference does.
            cap = cfg.final_logit_softcap
            capped = cap is not None and cap > 0.0
            token_slice = token_ctx.slice_for(offset, t_prime)
            loss_out = per_token_loss[offset:offset + t_prime]
            if capped and getattr(loss_fn, "supports_logit_softcap", False):
                dZ, aux = loss_fn.compute(logits, token_slice, loss_scale=loss_scale, per_token_loss_out=loss_out,
                                          logit_softcap=float(cap))
            else:
                gate = flextrain_logit_softcap_fwd(logits, float(cap)) if capped else None
                dZ, aux = loss_fn.compute(logits, token_slice, loss_scale=loss_scale, per_token_loss_out=loss_out)
                if gate is not None:
                    flextrain_logit_softcap_bwd(dZ, gate)
                    del gate
            if "next_prediction" in aux:
                next_prediction[offset:offset + t_prime].copy_(aux.pop("next_prediction"))
                next_prediction_prob[offset:offset + t_prime].copy_(aux.pop("next_prediction_prob"))
                any_next_prediction = True
            if aux:
                aux_chunks.append(aux)

            if g_head_proj is not None:
                if g_head_proj.stride(1) == 1:      # (d, V) row-major: g += scale * h.T @ dZ
                    disp.matmul(stream, A=head_in.T, B=dZ, C=g_head_proj, D=g_head_proj, alpha=loss_scale, beta=1.0)
                else:                               # view of a (V, d) tensor: g.T += scale * dZ.T @ h
                    g_t = g_head_proj.T
                    disp.matmul(stream, A=dZ.T, B=head_in, C=g_t, D=g_t, alpha=loss_scale, beta=1.0)
            dx_head = dx_head_buf[:t_prime]
            disp.matmul(stream, A=dZ, B=w_head_proj.T, D=dx_head, alpha=loss_scale, beta=0.0)
            dx_slice, _, _ = flextrain_rmsnorm_bwd(dx_head, x_slice, w_final_norm, rstd, dW=g_final_norm)
            x_slice.copy_(dx_slice)
            offset += t_prime

        stats = LossStats(
            per_token_loss=per_token_loss,
            next_prediction=next_prediction if any_next_prediction else per_token_loss.new_empty(0, dtype=torch.int64),
            next_prediction_prob=next_prediction_prob if any_next_prediction else per_token_loss.new_empty(0),
            token_count=num_tokens,
        )
        if aux_chunks:
            stats.aux_chunks = aux_chunks
        return x, stats
