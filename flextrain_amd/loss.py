"""Per-token loss objects for :class:`flextrain_amd.head.LMHead`, with the
interface of flextrain/nn/loss.py:53-316 (``TokenSlice``, ``TokenContext``,
``LossFn``, ``CrossEntropyLoss``)."""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Mapping, Protocol, runtime_checkable

import torch

from .ops.softmax_ce import (
    flextrain_cross_entropy_loss,
    flextrain_softmax,
    flextrain_softmax_cross_entropy,
)

IGNORE_INDEX = -100


@dataclass
class TokenSlice:
    """Per-token context of one micro-chunk (flextrain/nn/loss.py:53-99)."""
    offset: int
    size: int
    labels: torch.Tensor | None = None
    loss_mask: torch.Tensor | None = None
    advantages: torch.Tensor | None = None
    ref_logprobs: torch.Tensor | None = None
    extra: Mapping[str, torch.Tensor] = field(default_factory=dict)


@dataclass
class TokenContext:
    """Per-token context of a whole training chunk (flextrain/nn/loss.py:102-165)."""
    labels: torch.Tensor | None = None
    loss_mask: torch.Tensor | None = None
    advantages: torch.Tensor | None = None
    ref_logprobs: torch.Tensor | None = None
    extra: Mapping[str, torch.Tensor] = field(default_factory=dict)

    def slice_for(self, offset: int, size: int) -> TokenSlice:
        cut = lambda t: None if t is None else t[offset:offset + size]
        return TokenSlice(offset=offset, size=size, labels=cut(self.labels), loss_mask=cut(self.loss_mask),
                          advantages=cut(self.advantages), ref_logprobs=cut(self.ref_logprobs),
                          extra={k: v[offset:offset + size] for k, v in self.extra.items()})

    @property
    def total_tokens(self) -> int:
        for t in (self.labels, self.loss_mask, self.advantages, self.ref_logprobs):
            if t is not None:
                return int(t.shape[0])
        for v in self.extra.values():
            return int(v.shape[0])
        raise ValueError("TokenContext is empty; cannot infer total_tokens")


@runtime_checkable
class LossFn(Protocol):
    """``compute(logits, token_slice, *, loss_scale, per_token_loss_out) -> (dZ, aux)``;
    dZ is returned UNSCALED (the head folds ``loss_scale`` into its GEMM alpha).
    flextrain/nn/loss.py:168-205."""

    def compute(self, logits, token_slice, *, loss_scale, per_token_loss_out): ...


class CrossEntropyLoss:
    """Softmax + label cross-entropy (flextrain/nn/loss.py:208-316).

    ``fused=True`` (default): one kernel turns the logits into dZ in place and
    takes the loss from the fp32 log-sum-exp; ignore-index rows and ``loss_mask``
    are handled inside the kernel, so there is no host synchronisation.
    ``fused=False``: the reference's sequence — softmax into a separate probability
    buffer (rounded to the compute dtype), loss from ``-log p``, torch-side masking
    with its two ``.item()`` synchronisations."""

    def __init__(self, ignore_index: int = IGNORE_INDEX, fused: bool = True) -> None:
        self.ignore_index = ignore_index
        self.fused = fused

    @property
    def supports_logit_softcap(self) -> bool:
        """Whether ``compute`` takes ``logit_softcap=`` and applies the final-logit soft cap itself
        (the fused kernel does, inside its two sweeps; the head then skips its own capping passes)."""
        return self.fused

    def compute(self, logits, token_slice, *, loss_scale, per_token_loss_out, logit_softcap=None):
        if token_slice.labels is None:
            raise ValueError("CrossEntropyLoss requires token_slice.labels")
        labels = token_slice.labels
        n = token_slice.size
        next_pred = torch.empty(n, dtype=torch.int64, device=logits.device)
        next_prob = torch.empty(n, dtype=torch.float32, device=logits.device)
        if self.fused:
            dZ, _ = flextrain_softmax_cross_entropy(
                logits, labels, L=per_token_loss_out, loss_mask=token_slice.loss_mask, max_idx_out=next_pred,
                max_val_out=next_prob, ignore_index=self.ignore_index, logit_softcap=logit_softcap)
            return dZ, {"next_prediction": next_pred, "next_prediction_prob": next_prob}
        if logit_softcap is not None:
            raise ValueError("the unfused sequence does not cap logits; cap them before calling compute")
        ignore_rows = labels == self.ignore_index
        any_ignore = bool(ignore_rows.any().item())
        safe = torch.where(ignore_rows, torch.zeros_like(labels), labels) if any_ignore else labels
        probs = torch.empty_like(logits)
        flextrain_softmax(logits, out=probs, max_idx_out=next_pred, max_val_out=next_prob)
        dZ, _ = flextrain_cross_entropy_loss(probs, safe, L=per_token_loss_out)
        include = ~ignore_rows if any_ignore else None
        if token_slice.loss_mask is not None:
            lm = token_slice.loss_mask.to(dtype=torch.bool)
            include = lm if include is None else (include & lm)
        if include is not None and not bool(include.all().item()):
            dZ.mul_(include.to(dtype=logits.dtype).unsqueeze(-1))
            per_token_loss_out.masked_fill_(~include, 0.0)
        return dZ, {"next_prediction": next_pred, "next_prediction_prob": next_prob}
