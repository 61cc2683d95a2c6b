"""Host-side decisions of the grouped (per-expert) launches, on the CPU: which operand sets the fused and
gathering launches take (the block falls back to the one-to-one launches otherwise), and that the
wrappers refuse what the predicates refuse before anything reaches the library.  Only tensor metadata
is inspected, so CPU tensors serve."""
from __future__ import annotations

import pytest
import torch

from flextrain_amd import full_moe
from flextrain_amd.head import LMHeadConfig
from flextrain_amd.loss import CrossEntropyLoss
from flextrain_amd.ops import grouped

BF, F16, F32 = torch.bfloat16, torch.float16, torch.float32


def _set(T=1024, K=8, E=8, d=256, F=128, dt=BF, srw_dt=None, dprob_dt=None):
    TK = T * K
    return dict(dy=torch.empty(T, d, dtype=dt), x=torch.empty(T, d, dtype=dt), w_down=torch.empty(E, d, F, dtype=dt),
                x_up=torch.empty(TK, 2 * F, dtype=dt), srw=torch.empty(TK, 1, dtype=srw_dt or dt),
                dx_up=torch.empty(TK, 2 * F, dtype=dt), dprob=torch.empty(TK, 1, dtype=dprob_dt or dt),
                dy_sorted=torch.empty(TK, d, dtype=dt), act=torch.empty(TK, F, dtype=dt))


def _fused(s, **kw):
    a = dict(dy=s["dy_sorted"], w_down=s["w_down"], x_up=s["x_up"], srw=s["srw"], dx_up=s["dx_up"], fwd_act=s["act"],
             dprob=s["dprob"])
    a.update(kw)
    return grouped.grouped_swiglu_bwd_supported(a["dy"], a["w_down"], a["x_up"], a["srw"], a["dx_up"], a["fwd_act"],
                                                a["dprob"], dy_is_unsorted=a.get("unsorted", False))


def test_fused_dgrad_takes_the_block_shapes():
    s = _set()
    assert _fused(s)
    assert _fused(s, fwd_act=None)
    assert _fused(_set(dt=F16))
    assert _fused(_set(srw_dt=F32, dprob_dt=F32))
    assert _fused(s, dy=s["dy"], unsorted=True)              # the (T, d) upstream gradient, gathered


def test_fused_dgrad_refuses_what_the_kernel_cannot_take():
    s = _set()
    assert not _fused(_set(E=64))                            # 128 rows per expert: 128-row tiles
    assert not _fused(_set(dt=F32))
    assert not _fused(s, srw=s["srw"].to(F16))               # neither the activations' dtype nor fp32
    assert not _fused(s, dprob=s["dprob"][:-1])              # one entry per routed row
    assert not _fused(s, x_up=s["x_up"][:, :-8])             # rows hold 2 F elements
    assert not _fused(s, dx_up=s["dx_up"].t().contiguous().t())     # unit stride along the row
    assert not _fused(s, x_up=torch.empty(s["x_up"].shape[0], 2 * 128 + 4, dtype=BF)[:, :256])    # row stride not a multiple of 8
    assert not _fused(s, x_up=torch.empty(s["x_up"].numel() + 8, dtype=BF)[4:-4].view_as(s["x_up"]))   # 8-byte aligned only
    assert not _fused(s, w_down=s["w_down"].transpose(1, 2))  # the (E, d, F) layout, contiguous
    assert not _fused(s, dy=s["dy_sorted"][:-1])             # a sorted dy has one row per routed pair
    assert not _fused(_set(F=124))
    assert not _fused(_set(d=252))
    assert not _fused(s, fwd_act=s["act"][:, :-8])


def test_gathered_operands():
    ok = grouped.gathered_operand_supported
    x = torch.empty(1024, 256, dtype=BF)
    assert ok(x) and ok(x[:512]) and ok(torch.empty(1024, 512, dtype=F16)[:, :256])
    assert not ok(x.float())
    assert not ok(x.t())
    assert not ok(x[:, 4:])                                  # 8-byte aligned rows
    assert not ok(torch.empty(1024, 260, dtype=BF)[:, :256]) # row stride 260
    assert not ok(torch.empty(1 << 22, 1024, dtype=BF, device="meta")[:, :8])   # 8 GB span: beyond 32-bit lane offsets
    assert ok(torch.empty(1 << 20, 1024, dtype=BF, device="meta")[:, :8])
    assert not ok(x.view(2, 512, 256))


def test_block_takes_the_gathered_backward_only_with_every_operand_fit():
    s = _set()
    args = lambda **kw: [dict(s, **kw)[k] for k in ("dy", "x", "w_down", "x_up", "srw", "dx_up", "dprob")]
    assert full_moe.gathered_backward_supported(*args())
    assert not full_moe.gathered_backward_supported(*args(x=s["x"][:-1]))         # dy and x are the same tokens
    assert not full_moe.gathered_backward_supported(*args(x=s["x"].float()))
    assert not full_moe.gathered_backward_supported(*args(x_up=torch.empty(s["x_up"].shape[0] + 256, 256, dtype=BF)))
    small = _set(E=64)
    assert not full_moe.gathered_backward_supported(*[small[k] for k in ("dy", "x", "w_down", "x_up", "srw", "dx_up", "dprob")])


def test_wrappers_refuse_before_the_library_is_called():
    s = _set()
    counts = torch.zeros(8, dtype=torch.int32)
    with pytest.raises(ValueError, match="unsupported operands"):
        grouped.flextrain_grouped_gemm_rows_swiglu_bwd(s["dy_sorted"].float(), s["w_down"], counts, s["x_up"], s["srw"],
                                                       s["dx_up"], s["dprob"])
    G = torch.zeros(8, 256, 256, dtype=BF)
    rs = torch.zeros(s["x_up"].shape[0], dtype=torch.int32)
    with pytest.raises(ValueError, match="at most one operand"):
        grouped.flextrain_grouped_gemm_wgrad(s["x"], s["x"], G, counts, a_row_sources=rs, b_row_sources=rs)
    with pytest.raises(ValueError):
        # a CPU map: row sources live on the GPU with one int32 per routed row
        grouped.flextrain_grouped_gemm_wgrad(s["dx_up"], s["x"], torch.zeros(8, 256, 256, dtype=BF), counts, b_row_sources=rs)


def test_head_and_loss_defaults():
    cfg = LMHeadConfig(d_model=64, vocab_size=128, head_chunk_size=16)
    assert cfg.fuse_chunks == 1                              # the reference's schedule: one chunk per GEMM group
    assert cfg.logits_buffer_bytes == 4 << 30
    assert CrossEntropyLoss().supports_logit_softcap and not CrossEntropyLoss(fused=False).supports_logit_softcap
