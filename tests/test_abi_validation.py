"""Argument checks of the C ABI, on the CPU: every call below is refused by the entry point's own
host-side validation (return -1, one line on stderr) BEFORE anything is enqueued, so the pointers are
never dereferenced and no GPU is needed.  Each case breaks exactly one rule; the valid twin of every
call is what the GPU parity tests launch."""
from __future__ import annotations

import pytest

from flextrain_amd._lib import lib

BF16, F16, F32 = 2, 1, 0
P = 0x7F0000001000          # a 16-byte-aligned, never-dereferenced address
ODD = P + 2                 # misaligned for 16-byte accesses
STREAM = None


def _ws(E, rows):
    return int(lib().fx_grouped_ws_bytes(E, rows))


# ------------------------------------------------------------------ softmax-CE and the soft cap
def _smce(**kw):
    a = dict(logits=P, dz=P, labels=P, lab64=1, mask=None, loss=P, idx=None, val=None, rows=4, V=64, si=64, so=64,
             ignore=-100, max_loss=100.0, cap=0.0, dt=BF16)
    a.update(kw)
    return lib().fx_softmax_ce(a["logits"], a["dz"], a["labels"], a["lab64"], a["mask"], a["loss"], a["idx"], a["val"],
                               a["rows"], a["V"], a["si"], a["so"], a["ignore"], a["max_loss"], a["cap"], a["dt"], STREAM)


@pytest.mark.parametrize("kw", [dict(rows=-1), dict(V=0), dict(cap=-1.0), dict(cap=float("nan")), dict(logits=None),
                                dict(loss=None), dict(si=32), dict(so=8), dict(dt=7)])
def test_softmax_ce_refuses(kw):
    assert _smce(**kw) == -1


def test_softmax_ce_with_no_rows_is_a_no_op():
    assert _smce(rows=0, logits=None, dz=None, labels=None, loss=None) == 0


@pytest.mark.parametrize("kw", [dict(cap=0.0), dict(cap=-2.0), dict(V=0), dict(rows=-3), dict(stride=16), dict(gstride=8),
                                dict(logits=None), dict(gate=None), dict(dt=9)])
def test_softcap_passes_refuse(kw):
    a = dict(logits=P, gate=P, rows=4, V=64, stride=64, gstride=64, cap=30.0, dt=BF16)
    a.update(kw)
    assert lib().fx_softcap_fwd(a["logits"], a["gate"], a["rows"], a["V"], a["stride"], a["gstride"], a["cap"], a["dt"],
                                STREAM) == -1
    if "cap" not in kw:
        assert lib().fx_softcap_bwd(a["logits"], a["gate"], a["rows"], a["V"], a["stride"], a["gstride"], a["dt"],
                                    STREAM) == -1


# ------------------------------------------------------------------ grouped weight gradient with a gathered operand
def _wgrad(**kw):
    E, rows = 8, 4096
    a = dict(A=P, lda=1536, B=P, ldb=2048, G=P, ldg=2048, gstride=1536 * 2048, g_dt=BF16, counts=P, E=E, rows=rows,
             M=1536, N=2048, alpha=1.0, beta=1.0, dt=BF16, ws=P, ws_bytes=_ws(E, rows), amap=None, arows=0, bmap=None,
             brows=0)
    a.update(kw)
    return lib().fx_grouped_gemm_wgrad(a["A"], a["lda"], a["B"], a["ldb"], a["G"], a["ldg"], a["gstride"], a["g_dt"],
                                       a["counts"], a["E"], a["rows"], a["M"], a["N"], a["alpha"], a["beta"], a["dt"],
                                       a["ws"], a["ws_bytes"], a["amap"], a["arows"], a["bmap"], a["brows"], STREAM)


@pytest.mark.parametrize("kw", [
    dict(E=0), dict(rows=-1), dict(M=0), dict(A=None), dict(G=None), dict(ws=None), dict(ws_bytes=16), dict(dt=F32),
    dict(g_dt=F16), dict(A=ODD), dict(lda=1540), dict(N=2044), dict(lda=1 << 23),
    dict(amap=P, arows=512, bmap=P, brows=512),          # both operands gathered
    dict(amap=P, arows=0), dict(bmap=P, brows=-5),       # a map without its source's row count
    dict(bmap=P, brows=1 << 21),                         # 2 Mi rows x 2048 x 2 B = 8 GB: beyond the 32-bit lane offsets
])
def test_grouped_wgrad_refuses(kw):
    assert _wgrad(**kw) == -1


# ------------------------------------------------------------------ dgrad with the SwiGLU backward in its epilogue
def _swb(**kw):
    E, rows, F, K = 8, 4096, 768, 2048
    a = dict(dy=P, lddy=K, w=P, ldb=F, wstride=K * F, trans_b=0, x_up=P, ldx=2 * F, srw=P, srw_dt=BF16, dx_up=P,
             lddx=2 * F, act=None, ldact=F, dprob=P, dprob_dt=BF16, counts=P, E=E, rows=rows, F=F, K=K, dt=BF16, ws=P,
             ws_bytes=_ws(E, rows), part=P, part_bytes=int(lib().fx_grouped_swiglu_bwd_ws_bytes(rows, F)), dymap=None,
             dyrows=0)
    a.update(kw)
    return lib().fx_grouped_gemm_rows_swiglu_bwd(
        a["dy"], a["lddy"], a["w"], a["ldb"], a["wstride"], a["trans_b"], a["x_up"], a["ldx"], a["srw"], a["srw_dt"],
        a["dx_up"], a["lddx"], a["act"], a["ldact"], a["dprob"], a["dprob_dt"], a["counts"], a["E"], a["rows"], a["F"],
        a["K"], a["dt"], a["ws"], a["ws_bytes"], a["part"], a["part_bytes"], a["dymap"], a["dyrows"], STREAM)


@pytest.mark.parametrize("kw", [
    dict(E=0), dict(F=0), dict(K=-8), dict(dy=None), dict(srw=None), dict(dprob=None), dict(ws_bytes=64),
    dict(part=None), dict(part_bytes=1024), dict(part=ODD), dict(dt=F32), dict(srw_dt=F16), dict(dprob_dt=F16),
    dict(rows=1024),                                     # 128 rows per expert: 128-row tiles, the fused form needs 256
    dict(x_up=ODD), dict(ldx=2 * 768 + 4), dict(K=2044), dict(F=764), dict(ldx=768), dict(lddx=1000),
    dict(act=P, ldact=760), dict(lddy=1 << 23),
    dict(dymap=P, dyrows=0), dict(dymap=P, dyrows=1 << 21),
])
def test_fused_dgrad_swiglu_bwd_refuses(kw):
    assert _swb(**kw) == -1


def test_tile_height_and_workspace_sizes():
    L = lib()
    assert L.fx_grouped_rows_tile_height(8, 4096) == 256      # 512 rows per expert
    assert L.fx_grouped_rows_tile_height(256, 16384) == 128   # 64 rows per expert
    assert L.fx_grouped_rows_tile_height(128, 65536) == 256
    # one fp32 slot per row, column tile and wave column (4 per 256-column tile)
    assert L.fx_grouped_swiglu_bwd_ws_bytes(65536, 768) == 65536 * 3 * 4 * 4
    assert L.fx_grouped_swiglu_bwd_ws_bytes(100, 192) == 100 * 1 * 4 * 4
    # plan header (4 words) + E + 1 offsets... : never shrinks with more rows or experts
    assert L.fx_grouped_ws_bytes(8, 4096) <= L.fx_grouped_ws_bytes(8, 8192) <= L.fx_grouped_ws_bytes(16, 8192)


# ------------------------------------------------------------------ sort, optimizer, norm: structural requirements
def test_expert_sort_refuses_a_short_workspace_and_oversized_inputs():
    L = lib()
    need = int(L.fx_moe_sort_ws_bytes(65536, 128))
    assert need == (128 * 256 + 2 * 128) * 4
    assert L.fx_moe_sort(P, 0, 65536, 128, P, 0, P, None, P, need - 4, STREAM) == -1
    assert L.fx_moe_sort(P, 0, 65536, 128, P, 0, P, None, None, need, STREAM) == -1
    assert L.fx_moe_sort(P, 0, -1, 128, P, 0, P, None, P, need, STREAM) == -1
    assert L.fx_moe_sort(P, 0, 65536, 1 << 15, P, 0, P, None, P, 1 << 40, STREAM) == -1     # histogram beyond the LDS
    # the allocation-free variant names its limit instead of overrunning its fixed array
    words = int(L.fx_moe_sort_noalloc_max_words())
    pairs = (words // 512 + 8) * 256
    assert 512 * (pairs // 256) + 2 * 512 > words
    assert L.fx_moe_sort_noalloc(P, 0, pairs, 512, P, 0, P, None, STREAM) == -1
    assert L.fx_moe_sort_noalloc(P, 0, -1, 512, P, 0, P, None, STREAM) == -1


def test_row_sources_refuses():
    L = lib()
    assert L.fx_moe_row_sources(P, 0, -1, 8, P, STREAM) == -1
    assert L.fx_moe_row_sources(P, 0, 16, 0, P, STREAM) == -1
    assert L.fx_moe_row_sources(None, 0, 16, 8, P, STREAM) == -1
    assert L.fx_moe_row_sources(P, 0, 0, 8, None, STREAM) == 0


def test_adamw_refuses():
    L = lib()
    hp = (3e-5, 0.9, 0.95, 1e-8, 0.1, 0.1, 0.05)
    assert L.fx_adamw_step(P, P, P, P, None, -1, F32, BF16, F32, *hp, STREAM) == -1
    assert L.fx_adamw_step(P, None, P, P, None, 1024, F32, BF16, F32, *hp, STREAM) == -1
    assert L.fx_adamw_step(P, P, ODD, P, None, 1024, F32, BF16, F32, *hp, STREAM) == -1
    assert L.fx_adamw_step(P, P, P, P, ODD, 1024, F32, BF16, F32, *hp, STREAM) == -1
    assert L.fx_adamw_step(None, None, None, None, None, 0, F32, BF16, F32, *hp, STREAM) == 0
    # streamed chunk: sub-chunks are multiples of 8 elements, 1..16 slots, three explicit streams, workspace sized
    S = 0x1000                                                               # stands for a stream handle; never used
    need = int(L.fx_adamw_stream_ws_bytes(4096, 3, F32, BF16, F32, 1))
    ok = dict(sub=4096, slots=3, ws=P, ws_bytes=need, s_in=S, s_c=S, s_out=S, p=P)
    for kw in (dict(sub=4100), dict(sub=0), dict(slots=0), dict(slots=17), dict(ws=None), dict(ws_bytes=need - 1),
               dict(s_in=None), dict(s_out=None), dict(p=ODD), dict(p=None)):
        a = dict(ok, **kw)
        assert L.fx_adamw_stream_chunk(a["p"], P, P, P, P, 0, 1 << 20, F32, BF16, F32, *hp, a["ws"], a["ws_bytes"],
                                       a["sub"], a["slots"], a["s_in"], a["s_c"], a["s_out"], None) == -1, kw


def test_rmsnorm_refuses():
    L = lib()
    need = int(L.fx_rmsnorm_bwd_ws_bytes(2048, 4096))
    assert need == 256 * 4096 * 4                                  # one fp32 partial row per workgroup, 256 at most
    args = lambda **kw: dict(dict(dy=P, x=P, w=P, rstd=P, dx=P, dw=P, rows=2048, ncols=4096, ws=P, ws_bytes=need), **kw)
    for kw in (dict(rows=-1), dict(ncols=0), dict(dy=None), dict(rstd=None), dict(dx=None), dict(ws=None),
               dict(ws_bytes=need - 4)):
        a = args(**kw)
        assert L.fx_rmsnorm_bwd(a["dy"], a["x"], a["w"], a["rstd"], a["dx"], 0, a["dw"], F32, 1, None, a["rows"],
                                a["ncols"], BF16, BF16, a["ws"], a["ws_bytes"], STREAM) == -1, kw
    assert L.fx_rmsnorm_fwd(P, P, P, None, 16, 4096, 1e-5, BF16, BF16, 0, STREAM) == -1
    assert L.fx_rmsnorm_fwd(P, P, P, P, 16, -4, 1e-5, BF16, BF16, 0, STREAM) == -1
    assert L.fx_rmsnorm_fwd(None, None, None, None, 0, 4096, 1e-5, BF16, BF16, 0, STREAM) == 0
