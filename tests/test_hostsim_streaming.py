"""The streamed AdamW chunk and the batched activation-field copies in the host simulation: host buffers,
staging workspace and copy-out buffers are guard-paged and exactly sized, so the sub-chunk arithmetic (slot
rotation, the last partial sub-chunk, field pitches) cannot step outside them unnoticed; results against the
oracle and against plain copies."""
from __future__ import annotations

import ctypes

import pytest
import torch

from oracle import adamw as o_adam
from tests.hostsim import sim

from tests.hostsim.build import needs_host_clang

pytestmark = needs_host_clang

BF, F32 = torch.bfloat16, torch.float32
G, P = sim.guard, sim.p


@pytest.mark.parametrize("n,sub,slots,ring", [(10_000, 4096, 3, True), (4096 * 3, 4096, 2, False), (777, 4096, 3, True),
                                              (50_000, 8192, 1, True), (33, 8, 16, False)])
@pytest.mark.parametrize("staged_copy", [True, False])
def test_streamed_adamw_chunk(n, sub, slots, ring, staged_copy):
    g = torch.Generator().manual_seed(n)
    p = (torch.randn(n, generator=g) * 0.02)
    gr = (torch.randn(n, generator=g) * 1e-3).to(BF)
    m, v = torch.randn(n, generator=g) * 1e-4, torch.rand(n, generator=g) * 1e-6
    hp = dict(lr=3e-3, beta1=0.9, beta2=0.95, eps=1e-8, weight_decay=0.1)
    L = sim.lib()
    ws_bytes = int(L.fx_adamw_stream_ws_bytes(sub, slots, 0, 2, 0, int(staged_copy)))
    ws = G(torch.empty(ws_bytes, dtype=torch.uint8), align=256)
    hp_, hg, hm, hv, hc = G(p), G(gr), G(m), G(v), G(torch.empty(n, dtype=BF))
    handle = ctypes.c_void_p()
    if ring:
        assert L.fx_stream_ring_create(slots, ctypes.byref(handle)) == 0
    S = 0x10                                                     # stands for three distinct stream handles
    for step in (1, 2):                                          # the second call reuses the ring's slot state
        assert L.fx_adamw_stream_chunk(P(hp_), P(hg), P(hm), P(hv), P(hc), 0 if staged_copy else 1, n, 0, 2, 0, hp["lr"], hp["beta1"],
                                       hp["beta2"], hp["eps"], hp["weight_decay"], 1 - hp["beta1"] ** step, 1 - hp["beta2"] ** step,
                                       P(ws), ws_bytes, sub, slots, S, S + 1, S + 2, handle if ring else None) == 0
        # as a caller does before it reads the results (and before the next call reads them as its inputs): the
        # host waits for the copies out, and for the kernels where they write the bf16 copy themselves
        L.hostsim_order_stream_sync(ctypes.c_uint64(S + 2))
        L.hostsim_order_stream_sync(ctypes.c_uint64(S + 1))
        p, m, v, c = o_adam.adamw_step(p, gr, m, v, step=step, **hp)
        torch.testing.assert_close(hp_, p, rtol=1e-5, atol=1e-7)
        torch.testing.assert_close(hm, m, rtol=1e-5, atol=1e-9)
        torch.testing.assert_close(hv, v, rtol=1e-5, atol=1e-11)
        torch.testing.assert_close(hc.float(), c.float(), rtol=1e-2, atol=1e-4)
    if ring:
        assert L.fx_stream_ring_destroy(handle) == 0


def test_batched_field_copies():
    g = torch.Generator().manual_seed(4)
    L = sim.lib()
    # three fields: contiguous, a narrowed view of wider rows (pitch > row), a single row
    srcs = [torch.randint(0, 255, (40, 64), generator=g, dtype=torch.uint8), torch.randint(0, 255, (16, 96), generator=g, dtype=torch.uint8),
            torch.randint(0, 255, (1, 24), generator=g, dtype=torch.uint8)]
    rows, row_bytes = [40, 16, 1], [64, 48, 24]
    src_pitch, dst_pitch = [64, 96, 24], [64, 80, 24]
    gs = [G(t) for t in srcs]
    gd = [G(torch.zeros(r, dp, dtype=torch.uint8)) for r, dp in zip(rows, dst_pitch)]
    arr = lambda vals: (ctypes.c_void_p * len(vals))(*vals)
    i64 = lambda vals: (ctypes.c_int64 * len(vals))(*vals)
    for direction in (0, 1, 2):
        for d in gd:
            d.zero_()
        assert L.fx_copy_fields(3, arr([P(d) for d in gd]), arr([P(s) for s in gs]), i64(rows), i64(row_bytes), i64(dst_pitch), i64(src_pitch),
                                direction, None) == 0
        for d, s, rb in zip(gd, srcs, row_bytes):
            assert torch.equal(d[:, :rb], s[:, :rb]) and bool((d[:, rb:] == 0).all())
    assert L.fx_copy_fields(3, arr([P(d) for d in gd]), arr([P(s) for s in gs]), i64(rows), i64(row_bytes), i64([64, 40, 24]), i64(src_pitch),
                            0, None) == -1                       # a pitch smaller than its row
