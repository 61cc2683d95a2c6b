"""RMSNorm forward / backward: the kernels' own source run on the CPU by the host simulation
(tests/hostsim) on guard-paged buffers, against the oracle.  Covers every tile configuration of the
launch code (row widths from 8 to 16384 and the any-shape fallback) and ragged row counts."""
from __future__ import annotations

import pytest
import torch

from oracle import rmsnorm as o_norm
from tests.hostsim import sim

from tests.hostsim.build import needs_host_clang

pytestmark = needs_host_clang

BF = torch.bfloat16


def _run(rows, ncols, dt=BF, wdt=BF, accumulate=False, with_y=False):
    g = torch.Generator().manual_seed(rows * 131 + ncols)
    x = torch.randn(rows, ncols, generator=g).to(dt)
    dy = torch.randn(rows, ncols, generator=g).to(dt)
    w = (1 + 0.1 * torch.randn(ncols, generator=g)).to(wdt)
    L = sim.lib()
    gx, gw, gdy = sim.guard(x), sim.guard(w), sim.guard(dy)
    y, rstd = sim.guard(torch.empty_like(x)), sim.guard(torch.empty(rows, dtype=torch.float32))
    assert L.fx_rmsnorm_fwd(sim.p(gx), sim.p(gw), sim.p(y), sim.p(rstd), rows, ncols, 1e-5, sim.DT[dt], sim.DT[wdt], 0, None) == 0
    y_ref, rstd_ref = o_norm.rmsnorm_fwd(x, w, eps=1e-5)
    torch.testing.assert_close(y.float(), y_ref.float(), rtol=1e-2, atol=1e-2)
    torch.testing.assert_close(rstd, rstd_ref.reshape(-1), rtol=1e-5, atol=1e-6)
    y2 = sim.guard(torch.empty_like(x))
    assert L.fx_rmsnorm_fwd(sim.p(gx), sim.p(gw), sim.p(y2), sim.p(rstd), rows, ncols, 1e-5, sim.DT[dt], sim.DT[wdt], 1, None) == 0
    assert torch.equal(y2, y)                                   # recompute from the saved rstd: the same bits
    dx0 = torch.randn(rows, ncols, generator=g).to(dt) if accumulate else None
    dw0 = torch.randn(ncols, generator=g) if accumulate else None
    dx = sim.guard(dx0 if accumulate else torch.empty_like(x))
    dw = sim.guard(dw0 if accumulate else torch.empty(ncols))
    yb = sim.guard(torch.empty_like(x)) if with_y else None
    ws_bytes = int(L.fx_rmsnorm_bwd_ws_bytes(rows, ncols))
    ws = sim.guard(torch.empty(max(ws_bytes // 4, 1)))
    assert L.fx_rmsnorm_bwd(sim.p(gdy), sim.p(gx), sim.p(gw), sim.p(rstd), sim.p(dx), int(accumulate), sim.p(dw), 0, int(accumulate),
                            sim.p(yb), rows, ncols, sim.DT[dt], sim.DT[wdt], sim.p(ws), ws_bytes, None) == 0
    dx_ref, dw_ref, yr = o_norm.rmsnorm_bwd(dy, x, w, rstd_ref, dx_old=dx0, dw_old=dw0, recompute_output=with_y)
    torch.testing.assert_close(dx.float(), dx_ref.float(), rtol=1e-2, atol=2e-2 if accumulate else 1e-2)
    torch.testing.assert_close(dw, dw_ref, rtol=1e-3, atol=1e-2 * max(1.0, rows ** 0.5))
    if with_y:
        torch.testing.assert_close(yb.float(), yr.float(), rtol=1e-2, atol=1e-2)


@pytest.mark.parametrize("ncols", [8, 128, 136, 256, 512, 1000, 1024, 2048, 4096, 8192, 16384])
def test_vector_configurations(ncols):
    _run(5, ncols)


@pytest.mark.parametrize("rows", [1, 3, 64, 130])
def test_ragged_row_counts(rows):
    _run(rows, 1024, accumulate=True, with_y=True)
    _run(rows, 256, wdt=torch.float32)


def test_fallback_shapes_and_types():
    _run(7, 100)                     # not a multiple of 8: the any-shape kernels
    _run(4, 20000)                   # wider than the widest vector configuration
    _run(6, 512, dt=torch.float16, wdt=torch.float16)
    _run(6, 512, dt=torch.float32, wdt=torch.float32)
