"""The MFMA GEMM kernels behind the dispatcher ABI, run on the CPU by the host simulation (tests/hostsim):
the kernels' own source with the matrix instruction, the transposing LDS read and the LDS-DMA load
replaced by functions of the same documented meaning, on guard-paged operands, outputs and workspace,
against fp32 matrix products.  Shapes cover the four operand layouts, ragged tile edges, K tails and
K below one step, leading dimensions wider than the rows, every tile form the dispatcher picks
(128 x 128, 256 x 256, K splits with the reduction pass) and the accumulate-in-place epilogue."""
from __future__ import annotations

import pytest
import torch

from tests.hostsim import sim

from tests.hostsim.build import needs_host_clang

pytestmark = needs_host_clang

BF, F16, F32 = torch.bfloat16, torch.float16, torch.float32
G, P = sim.guard, sim.p


@pytest.fixture(autouse=True, params=["loads land late", "loads land early"])
def dma_timing(request):
    """Every test runs at both extremes of what the hardware may do with a load into LDS: landing only when
    the issuing lane's counted wait says it must have (a read that the wait does not cover sees stale data),
    and landing at its issue (a load into a buffer that other lanes still read shows as wrong results)."""
    sim.lib().hostsim_set_dma_eager(int(request.param == "loads land early"))
    yield
    sim.lib().hostsim_set_dma_eager(0)


@pytest.fixture(scope="module")
def ctx():
    L = sim.lib()
    c = L.create_dispatcher(8, 4)
    yield c
    L.destroy_dispatcher(c)


def _matmul(ctx, M, N, K, ta, tb, dt=BF, ddt=None, beta=0.0, alpha=1.0, pad=0, ws_floats=1 << 20, seed=0):
    ddt = ddt or dt
    g = torch.Generator().manual_seed(M * 7 + N * 3 + K + seed)
    def operand(rows, cols):
        full = torch.randn(rows, cols + pad, generator=g).to(dt)
        return full, full[:, :cols]
    Af, A = operand(K, M) if ta else operand(M, K)
    Bf, B = operand(N, K) if tb else operand(K, N)
    C = torch.randn(M, N, generator=g).to(ddt)
    gA, gB = G(Af), G(Bf)
    D = G(C) if beta else G(torch.full((M, N), 7.0, dtype=ddt))
    ws = G(torch.empty(ws_floats, dtype=F32)) if ws_floats else None
    rc = sim.lib().dispatch_matmul(ctx, 0, M, N, K, P(gA), Af.stride(0), P(gB), Bf.stride(0), P(D) if beta else 0, N, P(D), N,
                                   P(ws) if ws is not None else 0, ws_floats * 4, sim.DT[dt], sim.DT[dt], sim.DT[ddt], sim.DT[ddt], 0,
                                   alpha, beta, int(ta), int(tb))
    assert rc == 0
    ref = alpha * ((A.t() if ta else A).float() @ (B.t() if tb else B).float()) + beta * C.float()
    scale = float(ref.abs().max()) + 1e-6
    tol = 1e-5 if ddt == F32 else 1e-2
    torch.testing.assert_close(D.float(), ref.to(ddt).float(), rtol=tol, atol=tol * scale)


@pytest.mark.parametrize("ta,tb", [(0, 1), (0, 0), (1, 0), (1, 1)])
@pytest.mark.parametrize("M,N,K", [(64, 64, 64), (8, 8, 8), (130, 72, 200), (300, 520, 136), (257, 255 + 1, 24), (40, 600, 64)])
def test_layouts_and_ragged_edges(ctx, ta, tb, M, N, K):
    _matmul(ctx, M, N, K, ta, tb)


@pytest.mark.parametrize("ta,tb", [(0, 1), (1, 0)])
def test_leading_dimensions_wider_than_the_rows(ctx, ta, tb):
    _matmul(ctx, 136, 264, 192, ta, tb, pad=24)


def test_accumulate_in_place_and_output_types(ctx):
    _matmul(ctx, 264, 136, 128, 1, 0, ddt=F32, beta=1.0, alpha=0.5)        # a weight gradient: fp32 accumulator, C is D
    _matmul(ctx, 264, 136, 72, 0, 1, beta=1.0)                             # a residual epilogue in bf16
    _matmul(ctx, 72, 136, 64, 0, 0, dt=F16)
    _matmul(ctx, 520, 264, 64, 0, 1)                                       # 256 x 256 tiles with ragged edges


def test_long_k_few_tiles_takes_the_k_splits(ctx):
    _matmul(ctx, 64, 128, 4096 + 40, 0, 0)                                 # partial sums in the workspace, then the reduction
    _matmul(ctx, 64, 128, 4096 + 40, 0, 0, ws_floats=0)                    # no workspace: the same problem unsplit
    _matmul(ctx, 136, 72, 2048, 1, 0, ddt=F32, beta=1.0)


def test_zero_sized_problems_are_no_ops(ctx):
    L = sim.lib()
    for M, N, K in ((0, 8, 8), (8, 0, 8), (8, 8, 0)):
        assert L.dispatch_matmul(ctx, 0, M, N, K, 0, 8, 0, 8, 0, 8, 0, 8, 0, 0, 2, 2, 2, 2, 0, 1.0, 0.0, 0, 0) == 0


def test_random_shapes_layouts_and_paddings(ctx):
    """A sweep nobody chose by hand: any M, N, K (odd ones take the generic kernel), any layout, rows wider
    than needed, accumulation or not, with or without a workspace.  Every operand ends at a guard page."""
    g = torch.Generator().manual_seed(2024)
    r = lambda lo, hi: int(torch.randint(lo, hi + 1, (1,), generator=g))
    for case in range(48):
        multiple = 8 if case % 3 else 1
        M, N, K = (r(1, 40) * multiple for _ in range(3))
        if case % 8 == 0:
            K = r(1, 20) * 64 + r(0, 7) * 8                  # long enough for several K-steps and a tail
        _matmul(ctx, M, N, K, r(0, 1), r(0, 1), ddt=(BF, F32)[r(0, 1)], beta=float(r(0, 1)), alpha=(1.0, 0.5)[r(0, 1)],
                pad=r(0, 2) * 8, ws_floats=(1 << 18) * r(0, 1), seed=case)
