"""The MFMA GEMM behind the dispatcher ABI against fp32 CPU matmul.  Shapes and
checks follow the reference's own dispatcher tests
(helpers/matmul_dispatcher/tests/test_matmul_fast.py:44-149): max relative
error < 5e-2 (denominator clamped at 1e-3), alpha/beta/C-is-D in place, all
transpose combinations, matmul == matmul_fast bit for bit."""
import pytest
import torch

from flextrain_amd.matmul_dispatcher import CublasLtDispatcher, tensor_layout
from util import gen, randn

pytestmark = pytest.mark.gpu


def _ref(A, B, C=None, alpha=1.0, beta=0.0):
    r = alpha * (A.float() @ B.float())
    if C is not None:
        r = r + beta * C.float()
    return r


def _check(D, want, dtype):
    got = D.float().cpu()
    rel = ((got - want).abs() / want.abs().clamp(min=1e-3)).max().item()
    tol = 5e-2 if dtype != torch.float32 else 1e-3
    scale = want.abs().max().item()
    assert (got - want).abs().max().item() <= tol * max(scale, 1.0), f"abs err, scale {scale}"
    close = ((got - want).abs() <= 1e-2 * want.abs() + 1e-2 * max(scale, 1.0) * 0.05)
    assert close.float().mean().item() > 0.999, f"max rel {rel}"


SHAPES = [(200, 1024, 2048), (500, 2048, 512), (37, 16, 4096), (16, 1024, 16), (256, 256, 64), (1024, 1536, 2048),
          (513, 768, 2048), (128, 128, 8), (1, 8, 8), (3000, 4096, 1024),
          (2040, 3200, 200)]   # the last one takes the 256 x 128 tile (one full round of workgroups), ragged in M and K


@pytest.mark.parametrize("M,N,K", SHAPES)
@pytest.mark.parametrize("ta,tb", [(0, 0), (0, 1), (1, 0), (1, 1)])
def test_bf16_all_layouts(dev, M, N, K, ta, tb):
    g = gen(M * 7 + N * 3 + K + ta * 2 + tb)
    A = randn(g, M, K, std=0.5)
    B = randn(g, K, N, std=0.5)
    Ad = A.t().contiguous().to(dev).t() if ta else A.to(dev)
    Bd = B.t().contiguous().to(dev).t() if tb else B.to(dev)
    assert tensor_layout(Ad)[2] == (ta if M > 1 and K > 1 else tensor_layout(Ad)[2])
    disp = CublasLtDispatcher()
    s = torch.cuda.current_stream().cuda_stream
    D = disp.matmul(s, Ad, Bd)
    _check(D, _ref(A, B), torch.bfloat16)
    D2 = torch.empty_like(D)
    disp.matmul_fast(s, Ad, Bd, D=D2)
    assert torch.equal(D, D2)


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32, torch.bfloat16])
def test_alpha_beta_in_place_and_dtypes(dev, dtype):
    g = gen(5)
    M, N, K = 300, 512, 1024
    A, B, C = randn(g, M, K, dtype=dtype, std=0.3), randn(g, K, N, dtype=dtype, std=0.3), randn(g, M, N, dtype=dtype)
    disp = CublasLtDispatcher()
    s = torch.cuda.current_stream().cuda_stream
    Cd = C.to(dev)
    out = disp.matmul(s, A.to(dev), B.to(dev), C=Cd, D=Cd, alpha=0.5, beta=1.0)   # accumulate in place
    assert out.data_ptr() == Cd.data_ptr()
    _check(out, _ref(A, B, C, 0.5, 1.0), dtype)
    Dd = torch.empty(M, N, dtype=dtype, device=dev)
    disp.matmul(s, A.to(dev), B.to(dev), C=C.to(dev), D=Dd, alpha=2.0, beta=-0.5)
    _check(Dd, _ref(A, B, C, 2.0, -0.5), dtype)


def test_fp32_output_from_bf16_inputs_and_strided_views(dev):
    g = gen(6)
    M, N, K = 640, 384, 256
    big_a = randn(g, M, 2 * K, std=0.5)
    big_b = randn(g, N, 3 * K, std=0.5)       # stored (N, K): used transposed
    A, Bt = big_a[:, K:], big_b[:, K:2 * K]
    disp = CublasLtDispatcher()
    s = torch.cuda.current_stream().cuda_stream
    Ad, Btd = big_a.to(dev)[:, K:], big_b.to(dev)[:, K:2 * K]
    D = torch.zeros(M, 2 * N, dtype=torch.float32, device=dev)
    disp.matmul(s, Ad, Btd.t(), D=D[:, N:])
    _check(D[:, N:], _ref(A, Bt.t()), torch.bfloat16)
    assert not D[:, :N].any()


def test_cache_statistics_and_noop(dev):
    disp = CublasLtDispatcher(round_multiple=32)
    s = torch.cuda.current_stream().cuda_stream
    A = torch.ones(64, 64, dtype=torch.bfloat16, device=dev)
    assert disp.get_stats()["matmuls_called"] == 0
    disp.matmul(s, A, A)            # new algorithm
    disp.matmul(s, A, A)            # exact hit
    A2 = torch.ones(40, 64, dtype=torch.bfloat16, device=dev)
    disp.matmul(s, A2, A)           # rounds up to (64,64,64): fuzzy hit
    st = disp.get_stats()
    assert (st["matmuls_called"], st["algos_saved"], st["algo_hits"]) == (3, 1, 2)
    # zero-sized problems: the C entry returns 0 without work, the wrapper raises
    rc = disp._lib.dispatch_matmul(disp.ctx, s, 0, 64, 64, A.data_ptr(), 64, A.data_ptr(), 64, 0, 64,
                                   A.data_ptr(), 64, 0, 0, 2, 2, 2, 2, 0, 1.0, 0.0, 0, 0)
    assert rc == 0
    with pytest.raises(ValueError):
        disp.matmul(s, A[:0], A)
    with pytest.raises(ValueError):
        disp.matmul(s, A, torch.ones(32, 64, dtype=torch.bfloat16, device=dev))
    with pytest.raises(ValueError):
        tensor_layout(torch.ones(8, 8, 2, device=dev)[:, :, 0])


@pytest.mark.parametrize("M,N,K,ta,tb", [(256, 512, 16384, 0, 0), (300, 520, 8200, 0, 1), (1024, 4096, 32064, 0, 0),
                                         (512, 256, 12288, 1, 0)])
def test_long_k_few_tiles_splits_along_k(dev, M, N, K, ta, tb):
    """Few output tiles and a long K: the dispatcher cuts K into ranges, keeps fp32 partial sums in
    its workspace and reduces them (alpha / beta / C applied once, in the reduction)."""
    g = gen(M + K)
    A, B, C = randn(g, M, K, std=0.25), randn(g, K, N, std=0.25), randn(g, M, N)
    Ad = A.t().contiguous().to(dev).t() if ta else A.to(dev)
    Bd = B.t().contiguous().to(dev).t() if tb else B.to(dev)
    disp = CublasLtDispatcher()
    s = torch.cuda.current_stream().cuda_stream
    D = disp.matmul(s, Ad, Bd)
    assert disp.workspace is not None and disp.workspace.numel() == 64 * 1024 * 1024
    _check(D, _ref(A, B), torch.bfloat16)
    Cd = C.to(dev)
    disp.matmul(s, Ad, Bd, C=Cd, D=Cd, alpha=0.5, beta=1.0)
    _check(Cd, _ref(A, B, C, 0.5, 1.0), torch.bfloat16)
    # the same shape without a workspace runs unsplit and agrees
    rc_ws, disp.ws_ptr, disp.workspace_size = disp.ws_ptr, 0, 0
    D2 = torch.empty_like(D)
    disp.matmul_fast(s, Ad, Bd, D=D2)
    _check(D2, _ref(A, B), torch.bfloat16)
