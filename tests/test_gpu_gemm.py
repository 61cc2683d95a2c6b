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
    assert bool(close.all()), f"{int((~close).sum())} of {close.numel()} outside rtol 1e-2, max rel {rel}"


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


@pytest.mark.parametrize("fast", [False, True])
@pytest.mark.parametrize("first_aligned", [True, False])
def test_one_dispatcher_aligned_then_offset_view_then_aligned(dev, fast, first_aligned):
    """The cached kernel choice must follow operand alignment: a column slice that starts 2 elements
    (4 bytes) into a row has the same shape and leading dimension as the aligned operand but cannot
    take the 16-byte loads of the MFMA kernel, and an unaligned first call must not pin the
    one-element-per-lane kernel on later aligned calls of that shape."""
    g = gen(91)
    M, N, K = 384, 512, 256
    wide = randn(g, M, K + 8, std=0.5)                   # lda = K + 8 for every view below
    B = randn(g, K, N, std=0.5)
    wd, Bd = wide.to(dev), B.to(dev)
    views = {True: (wide[:, :K], wd[:, :K]), False: (wide[:, 2:2 + K], wd[:, 2:2 + K])}
    assert views[True][1].data_ptr() % 16 == 0 and views[False][1].data_ptr() % 16 == 4
    disp = CublasLtDispatcher()
    s = torch.cuda.current_stream().cuda_stream
    call = disp.matmul_fast if fast else disp.matmul
    order = [first_aligned, not first_aligned, first_aligned, not first_aligned]
    outs = []
    for aligned in order:
        D = torch.empty(M, N, dtype=torch.bfloat16, device=dev)
        call(s, views[aligned][1], Bd, D=D)
        _check(D, _ref(views[aligned][0], B), torch.bfloat16)
        outs.append(D)
    assert torch.equal(outs[0], outs[2]) and torch.equal(outs[1], outs[3])
    st = disp.get_stats()
    # one MFMA tile choice saved (by the aligned call), calls 3 and 4 are exact hits of their own entries
    assert (st["matmuls_called"], st["algos_saved"], st["algo_hits"]) == (4, 1, 2)
    # the aligned calls ran the MFMA kernel, the offset ones did not: bf16 accumulation order differs
    # between the two kernels, but each is deterministic
    C0 = randn(g, M, N)
    Dc = C0.to(dev).clone()
    call(s, views[True][1], Bd, C=Dc, D=Dc, beta=1.0)     # same shape with a C term: a separate entry again
    _check(Dc, _ref(views[True][0], B, C0, 1.0, 1.0), torch.bfloat16)


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


# ---------------------------------------------------------------- products that share A, one launch
@pytest.mark.parametrize("M,K,Ns", [(512, 1024, (256, 256)),            # 128 x 128 tiles
                                    (4096, 512, (1024, 1024)),          # 256 x 256 tiles
                                    (696, 328, (136, 1000, 8)),         # ragged everywhere, three segments
                                    (4104, 192, (520, 264, 256, 1032))])  # four segments, large tile
@pytest.mark.parametrize("ta,tb", [(0, 0), (0, 1), (1, 0), (1, 1)])
def test_shared_a_products_in_one_launch(dev, M, K, Ns, ta, tb):
    g = gen(M + K + sum(Ns) + 2 * ta + tb)
    A = randn(g, M, K, std=0.5)
    Bs = [randn(g, K, n, std=0.5) for n in Ns]
    Cs = [randn(g, M, n) for n in Ns]
    Ad = A.t().contiguous().to(dev).t() if ta else A.to(dev)
    Bd = [b.t().contiguous().to(dev).t() if tb else b.to(dev) for b in Bs]
    disp = CublasLtDispatcher()
    s = torch.cuda.current_stream().cuda_stream
    assert disp._segments_ok(Ad, Bd, [torch.empty(M, n, dtype=torch.bfloat16, device=dev) for n in Ns], None)
    # beta = 0 into fresh outputs
    Ds = [torch.full((M, n), float("nan"), dtype=torch.bfloat16, device=dev) for n in Ns]
    disp.matmul_shared_a(s, Ad, Bd, Ds)
    for i, n in enumerate(Ns):
        _check(Ds[i], _ref(A, Bs[i]), torch.bfloat16)
        # the same tile kernel and K order as a call of its own, when that call takes no K splits
        alone = disp.matmul(s, Ad, Bd[i])
        _check(Ds[i], alone.float().cpu(), torch.bfloat16)
    # accumulate in place: D = 0.5 * A B + 2 C with C is D
    Dd = [c.to(dev) for c in Cs]
    disp.matmul_shared_a(s, Ad, Bd, Dd, Cs=Dd, alpha=0.5, beta=2.0)
    for i in range(len(Ns)):
        _check(Dd[i], _ref(A, Bs[i], Cs[i], 0.5, 2.0), torch.bfloat16)


def test_shared_a_outputs_inside_wider_buffers_and_fp16(dev):
    g = gen(77)
    M, K, Ns = 384, 256, (128, 384)
    A = randn(g, M, K, dtype=torch.float16, std=0.5)
    Bs = [randn(g, K, n, dtype=torch.float16, std=0.5) for n in Ns]
    wide = torch.full((M, 1024), 7.0, dtype=torch.float16, device=dev)
    Ds = [wide[:, 8:8 + Ns[0]], wide[:, 256:256 + Ns[1]]]        # row stride 1024, the first 16-byte aligned only
    disp = CublasLtDispatcher()
    disp.matmul_shared_a(torch.cuda.current_stream().cuda_stream, A.to(dev), [b.to(dev) for b in Bs], Ds)
    for i in range(2):
        _check(Ds[i], _ref(A, Bs[i]), torch.float16)
    assert torch.all(wide[:, :8] == 7.0) and torch.all(wide[:, 8 + Ns[0]:256] == 7.0) and torch.all(wide[:, 256 + Ns[1]:] == 7.0)


def test_shared_a_falls_back_to_separate_calls(dev):
    """Operands the one-launch form does not take (fp32 outputs, mixed forms of B, odd sizes) give
    the same results through one dispatcher call per product."""
    g = gen(78)
    M, K = 130, 264
    A = randn(g, M, K, std=0.5)
    B0, B1 = randn(g, K, 72, std=0.5), randn(g, K, 200, std=0.5)
    disp = CublasLtDispatcher()
    s = torch.cuda.current_stream().cuda_stream
    Ad = A.to(dev)
    mixed = [B0.to(dev), B1.t().contiguous().to(dev).t()]
    Ds = [torch.empty(M, 72, dtype=torch.bfloat16, device=dev), torch.empty(M, 200, dtype=torch.bfloat16, device=dev)]
    assert not disp._segments_ok(Ad, mixed, Ds, None)
    disp.matmul_shared_a(s, Ad, mixed, Ds)
    _check(Ds[0], _ref(A, B0), torch.bfloat16)
    _check(Ds[1], _ref(A, B1), torch.bfloat16)
    D32 = [torch.empty(M, 72, dtype=torch.float32, device=dev), torch.empty(M, 200, dtype=torch.float32, device=dev)]
    assert not disp._segments_ok(Ad, [B0.to(dev), B1.to(dev)], D32, None)
    disp.matmul_shared_a(s, Ad, [B0.to(dev), B1.to(dev)], D32)
    _check(D32[0], _ref(A, B0), torch.float32)
    with pytest.raises(ValueError):
        disp.matmul_shared_a(s, Ad, mixed, Ds[:1])


# ---------------------------------------------------------------- a sum of products, one launch
def _ref_sum(As, Bs, C=None, alpha=1.0, beta=0.0):
    r = sum(a.float() @ b.float() for a, b in zip(As, Bs)) * alpha
    if C is not None:
        r = r + beta * C.float()
    return r


@pytest.mark.parametrize("M,N,Ks", [(512, 384, (256, 64)),               # 128 x 128 tiles
                                    (4096, 4096, (512, 128, 128)),        # 256 x 256 tiles, short second and third products
                                    (696, 1000, (200, 72, 8)),            # ragged everywhere, K tails
                                    (3080, 4104, (64, 192, 136, 320))])   # four products
@pytest.mark.parametrize("ta,tb", [(0, 0), (0, 1), (1, 0), (1, 1)])
def test_sum_of_products_in_one_launch(dev, M, N, Ks, ta, tb):
    g = gen(M + N + sum(Ks) + 2 * ta + tb)
    As = [randn(g, M, k, std=0.5) for k in Ks]
    Bs = [randn(g, k, N, std=0.5) for k in Ks]
    C = randn(g, M, N)
    Ad = [a.t().contiguous().to(dev).t() if ta else a.to(dev) for a in As]
    Bd = [b.t().contiguous().to(dev).t() if tb else b.to(dev) for b in Bs]
    disp = CublasLtDispatcher()
    s = torch.cuda.current_stream().cuda_stream
    D = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device=dev)
    assert disp._ksum_ok(Ad, Bd, None, D)
    disp.matmul_sum(s, Ad, Bd, D=D)
    _check(D, _ref_sum(As, Bs), torch.bfloat16)
    # against the chain of accumulating calls it replaces (rounded after every product)
    chain = disp.matmul(s, Ad[0], Bd[0])
    for a, b in zip(Ad[1:], Bd[1:]):
        disp.matmul(s, a, b, C=chain, D=chain, beta=1.0)
    want = _ref_sum(As, Bs)
    err_fused = (D.float().cpu() - want).abs().mean().item()
    err_chain = (chain.float().cpu() - want).abs().mean().item()
    assert err_fused <= err_chain * 1.02 + 1e-6     # one rounding instead of one per product
    # alpha, beta and C is D; fp32 output
    Dc = C.to(dev)
    disp.matmul_sum(s, Ad, Bd, C=Dc, D=Dc, alpha=0.5, beta=2.0)
    _check(Dc, _ref_sum(As, Bs, C, 0.5, 2.0), torch.bfloat16)
    D32 = torch.empty(M, N, dtype=torch.float32, device=dev)
    assert disp._ksum_ok(Ad, Bd, None, D32)
    disp.matmul_sum(s, Ad, Bd, D=D32)
    _check(D32, _ref_sum(As, Bs), torch.float32)


def _check_chain(D, want):
    """A chain of accumulating bf16 calls rounds after every product: twice the single-rounding bound."""
    got = D.float().cpu()
    scale = max(want.abs().max().item(), 1.0)
    assert (got - want).abs().max().item() <= 5e-2 * scale
    bad = (got - want).abs() > 2e-2 * want.abs() + 1e-3 * scale
    assert not bool(bad.any()), f"{int(bad.sum())} of {bad.numel()} outside the chain bound"


def test_sum_of_products_falls_back_to_a_chain(dev):
    g = gen(91)
    M, N = 130, 72
    As = [randn(g, M, 264, std=0.5), randn(g, M, 100, std=0.5)]     # K = 100 is not a multiple of 8
    Bs = [randn(g, 264, N, std=0.5), randn(g, 100, N, std=0.5)]
    disp = CublasLtDispatcher()
    s = torch.cuda.current_stream().cuda_stream
    Ad, Bd = [a.to(dev) for a in As], [b.to(dev) for b in Bs]
    D = torch.empty(M, N, dtype=torch.bfloat16, device=dev)
    assert not disp._ksum_ok(Ad, Bd, None, D)
    out = disp.matmul_sum(s, Ad, Bd)
    _check_chain(out, _ref_sum(As, Bs))
    C = randn(g, M, N)
    Dc = C.to(dev)
    disp.matmul_sum(s, Ad, Bd, C=Dc, D=Dc, alpha=2.0, beta=0.5)
    # the chain applies alpha to every product and beta to C once
    _check_chain(Dc, _ref_sum(As, Bs, C, 2.0, 0.5))
    with pytest.raises(ValueError):
        disp.matmul_sum(s, Ad, Bd[:1])


def test_fused_entry_points_reject_what_they_cannot_take(dev):
    """Through the C ABI directly: a non-zero return and no launch for counts out of range,
    misaligned operands, sizes off the 8-element grid and unsupported dtypes."""
    import ctypes

    from flextrain_amd._lib import lib

    L = lib()
    s = torch.cuda.current_stream().cuda_stream
    A = torch.zeros(64, 72, dtype=torch.bfloat16, device=dev)
    B = torch.zeros(72, 64, dtype=torch.bfloat16, device=dev)
    D = torch.full((64, 64), 3.0, dtype=torch.bfloat16, device=dev)
    vp, i64, ci = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int

    def segments(nseg, a=A, b=B, ldb=64, n=64, dt=2):
        m = max(nseg, 1)
        return L.fx_gemm_segments(a.data_ptr(), 72, 0, nseg, (vp * m)(*[b.data_ptr()] * m), (i64 * m)(*[ldb] * m), 0, None, None,
                                  (vp * m)(*[D.data_ptr()] * m), (i64 * m)(*[64] * m), 64, (ci * m)(*[n] * m), 72, 1.0, 0.0, dt, s)

    assert segments(2) == 0
    assert segments(0) != 0 and segments(5) != 0
    assert segments(2, b=B.view(-1)[4:4 + 64 * 64].view(64, 64)) != 0      # B 8 bytes off the 16-byte grid
    assert segments(2, n=60) != 0                                          # columns of a (K, N) operand not a multiple of 8
    assert segments(2, dt=0) != 0                                          # fp32 inputs

    def ksum(nseg, k=72, d_dt=2, dt=2):
        m = max(nseg, 1)
        return L.fx_gemm_ksum(nseg, (vp * m)(*[A.data_ptr()] * m), (i64 * m)(*[72] * m), 0, (vp * m)(*[B.data_ptr()] * m),
                              (i64 * m)(*[64] * m), 0, (ci * m)(*[k] * m), None, 0, D.data_ptr(), 64, 64, 64, 1.0, 0.0, dt, d_dt, s)

    assert ksum(2) == 0
    assert ksum(0) != 0 and ksum(5) != 0
    assert ksum(2, k=68) != 0 and ksum(2, k=0) != 0
    assert ksum(2, d_dt=1) != 0 and ksum(2, dt=1, d_dt=0) != 0            # bf16 -> fp16, fp16 -> fp32
    torch.cuda.synchronize()
    assert torch.all(D == 0)     # the accepted calls wrote zeros (A, B are zero); the rejected ones nothing


def test_sum_of_products_fp16(dev):
    g = gen(93)
    M, N, Ks = 520, 392, (128, 72)
    As = [randn(g, M, k, dtype=torch.float16, std=0.5) for k in Ks]
    Bs = [randn(g, k, N, dtype=torch.float16, std=0.5) for k in Ks]
    disp = CublasLtDispatcher()
    Ad, Bd = [a.to(dev) for a in As], [b.t().contiguous().to(dev).t() for b in Bs]
    D = torch.empty(M, N, dtype=torch.float16, device=dev)
    assert disp._ksum_ok(Ad, Bd, None, D)
    disp.matmul_sum(torch.cuda.current_stream().cuda_stream, Ad, Bd, D=D)
    _check(D, _ref_sum(As, Bs), torch.float16)


def test_raw_fast_call_entry(dev):
    """The 24-argument C entry (helpers/matmul_dispatcher/src/dispatch_pyext.cpp:37-140): same bits as
    matmul, RuntimeError when dispatch_matmul reports failure."""
    from flextrain_amd import matmul_dispatcher as md

    g = gen(77)
    A, B = randn(g, 300, 512, std=0.5).to(dev), randn(g, 512, 640, std=0.5).to(dev)
    disp = CublasLtDispatcher()
    s = torch.cuda.current_stream().cuda_stream
    want = disp.matmul(s, A, B)
    D = torch.zeros_like(want)
    disp._ensure_workspace(A.device)
    args = [disp._ctx_int, s, 300, 640, 512, A.data_ptr(), 512, 0, B.data_ptr(), 640, 0, 0, 640, D.data_ptr(), 640,
            disp.ws_ptr, disp.workspace_size, 2, 2, 2, 2, 0, 1.0, 0.0]
    assert md.matmul_fast(*args) is None
    assert torch.equal(D, want)
    # integer alpha / beta are accepted like floats
    args[22], args[23] = 1, 0
    md.matmul_fast(*args)
    assert torch.equal(D, want)
    bad = list(args)
    bad[5] = 0                      # null A: dispatch_matmul returns non-zero
    with pytest.raises(RuntimeError):
        md.matmul_fast(*bad)
    bad = list(args)
    bad[17] = 1                     # A and B dtypes differ
    with pytest.raises(RuntimeError):
        md.matmul_fast(*bad)
