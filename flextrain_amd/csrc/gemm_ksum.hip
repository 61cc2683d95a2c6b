// A sum of products into one output, as one launch:
//   D = alpha * sum_i op(A_i) * op(B_i) + beta * C,   op(A_i): M x K_i,  op(B_i): K_i x N.
//
// The reference accumulates such sums with one dispatcher call per product and beta = 1: the
// gradient with respect to the attention-norm output is dq Wq^T, += dk Wk^T, += dv Wv^T
// (flextrain/nn/blocks/attention.py:712-775), the gradient entering the FFN norm dx1 W1^T, += dx3 W3^T
// (flextrain/nn/blocks/ffn_dense.py:193-235).  Every further call re-reads and re-writes the whole
// output, and the short products (K = 1024 for key / value) spend a large share of their time in
// prologue and epilogue.  Here a workgroup keeps its accumulators across the products: the K loop
// runs once per pair, the epilogue once.  The sum is formed in fp32 and rounded once (the separate
// calls round after every product).
#include "gemm_core2.h"
#include "flexhip.h"

namespace fx {

constexpr int MAX_KSEG = FX_GEMM_MAX_SEGMENTS;

struct KSegments {
    const void* a[MAX_KSEG];
    const void* b[MAX_KSEG];
    int64_t lda[MAX_KSEG], ldb[MAX_KSEG];
    int k[MAX_KSEG];
};

template <typename T, typename TD, int BM, int BN, int WAVES_M, int WAVES_N, bool A_MN, bool B_MN>
__global__ __launch_bounds__(WAVES_M * WAVES_N * 64) void gemm_ksum_kernel(
    const KSegments sg, int nseg, const TD* C, TD* D, int64_t ldc, int64_t ldd, int M, int N, float alpha, float beta,
    int tiles_m, int tiles_n) {
    extern __shared__ __align__(16) unsigned char smem_raw[];
    T* smem = reinterpret_cast<T*>(smem_raw);
    constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N;
    int tm, tn;
    tile_coords(blockIdx.x, tiles_m, tiles_n, tm, tn);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int wm = wave / WAVES_N, wn = wave % WAVES_N;
    f32x16_t acc[WM / 32][WN / 32];
#pragma unroll
    for (int i = 0; i < WM / 32; ++i)
#pragma unroll
        for (int j = 0; j < WN / 32; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;
    for (int s = 0; s < nseg; ++s) {
        // select the pair with compares (the struct stays in the kernel-argument segment)
        const void* ap = sg.a[0];
        const void* bp = sg.b[0];
        int64_t lda = sg.lda[0], ldb = sg.ldb[0];
        int k = sg.k[0];
#pragma unroll
        for (int u = 1; u < MAX_KSEG; ++u) {
            if (s == u) {
                ap = sg.a[u]; bp = sg.b[u];
                lda = sg.lda[u]; ldb = sg.ldb[u];
                k = sg.k[u];
            }
        }
        OperandView<T> a{reinterpret_cast<const T*>(ap), lda, M, tm * BM};
        OperandView<T> b{reinterpret_cast<const T*>(bp), ldb, N, tn * BN};
        gemm_mainloop2<T, BM, BN, WAVES_M, WAVES_N, A_MN, B_MN, false, false>(a, b, k, smem, acc);
    }
    epilogue_tile<T, TD, WM, WN>(acc, C, D, ldc, ldd, tm * BM + wm * WM, tn * BN + wn * WN, M, N, alpha, beta, smem, wave, lane);
}

template <typename T, typename TD, int BM, int BN, int WAVES_M, int WAVES_N, bool A_MN, bool B_MN>
static void launch_ksum(const KSegments& sg, int nseg, const void* C, void* D, int64_t ldc, int64_t ldd, int M, int N,
                        float alpha, float beta, hipStream_t s) {
    auto kern = gemm_ksum_kernel<T, TD, BM, BN, WAVES_M, WAVES_N, A_MN, B_MN>;
    constexpr size_t lds = gemm2_lds_bytes<T, BM, BN, WAVES_M, WAVES_N>();
    FX_ENSURE_DYNAMIC_LDS(kern, lds);
    const int tiles_m = (M + BM - 1) / BM, tiles_n = (N + BN - 1) / BN;
    kern<<<dim3((unsigned)(tiles_m * tiles_n)), WAVES_M * WAVES_N * 64, lds, s>>>(
        sg, nseg, reinterpret_cast<const TD*>(C), reinterpret_cast<TD*>(D), ldc, ldd, M, N, alpha, beta, tiles_m, tiles_n);
}

template <typename T, typename TD, int BM, int BN, int WAVES_M, int WAVES_N>
static void launch_ksum_layout(int ta, int tb, const KSegments& sg, int nseg, const void* C, void* D, int64_t ldc,
                               int64_t ldd, int M, int N, float alpha, float beta, hipStream_t s) {
    // operand form: A is MN-contiguous when transposed, B when NOT transposed
    if (!ta && tb) launch_ksum<T, TD, BM, BN, WAVES_M, WAVES_N, false, false>(sg, nseg, C, D, ldc, ldd, M, N, alpha, beta, s);
    else if (!ta && !tb) launch_ksum<T, TD, BM, BN, WAVES_M, WAVES_N, false, true>(sg, nseg, C, D, ldc, ldd, M, N, alpha, beta, s);
    else if (ta && tb) launch_ksum<T, TD, BM, BN, WAVES_M, WAVES_N, true, false>(sg, nseg, C, D, ldc, ldd, M, N, alpha, beta, s);
    else launch_ksum<T, TD, BM, BN, WAVES_M, WAVES_N, true, true>(sg, nseg, C, D, ldc, ldd, M, N, alpha, beta, s);
}

}  // namespace fx

using namespace fx;

extern "C" int fx_gemm_ksum(int nseg, const void* const* A, const int64_t* lda, int trans_a, const void* const* B,
                            const int64_t* ldb, int trans_b, const int* K, const void* C, int64_t ldc, void* D,
                            int64_t ldd, int M, int N, float alpha, float beta, int dt, int d_dt,
                            hipStream_t stream) {
    if (nseg < 1 || nseg > MAX_KSEG) FX_FAIL("fx_gemm_ksum: %d products (1..%d supported)", nseg, MAX_KSEG);
    if (M < 0 || N < 0) FX_FAIL("fx_gemm_ksum: bad shape");
    if (!A || !lda || !B || !ldb || !K || !D) FX_FAIL("fx_gemm_ksum: null pointer");
    if (dt != DT_BF16 && dt != DT_F16) FX_FAIL("fx_gemm_ksum: bf16 or fp16 inputs only");
    if (d_dt != dt && !(dt == DT_BF16 && d_dt == DT_F32)) FX_FAIL("fx_gemm_ksum: the output must match the inputs or be fp32 (bf16 inputs)");
    if (M == 0 || N == 0) return 0;
    if (!C || beta == 0.f) { C = nullptr; beta = 0.f; }
    if ((trans_a && (M & 7)) || (!trans_b && (N & 7)))
        FX_FAIL("fx_gemm_ksum: an operand's contiguous axis must be a multiple of 8");
    KSegments sg{};
    for (int i = 0; i < nseg; ++i) {
        if (K[i] <= 0) FX_FAIL("fx_gemm_ksum: product %d has K = %d", i, K[i]);
        if (!A[i] || !B[i]) FX_FAIL("fx_gemm_ksum: null operand in product %d", i);
        if (!aligned16(A[i]) || !aligned16(B[i]) || (lda[i] & 7) || (ldb[i] & 7) || lda[i] >= (1 << 23) ||
            ldb[i] >= (1 << 23) || (K[i] & 7))
            FX_FAIL("fx_gemm_ksum: operands of product %d must be 16-byte aligned, K and the leading dimensions multiples of 8, leading dimensions below 2^23", i);
        sg.a[i] = A[i];
        sg.b[i] = B[i];
        sg.lda[i] = lda[i];
        sg.ldb[i] = ldb[i];
        sg.k[i] = K[i];
    }
    // the largest tile when it gives at least three quarters of the CUs a workgroup, else 128 x 128
    const bool big = (long)((M + 255) / 256) * ((N + 255) / 256) >= 192;
#define FX_KS(TT, TD_)                                                                                                     \
    {                                                                                                                      \
        if (big) launch_ksum_layout<TT, TD_, 256, 256, 2, 4>(trans_a, trans_b, sg, nseg, C, D, ldc, ldd, M, N, alpha, beta, stream); \
        else launch_ksum_layout<TT, TD_, 128, 128, 2, 2>(trans_a, trans_b, sg, nseg, C, D, ldc, ldd, M, N, alpha, beta, stream);     \
    }
    if (dt == DT_BF16 && d_dt == DT_BF16) FX_KS(bf16, bf16)
    else if (dt == DT_BF16) FX_KS(bf16, float)
    else FX_KS(f16, f16)
#undef FX_KS
    FX_CHECK_LAUNCH("fx_gemm_ksum");
    return 0;
}
