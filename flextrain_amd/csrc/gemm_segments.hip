// Several GEMMs that share op(A), as one launch:  D_i = alpha * op(A) * op(B_i) + beta * C_i.
//
// The reference issues one dispatcher call per projection: key and value projections of a GQA
// block (flextrain/nn/blocks/attention.py:424-463) are two [T, d] x [d, 1024] products, and their
// weight gradients (attention.py:712-775) two [d, T] x [T, 1024] products.  Each alone has too few
// output tiles for 256 CUs (one round of small tiles, or K splits plus a reduction pass); side by
// side their column tiles make one grid: tile column tn belongs to the segment whose range of
// column tiles contains it, and a tile never straddles two segments.  Results are those of the
// separate calls (same tile kernels, same K order).
#include "gemm_core2.h"
#include "flexhip.h"

namespace fx {

constexpr int MAX_SEG = FX_GEMM_MAX_SEGMENTS;

struct Segments {
    const void* b[MAX_SEG];
    const void* c[MAX_SEG];
    void* d[MAX_SEG];
    int64_t ldb[MAX_SEG], ldc[MAX_SEG], ldd[MAX_SEG];
    int n[MAX_SEG];
    int tile_end[MAX_SEG];   // running count of column tiles up to and including segment i
};

template <typename T, int BM, int BN, int WAVES_M, int WAVES_N, bool A_MN, bool B_MN>
__global__ __launch_bounds__(WAVES_M * WAVES_N * 64) void gemm_segments_kernel(
    const T* __restrict__ A, int64_t lda, const Segments sg, int M, int K, float alpha, float beta, int tiles_m,
    int tiles_n) {
    extern __shared__ __align__(16) unsigned char smem_raw[];
    T* smem = reinterpret_cast<T*>(smem_raw);
    int tm, tn;
    tile_coords(blockIdx.x, tiles_m, tiles_n, tm, tn);
    // select the segment with compares (the struct stays in the kernel-argument segment)
    const void* bp = sg.b[0];
    const void* cp = sg.c[0];
    void* dp = sg.d[0];
    int64_t ldb = sg.ldb[0], ldc = sg.ldc[0], ldd = sg.ldd[0];
    int n = sg.n[0], first = 0;
#pragma unroll
    for (int s = 1; s < MAX_SEG; ++s) {
        if (tn >= sg.tile_end[s - 1]) {
            bp = sg.b[s]; cp = sg.c[s]; dp = sg.d[s];
            ldb = sg.ldb[s]; ldc = sg.ldc[s]; ldd = sg.ldd[s];
            n = sg.n[s]; first = sg.tile_end[s - 1];
        }
    }
    OperandView<T> a{A, lda, M, tm * BM};
    OperandView<T> b{reinterpret_cast<const T*>(bp), ldb, n, (tn - first) * BN};
    gemm_tile2<T, T, BM, BN, WAVES_M, WAVES_N, A_MN, B_MN>(a, b, reinterpret_cast<const T*>(cp), reinterpret_cast<T*>(dp),
                                                           ldc, ldd, M, n, K, alpha, beta, smem);
}

template <typename T, int BM, int BN, int WAVES_M, int WAVES_N, bool A_MN, bool B_MN>
static void launch_segments(const void* A, int64_t lda, Segments& sg, int nseg, int M, int K, float alpha, float beta,
                            hipStream_t s) {
    auto kern = gemm_segments_kernel<T, BM, BN, WAVES_M, WAVES_N, A_MN, B_MN>;
    constexpr size_t lds = gemm2_lds_bytes<T, BM, BN, WAVES_M, WAVES_N>();
    FX_ENSURE_DYNAMIC_LDS(kern, lds);
    int tiles_n = 0;
    for (int i = 0; i < MAX_SEG; ++i) {
        if (i < nseg) tiles_n += (sg.n[i] + BN - 1) / BN;
        sg.tile_end[i] = i < nseg ? tiles_n : 0x7fffffff;   // unused slots never match
    }
    const int tiles_m = (M + BM - 1) / BM;
    kern<<<dim3((unsigned)(tiles_m * tiles_n)), WAVES_M * WAVES_N * 64, lds, s>>>(reinterpret_cast<const T*>(A), lda, sg, M, K,
                                                                                 alpha, beta, tiles_m, tiles_n);
}

template <typename T, int BM, int BN, int WAVES_M, int WAVES_N>
static void launch_segments_layout(const void* A, int64_t lda, int ta, int tb, Segments& sg, int nseg, int M, int K,
                                   float alpha, float beta, hipStream_t s) {
    // operand form: A is MN-contiguous when transposed, B when NOT transposed
    if (!ta && tb) launch_segments<T, BM, BN, WAVES_M, WAVES_N, false, false>(A, lda, sg, nseg, M, K, alpha, beta, s);
    else if (!ta && !tb) launch_segments<T, BM, BN, WAVES_M, WAVES_N, false, true>(A, lda, sg, nseg, M, K, alpha, beta, s);
    else if (ta && tb) launch_segments<T, BM, BN, WAVES_M, WAVES_N, true, false>(A, lda, sg, nseg, M, K, alpha, beta, s);
    else launch_segments<T, BM, BN, WAVES_M, WAVES_N, true, true>(A, lda, sg, nseg, M, K, alpha, beta, s);
}

}  // namespace fx

using namespace fx;

extern "C" int fx_gemm_segments(const void* A, int64_t lda, int trans_a, int nseg, const void* const* B,
                                const int64_t* ldb, int trans_b, const void* const* C, const int64_t* ldc,
                                void* const* D, const int64_t* ldd, int M, const int* N, int K, float alpha,
                                float beta, int dt, hipStream_t stream) {
    if (nseg < 1 || nseg > MAX_SEG) FX_FAIL("fx_gemm_segments: %d segments (1..%d supported)", nseg, MAX_SEG);
    if (M < 0 || K <= 0) FX_FAIL("fx_gemm_segments: bad shape");
    if (!A || !B || !ldb || !D || !ldd || !N) FX_FAIL("fx_gemm_segments: null pointer");
    if (dt != DT_BF16 && dt != DT_F16) FX_FAIL("fx_gemm_segments: bf16 or fp16 only");
    if (M == 0) return 0;
    const bool has_c = C != nullptr && ldc != nullptr && beta != 0.f;
    if (!has_c) beta = 0.f;
    if (!aligned16(A) || (lda & 7) || lda >= (1 << 23) || (trans_a ? (M & 7) : (K & 7)))
        FX_FAIL("fx_gemm_segments: A must be 16-byte aligned, its contiguous axis and leading dimension multiples of 8, lda below 2^23");
    Segments sg{};
    long tiles256 = 0, tiles128 = 0;
    for (int i = 0; i < nseg; ++i) {
        if (N[i] <= 0) FX_FAIL("fx_gemm_segments: segment %d has %d columns", i, N[i]);
        if (!B[i] || !D[i] || (has_c && !C[i])) FX_FAIL("fx_gemm_segments: null operand in segment %d", i);
        if (!aligned16(B[i]) || (ldb[i] & 7) || ldb[i] >= (1 << 23) || (trans_b ? (K & 7) : (N[i] & 7)))
            FX_FAIL("fx_gemm_segments: B[%d] must be 16-byte aligned, its contiguous axis and leading dimension multiples of 8, ldb below 2^23", i);
        sg.b[i] = B[i];
        sg.c[i] = has_c ? C[i] : nullptr;
        sg.d[i] = D[i];
        sg.ldb[i] = ldb[i];
        sg.ldc[i] = has_c ? ldc[i] : 0;
        sg.ldd[i] = ldd[i];
        sg.n[i] = N[i];
        tiles256 += (N[i] + 255) / 256;
        tiles128 += (N[i] + 127) / 128;
    }
    tiles256 *= (M + 255) / 256;
    tiles128 *= (M + 127) / 128;
    (void)tiles128;
    // the largest tile when it gives at least three quarters of the CUs a workgroup, else 128 x 128
    const bool big = tiles256 >= 192;
#define FX_SEG(TT)                                                                                                    \
    {                                                                                                                 \
        if (big) launch_segments_layout<TT, 256, 256, 2, 4>(A, lda, trans_a, trans_b, sg, nseg, M, K, alpha, beta, stream); \
        else launch_segments_layout<TT, 128, 128, 2, 2>(A, lda, trans_a, trans_b, sg, nseg, M, K, alpha, beta, stream);     \
    }
    if (dt == DT_BF16) FX_SEG(bf16) else FX_SEG(f16)
#undef FX_SEG
    FX_CHECK_LAUNCH("fx_gemm_segments");
    return 0;
}
