// Gate / up projections of a dense gated FFN as ONE launch with the activation in the epilogue.
//
// The reference runs two GEMMs (x1 = h W_1, x3 = h W_3, both saved for the backward pass) and
// then a gated-activation kernel that reads them back (flextrain/nn/blocks/ffn_dense.py:130-146).
// Here a workgroup accumulates the same 128 columns of both products from one pass over its rows
// of h (each wave the same 64 columns of both), stores x1 and x3 and, from their rounded values,
// act(x1) * x3: the activation costs no
// extra pass over HBM and h is read once.  Results are those of the three separate launches.
#include "gemm_core2.h"
#include "flexhip.h"

namespace fx {

template <typename T, bool B_MN, int ACT>
__global__ __launch_bounds__(512) void gemm_dual_glu_kernel(
    const T* __restrict__ A, int64_t lda, const T* __restrict__ B1, const T* __restrict__ B2, int64_t ldb, T* P1, T* P2,
    int64_t ldp, T* ACTO, int64_t ldact, int M, int Nh, int K, int gate_first, int tiles_m, int tiles_n) {
    extern __shared__ __align__(16) unsigned char smem_raw[];
    int tm, tn;
    tile_coords(blockIdx.x, tiles_m, tiles_n, tm, tn);
    OperandView<T> a{A, lda, M, tm * 256};
    OperandView<T> b{B1, ldb, Nh, tn * 128, 64, B2};     // 4 x 2 waves of 64 x 128: 64 columns of each product per wave
    gemm_tile2_glu<T, 256, 256, 4, 2, B_MN, ACT>(a, b, P1, P2, ldp, ACTO, ldact, M, Nh, K, gate_first != 0,
                                                 reinterpret_cast<T*>(smem_raw));
}

template <typename T, bool B_MN, int ACT>
static void launch_dual(const void* A, int64_t lda, const void* B1, const void* B2, int64_t ldb, void* P1, void* P2,
                        int64_t ldp, void* act, int64_t ldact, int M, int Nh, int K, int gate_first, hipStream_t s) {
    auto kern = gemm_dual_glu_kernel<T, B_MN, ACT>;
    constexpr size_t lds = gemm2_glu_lds_bytes<T, 256, 256, 4, 2, false>();
    FX_ENSURE_DYNAMIC_LDS(kern, lds);
    const int tiles_m = (M + 255) / 256, tiles_n = (Nh + 127) / 128;
    kern<<<dim3((unsigned)(tiles_m * tiles_n)), 512, lds, s>>>(
        reinterpret_cast<const T*>(A), lda, reinterpret_cast<const T*>(B1), reinterpret_cast<const T*>(B2), ldb, reinterpret_cast<T*>(P1),
        reinterpret_cast<T*>(P2), ldp, reinterpret_cast<T*>(act), ldact, M, Nh, K, gate_first, tiles_m, tiles_n);
}

}  // namespace fx

using namespace fx;

extern "C" int fx_gemm_dual_glu(const void* A, int64_t lda, const void* B1, const void* B2, int64_t ldb, int trans_b,
                                void* P1, void* P2, int64_t ldp, void* act, int64_t ldact, int M, int Nh, int K,
                                int gate_first, int activation, int dt, hipStream_t stream) {
    if (M < 0 || Nh <= 0 || K <= 0) FX_FAIL("fx_gemm_dual_glu: bad shape");
    if (M == 0) return 0;
    if (!A || !B1 || !B2 || !P1 || !P2 || !act) FX_FAIL("fx_gemm_dual_glu: null pointer");
    if (dt != DT_BF16 && dt != DT_F16) FX_FAIL("fx_gemm_dual_glu: bf16 or fp16 only");
    if (lda >= (1 << 23) || ldb >= (1 << 23)) FX_FAIL("fx_gemm_dual_glu: leading dimensions must be below 2^23 elements");
    if (activation != ACT_SILU && activation != ACT_GELU_TANH) FX_FAIL("fx_gemm_dual_glu: unknown activation %d", activation);
    if ((K & 63) || (Nh & 7) || (lda & 7) || (ldb & 7) || (ldp & 7) || (ldact & 7) || !aligned16(A) || !aligned16(B1) ||
        !aligned16(B2) || !aligned16(P1) || !aligned16(P2) || !aligned16(act))
        FX_FAIL("fx_gemm_dual_glu: needs K %% 64 == 0, N %% 8 == 0, leading dimensions %% 8 == 0 and 16-byte aligned operands");
#define FX_DUAL(TT)                                                                                           \
    {                                                                                                         \
        if (activation == ACT_SILU) {                                                                         \
            if (trans_b) launch_dual<TT, false, ACT_SILU>(A, lda, B1, B2, ldb, P1, P2, ldp, act, ldact, M, Nh, K, gate_first, stream); \
            else launch_dual<TT, true, ACT_SILU>(A, lda, B1, B2, ldb, P1, P2, ldp, act, ldact, M, Nh, K, gate_first, stream); \
        } else {                                                                                              \
            if (trans_b) launch_dual<TT, false, ACT_GELU_TANH>(A, lda, B1, B2, ldb, P1, P2, ldp, act, ldact, M, Nh, K, gate_first, stream); \
            else launch_dual<TT, true, ACT_GELU_TANH>(A, lda, B1, B2, ldb, P1, P2, ldp, act, ldact, M, Nh, K, gate_first, stream); \
        }                                                                                                     \
    }
    if (dt == DT_BF16) FX_DUAL(bf16) else FX_DUAL(f16)
#undef FX_DUAL
    FX_CHECK_LAUNCH("fx_gemm_dual_glu");
    return 0;
}
