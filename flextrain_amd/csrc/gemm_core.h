// bf16 / fp16 MFMA GEMM building block for gfx950.
//
//   D[M,N] = alpha * op(A)[M,K] * op(B)[K,N] + beta * C[M,N]       (fp32 accumulate)
//
// One workgroup of 256 lanes (4 waves, 2x2) owns a BM x BN tile of D and walks
// K in steps of 64.  Each wave owns a (BM/2) x (BN/2) sub-tile built from
// v_mfma_f32_32x32x16 instructions.  Both operand tiles live in LDS in a
// "K-contiguous" form: row r (an m or n index) holds its 64 k-values as eight
// 16-byte chunks, chunk c stored at position c ^ (r & 7) so that the eight lanes
// that are serviced together by a ds_read_b128 / ds_write_b128 hit distinct banks.
//
// Operands come from global memory in one of two forms:
//   K-contiguous  (A not transposed, B transposed): 16-byte chunks are copied as is;
//   MN-contiguous (A transposed, B not transposed): a lane loads an 8(k) x 8(mn)
//     block as eight 16-byte rows, transposes it in registers with v_perm_b32 and
//     writes eight K-contiguous chunks.
// The next K-step's global loads are issued before the current step's MFMAs and
// parked in registers, so HBM/L2 latency overlaps the matrix pipe.
#pragma once
#include "common.h"

namespace fx {

typedef bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef f16 f16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x16_t __attribute__((ext_vector_type(16)));
typedef unsigned int u32x4_t __attribute__((ext_vector_type(4)));

template <typename T> struct Mfma32;
template <> struct Mfma32<bf16> {
    typedef bf16x8_t frag;
    static FX_DEV f32x16_t run(frag a, frag b, f32x16_t c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
    }
};
template <> struct Mfma32<f16> {
    typedef f16x8_t frag;
    static FX_DEV f32x16_t run(frag a, frag b, f32x16_t c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
    }
};

constexpr int GEMM_BK = 64;
constexpr int GEMM_THREADS = 256;

// One operand of one workgroup tile.
//   base : element pointer to the operand matrix of this problem
//   ld   : leading dimension in elements
//   ext  : extent along the tile's m (or n) axis, rows at or beyond it are never stored
//   origin: first m (or n) index of this tile
template <typename T>
struct OperandView {
    const T* base;
    int64_t ld;
    int ext;
    int origin;
    // Two-matrix tile (loaders instantiated with DUAL): tile rows >= half come from the matrix
    // at `base2` (same ld and extent), at index origin + row - half.
    int half = 0;
    const T* base2 = nullptr;
};

// Registers that park one K-step of one operand tile (ROWS x 64 elements):
// ROWS*8 chunks of 16 bytes over 256 lanes.
template <int ROWS>
struct Staged {
    static constexpr int N = ROWS * 8 / GEMM_THREADS;  // 8 for 256 rows, 4 for 128
    u32x4_t v[N];
};

FX_DEV u32x4_t ldg16(const void* p) { return *reinterpret_cast<const u32x4_t*>(p); }

// ---- global -> registers ---------------------------------------------------
template <typename T, int ROWS, bool MN_CONTIG>
FX_DEV void stage_load(Staged<ROWS>& st, const OperandView<T>& op, int k0, int K, int tid) {
    constexpr int N = Staged<ROWS>::N;
    const u32x4_t zero = {0u, 0u, 0u, 0u};
    if (!MN_CONTIG) {
        // chunk id = i*256 + tid : row = id/8, k-chunk = id%8
#pragma unroll
        for (int i = 0; i < N; ++i) {
            const int id = i * GEMM_THREADS + tid;
            const int r = id >> 3, c = id & 7;
            int g = op.origin + r;
            g = g < op.ext ? g : op.ext - 1;  // clamp: duplicates are never stored
            const int k = k0 + c * 8;
            st.v[i] = k < K ? ldg16(op.base + (int64_t)g * op.ld + k) : zero;
        }
    } else {
        // 8x8 blocks: block id = tid (+256 for the second half of 8-row groups):
        // kb = id%8 (k-chunk), nb = id/8 (group of 8 mn indices).  N == 8 rows of one
        // block when ROWS == 256; when ROWS == 128 a lane holds half a block (4 rows).
        constexpr int ROWS_PER_LANE = N;  // k-rows of the block held by this lane
        const int blocks = ROWS;          // (ROWS/8) * 8
        const int id = (ROWS_PER_LANE == 8) ? tid : (tid >> 1);
        const int half = (ROWS_PER_LANE == 8) ? 0 : (tid & 1);
        (void)blocks;
        const int kb = id & 7, nb = id >> 3;
        int g = op.origin + nb * 8;
        g = g + 8 <= op.ext ? g : op.ext - 8;
#pragma unroll
        for (int j = 0; j < N; ++j) {
            const int k = k0 + kb * 8 + half * 4 + j;
            st.v[j] = k < K ? ldg16(op.base + (int64_t)k * op.ld + g) : zero;
        }
    }
}

// ---- registers -> LDS (K-contiguous, swizzled) -------------------------------
template <typename T, int ROWS, bool MN_CONTIG>
FX_DEV void stage_store(const Staged<ROWS>& st, T* lds, int tid) {
    constexpr int N = Staged<ROWS>::N;
    if (!MN_CONTIG) {
#pragma unroll
        for (int i = 0; i < N; ++i) {
            const int id = i * GEMM_THREADS + tid;
            const int r = id >> 3, c = id & 7;
            *reinterpret_cast<u32x4_t*>(lds + r * GEMM_BK + ((c ^ (r & 7)) << 3)) = st.v[i];
        }
    } else if (N == 8) {
        const int kb = tid & 7, nb = tid >> 3;
        // in[j] = k-row j of the block: dword d holds mn = 2d (low half) and 2d+1 (high half)
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int d = i >> 1;
            const unsigned sel = (i & 1) ? 0x07060302u : 0x05040100u;
            u32x4_t o;
            o[0] = __builtin_amdgcn_perm(st.v[1][d], st.v[0][d], sel);
            o[1] = __builtin_amdgcn_perm(st.v[3][d], st.v[2][d], sel);
            o[2] = __builtin_amdgcn_perm(st.v[5][d], st.v[4][d], sel);
            o[3] = __builtin_amdgcn_perm(st.v[7][d], st.v[6][d], sel);
            const int r = nb * 8 + i;
            *reinterpret_cast<u32x4_t*>(lds + r * GEMM_BK + ((kb ^ (r & 7)) << 3)) = o;
        }
    } else {
        // half blocks: this lane holds k-rows half*4 .. half*4+3 -> 8-byte halves of each chunk
        const int id = tid >> 1, half = tid & 1;
        const int kb = id & 7, nb = id >> 3;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int d = i >> 1;
            const unsigned sel = (i & 1) ? 0x07060302u : 0x05040100u;
            uint2 o;
            o.x = __builtin_amdgcn_perm(st.v[1][d], st.v[0][d], sel);
            o.y = __builtin_amdgcn_perm(st.v[3][d], st.v[2][d], sel);
            const int r = nb * 8 + i;
            *reinterpret_cast<uint2*>(lds + r * GEMM_BK + ((kb ^ (r & 7)) << 3) + half * 4) = o;
        }
    }
}

// ---- epilogue ----------------------------------------------------------------
// acc layout of v_mfma_f32_32x32x16: lane l, register v ->
//   row = 8*(v/4) + 4*(l/32) + (v%4),  col = l%32.
template <typename TD>
FX_DEV void store_tile(const f32x16_t& acc, TD* D, const TD* C, int64_t ldd, int64_t ldc, int row0, int col0,
                       int M, int N, float alpha, float beta, int lane) {
    const int col = col0 + (lane & 31);
    if (col >= N) return;
#pragma unroll
    for (int v = 0; v < 16; ++v) {
        const int row = row0 + 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3);
        if (row < M) {
            float r = alpha * acc[v];
            if (beta != 0.f) r += beta * (float)C[(int64_t)row * ldc + col];
            D[(int64_t)row * ldd + col] = (TD)r;
        }
    }
}

// The whole tile computation.  `smem` must hold (BM + BN) * 64 elements of T.
template <typename T, typename TD, int BM, int BN, bool A_MN, bool B_MN>
FX_DEV void gemm_tile(const OperandView<T>& A, const OperandView<T>& B, const TD* C, TD* D, int64_t ldc,
                      int64_t ldd, int M, int N, int K, int kbegin, float alpha, float beta, T* smem) {
    constexpr int WM = BM / 2, WN = BN / 2;
    constexpr int TM = WM / 32, TN = WN / 32;
    typedef typename Mfma32<T>::frag frag;
    T* As = smem;
    T* Bs = smem + BM * GEMM_BK;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;

    f32x16_t acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

    Staged<BM> sa;
    Staged<BN> sb;
    const int nk = (K - kbegin + GEMM_BK - 1) / GEMM_BK;
    if (nk > 0) {
        stage_load<T, BM, A_MN>(sa, A, kbegin, K, tid);
        stage_load<T, BN, B_MN>(sb, B, kbegin, K, tid);
    }
    for (int kt = 0; kt < nk; ++kt) {
        __syncthreads();  // previous step's LDS reads are done
        stage_store<T, BM, A_MN>(sa, As, tid);
        stage_store<T, BN, B_MN>(sb, Bs, tid);
        __syncthreads();
        if (kt + 1 < nk) {
            stage_load<T, BM, A_MN>(sa, A, kbegin + (kt + 1) * GEMM_BK, K, tid);
            stage_load<T, BN, B_MN>(sb, B, kbegin + (kt + 1) * GEMM_BK, K, tid);
        }
#pragma unroll
        for (int ks = 0; ks < GEMM_BK / 16; ++ks) {
            frag af[TM], bfv[TN];
            const int chunk = ks * 2 + (lane >> 5);
#pragma unroll
            for (int i = 0; i < TM; ++i) {
                const int r = wm * WM + i * 32 + (lane & 31);
                af[i] = *reinterpret_cast<const frag*>(As + r * GEMM_BK + ((chunk ^ (r & 7)) << 3));
            }
#pragma unroll
            for (int j = 0; j < TN; ++j) {
                const int r = wn * WN + j * 32 + (lane & 31);
                bfv[j] = *reinterpret_cast<const frag*>(Bs + r * GEMM_BK + ((chunk ^ (r & 7)) << 3));
            }
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j) acc[i][j] = Mfma32<T>::run(af[i], bfv[j], acc[i][j]);
        }
    }
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
            store_tile<TD>(acc[i][j], D, C, ldd, ldc, A.origin + wm * WM + i * 32, B.origin + wn * WN + j * 32, M, N,
                           alpha, beta, lane);
}

}  // namespace fx
