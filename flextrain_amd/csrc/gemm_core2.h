// bf16 / fp16 MFMA GEMM building block for gfx950, second generation.
//
//   D[M,N] = alpha * op(A)[M,K] * op(B)[K,N] + beta * C[M,N]       (fp32 accumulate)
//
// A workgroup of WAVES_M x WAVES_N waves owns a BM x BN tile of D and walks K in steps of
// 64.  Each wave owns a (BM/WAVES_M) x (BN/WAVES_N) sub-tile built from
// v_mfma_f32_32x32x16.  Operand tiles live in LDS "K-contiguous": row r (an m or n index)
// holds its 64 k-values as eight 16-byte chunks, chunk c stored at position c ^ (r & 7).
// Two LDS buffers alternate, so a K-step needs one barrier: while the matrix pipe works on
// buffer t, the loads of step t+1 fill buffer t+1.
//
// Operands reach LDS in one of two ways:
//   K-contiguous in memory (A not transposed, B transposed): global_load_lds_dwordx4 moves
//     16 bytes per lane straight from global memory into LDS, no registers in between; the
//     XOR swizzle is applied to the global address (a lane picks the chunk that belongs at
//     its fixed LDS position).
//   M/N-contiguous in memory (A transposed, B not transposed): a lane loads an 8(k) x 8(mn)
//     block as eight 16-byte rows, transposes it in registers with v_perm_b32 and writes
//     eight K-contiguous chunks with ds_write_b128.
// Rows outside the matrix are clamped to the last valid row (their products are never
// stored); a K tail shorter than 64 goes through the register path, which zero-fills.
#pragma once
#include "gemm_core.h"

namespace fx {

#ifndef GEMM_SWZ_SHIFT
#define GEMM_SWZ_SHIFT 1
#endif
// Swizzle: chunk c of row r sits at position c ^ swz(r).
FX_DEV int swz(int r) { return (r >> GEMM_SWZ_SHIFT) & 7; }

typedef __attribute__((address_space(3))) void* lds_ptr_t;
typedef const __attribute__((address_space(1))) void* gbl_ptr_t;

// 16 bytes per lane, global -> LDS; lds_base is wave-uniform, lane l lands at lds_base + 16*l.
FX_DEV void load_to_lds16(const void* gptr, void* lds_base) {
    __builtin_amdgcn_global_load_lds((gbl_ptr_t)gptr, (lds_ptr_t)lds_base, 16, 0, 0);
}

// Direct copy of a ROWS x 64 K-contiguous tile.  One wave instruction covers 8 rows
// (8 lanes per row); instruction j of wave w covers rows (j*NW + w)*8 ...
template <typename T, int ROWS, int NW>
FX_DEV void tile_load_direct(const OperandView<T>& op, int k0, T* lds, int wave, int lane) {
    constexpr int NI = ROWS / 8 / NW;
    static_assert(ROWS % (8 * NW) == 0, "tile rows must split evenly over the waves");
    const int rr = lane >> 3, pos = lane & 7;
#pragma unroll
    for (int j = 0; j < NI; ++j) {
        const int r = (j * NW + wave) * 8 + rr;
        int g = op.origin + r;
        g = g < op.ext ? g : op.ext - 1;
        const int c = pos ^ swz(r);
        load_to_lds16(op.base + (int64_t)g * op.ld + k0 + c * 8, lds + (j * NW + wave) * 8 * GEMM_BK);
    }
}

// Register-staged tile (any operand form, zero-fills k >= K) for NT threads.
template <int ROWS, int NT>
struct Staged2 {
    static constexpr int N = ROWS * 8 / NT;
    u32x4_t v[N];
};

template <typename T, int ROWS, int NT, bool MN_CONTIG>
FX_DEV void stage2_load(Staged2<ROWS, NT>& st, const OperandView<T>& op, int k0, int K, int tid) {
    constexpr int N = Staged2<ROWS, NT>::N;
    const u32x4_t zero = {0u, 0u, 0u, 0u};
    if (!MN_CONTIG) {
#pragma unroll
        for (int i = 0; i < N; ++i) {
            const int id = i * NT + tid;
            const int r = id >> 3, c = id & 7;
            int g = op.origin + r;
            g = g < op.ext ? g : op.ext - 1;
            const int k = k0 + c * 8;
            st.v[i] = k < K ? ldg16(op.base + (int64_t)g * op.ld + k) : zero;
        }
    } else {
        // blocks of 8(k) x 8(mn): ROWS blocks in all; a lane holds N k-rows of one block
        // (N == 8: a whole block, N == 4: half of one, N == 2: a quarter)
        constexpr int LPB = 8 / N;  // lanes per block
        const int id = tid / LPB, part = tid % LPB;
        const int kb = id & 7, nb = id >> 3;
        int g = op.origin + nb * 8;
        g = g + 8 <= op.ext ? g : op.ext - 8;
#pragma unroll
        for (int j = 0; j < N; ++j) {
            const int k = k0 + kb * 8 + part * N + j;
            st.v[j] = k < K ? ldg16(op.base + (int64_t)k * op.ld + g) : zero;
        }
    }
}

template <typename T, int ROWS, int NT, bool MN_CONTIG>
FX_DEV void stage2_store(const Staged2<ROWS, NT>& st, T* lds, int tid) {
    constexpr int N = Staged2<ROWS, NT>::N;
    if (!MN_CONTIG) {
#pragma unroll
        for (int i = 0; i < N; ++i) {
            const int id = i * NT + tid;
            const int r = id >> 3, c = id & 7;
            *reinterpret_cast<u32x4_t*>(lds + r * GEMM_BK + ((c ^ swz(r)) << 3)) = st.v[i];
        }
    } else {
        constexpr int LPB = 8 / N;
        const int id = tid / LPB, part = tid % LPB;
        const int kb = id & 7, nb = id >> 3;
        // v[j] = k-row (part*N + j) of the block; dword d of it holds mn = 2d (low) and 2d+1 (high).
        // Output row i (mn index) gets k = part*N .. part*N+N-1: N halves = N/2 dwords.
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int d = i >> 1;
            const unsigned sel = (i & 1) ? 0x07060302u : 0x05040100u;
            const int r = nb * 8 + i;
            T* dst = lds + r * GEMM_BK + ((kb ^ swz(r)) << 3) + part * N;
            if constexpr (N == 8) {
                u32x4_t o;
                o[0] = __builtin_amdgcn_perm(st.v[1][d], st.v[0][d], sel);
                o[1] = __builtin_amdgcn_perm(st.v[3][d], st.v[2][d], sel);
                o[2] = __builtin_amdgcn_perm(st.v[5][d], st.v[4][d], sel);
                o[3] = __builtin_amdgcn_perm(st.v[7][d], st.v[6][d], sel);
                *reinterpret_cast<u32x4_t*>(dst) = o;
            } else if constexpr (N == 4) {
                uint2 o;
                o.x = __builtin_amdgcn_perm(st.v[1][d], st.v[0][d], sel);
                o.y = __builtin_amdgcn_perm(st.v[3][d], st.v[2][d], sel);
                *reinterpret_cast<uint2*>(dst) = o;
            } else {
                *reinterpret_cast<unsigned*>(dst) = __builtin_amdgcn_perm(st.v[1][d], st.v[0][d], sel);
            }
        }
    }
}

// MFMAs of one 64-wide K-step from LDS tiles As (BM rows) and Bs (BN rows).  The fragments
// of sub-step ks+1 are read from LDS while the MFMAs of sub-step ks run; scheduling
// barriers pin that order, because left alone the scheduler sinks every read to just
// before its first use and the matrix pipe idles for the LDS latency.
template <typename T, int WM, int WN>
FX_DEV void mma_step(const T* As, const T* Bs, int row_a0, int row_b0, int lane,
                     f32x16_t (&acc)[WM / 32][WN / 32]) {
    constexpr int TM = WM / 32, TN = WN / 32;
    constexpr int KS = GEMM_BK / 16;
    typedef typename Mfma32<T>::frag frag;
    frag af[2][TM], bfv[2][TN];
    const T* pa[TM];
    const T* pb[TN];
    int sa[TM], sb[TN];
#pragma unroll
    for (int i = 0; i < TM; ++i) {
        const int r = row_a0 + i * 32 + (lane & 31);
        pa[i] = As + r * GEMM_BK;
        sa[i] = swz(r);
    }
#pragma unroll
    for (int j = 0; j < TN; ++j) {
        const int r = row_b0 + j * 32 + (lane & 31);
        pb[j] = Bs + r * GEMM_BK;
        sb[j] = swz(r);
    }
    const int half = lane >> 5;
    // read r of sub-step ks: r < TM is A fragment r, otherwise B fragment r - TM
    auto fetch_one = [&](int ks, int slot, int r) {
        const int chunk = ks * 2 + half;
        if (r < TM) af[slot][r] = *reinterpret_cast<const frag*>(pa[r] + ((chunk ^ sa[r]) << 3));
        else bfv[slot][r - TM] = *reinterpret_cast<const frag*>(pb[r - TM] + ((chunk ^ sb[r - TM]) << 3));
    };
    constexpr int READS = TM + TN, MFMAS = TM * TN;
    constexpr int EVERY = 1;   // one LDS read after each of the first READS MFMAs
#pragma unroll
    for (int r = 0; r < READS; ++r) fetch_one(0, 0, r);
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
        const int cur = ks & 1;
        int r = 0;
#pragma unroll
        for (int m = 0; m < MFMAS; ++m) {
            const int i = m / TN, j = m % TN;
            __builtin_amdgcn_sched_barrier(0);
            acc[i][j] = Mfma32<T>::run(bfv[cur][j], af[cur][i], acc[i][j]);   // transposed tile: rows = n, columns = m
            if (ks + 1 < KS && m % EVERY == 0 && r < READS) {
                __builtin_amdgcn_sched_barrier(0);
                fetch_one(ks + 1, cur ^ 1, r);   // issues in the shadow of the MFMA above
                ++r;
            }
        }
        __builtin_amdgcn_sched_barrier(0);
    }
}

// Epilogue.  The accumulators hold the transposed tile (MFMA is called with the B fragment
// first): lane l, register v of acc[i][j] is D[row0 + 32i + l%32][col0 + 32j + 8*(v/4) + 4*(l/32) + v%4],
// i.e. a lane owns groups of 4 consecutive columns.  Each wave stages one 32-row band at a time in
// its own LDS region (fp32, row pitch WN + 4 floats) and reads it back so that a lane holds 8
// consecutive elements of one row: D (and C when beta != 0) move as 16-byte (bf16/fp16) or
// 2 x 16-byte (fp32) accesses, four full 256-byte row segments per wave instruction.
// `smem` must be free (all waves past their last LDS read) and hold NW * 32 * (WN + 4) floats.
typedef float f32x4_t __attribute__((ext_vector_type(4)));

template <int NW, int WN>
constexpr size_t epilogue_lds_bytes() { return (size_t)NW * 32 * (WN + 4) * sizeof(float); }

template <typename T, typename TD, int WM, int WN>
FX_DEV void epilogue_tile(f32x16_t (&acc)[WM / 32][WN / 32], const TD* C, TD* D, int64_t ldc, int64_t ldd, int row_base,
                          int col_base, int M, int N, float alpha, float beta, T* smem, int wave, int lane) {
    constexpr int TM = WM / 32, TN = WN / 32;
    constexpr int PITCH = WN + 4;
    constexpr int GROUPS = WN / 8;              // 8-element groups per staged row
    constexpr int PER_LANE = 32 * GROUPS / 64;  // groups per lane per band
    float* stage = reinterpret_cast<float*>(smem) + wave * 32 * PITCH;
    const bool vec_ok = ((ldd & 7) == 0) && ((reinterpret_cast<uintptr_t>(D) & 15u) == 0) &&
                        (beta == 0.f || (((ldc & 7) == 0) && ((reinterpret_cast<uintptr_t>(C) & 15u) == 0)));
#pragma unroll
    for (int i = 0; i < TM; ++i) {
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const f32x4_t q = {acc[i][j][4 * g], acc[i][j][4 * g + 1], acc[i][j][4 * g + 2], acc[i][j][4 * g + 3]};
                *reinterpret_cast<f32x4_t*>(stage + (lane & 31) * PITCH + j * 32 + 8 * g + 4 * (lane >> 5)) = q;
            }
        // a wave reads back only what it wrote itself; its LDS accesses complete in order
#pragma unroll
        for (int t = 0; t < PER_LANE; ++t) {
            const int id = t * 64 + lane;
            const int rr = id / GROUPS, cg = id % GROUPS;
            const int row = row_base + i * 32 + rr, col = col_base + cg * 8;
            if (row >= M || col >= N) continue;
            const float* src = stage + rr * PITCH + cg * 8;
            const f32x4_t lo = *reinterpret_cast<const f32x4_t*>(src), hi = *reinterpret_cast<const f32x4_t*>(src + 4);
            float o[8];
#pragma unroll
            for (int e = 0; e < 4; ++e) { o[e] = alpha * lo[e]; o[4 + e] = alpha * hi[e]; }
            TD* dst = D + (int64_t)row * ldd + col;
            if (vec_ok && col + 8 <= N) {
                if (beta != 0.f) {
                    float c[8];
                    load_f32<TD, 8>(C + (int64_t)row * ldc + col, c);
#pragma unroll
                    for (int e = 0; e < 8; ++e) o[e] += beta * c[e];
                }
                store_f32<TD, 8>(dst, o);
            } else {
                for (int e = 0; e < 8 && col + e < N; ++e) {
                    float r = o[e];
                    if (beta != 0.f) r += beta * (float)C[(int64_t)row * ldc + col + e];
                    dst[e] = (TD)r;
                }
            }
        }
    }
}

// LDS bytes a workgroup needs: two buffers of (BM + BN) x 64 elements, or the epilogue staging
// of all its waves if that is larger.
template <typename T, int BM, int BN, int WAVES_M, int WAVES_N>
constexpr size_t gemm2_lds_bytes() {
    constexpr size_t tiles = (size_t)2 * (BM + BN) * GEMM_BK * sizeof(T);
    constexpr size_t epi = epilogue_lds_bytes<WAVES_M * WAVES_N, BN / WAVES_N>();
    return tiles > epi ? tiles : epi;
}

template <typename T, typename TD, int BM, int BN, int WAVES_M, int WAVES_N, bool A_MN, bool B_MN>
FX_DEV void gemm_tile2(const OperandView<T>& A, const OperandView<T>& B, const TD* C, TD* D, int64_t ldc,
                       int64_t ldd, int M, int N, int K, float alpha, float beta, T* smem) {
    constexpr int NW = WAVES_M * WAVES_N, NT = NW * 64;
    constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N;
    constexpr int TM = WM / 32, TN = WN / 32;
    constexpr int BUF = (BM + BN) * GEMM_BK;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wm = wave / WAVES_N, wn = wave % WAVES_N;

    f32x16_t acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

    const int nfull = K / GEMM_BK;  // K-steps that need no zero fill
    Staged2<BM, NT> sa;
    Staged2<BN, NT> sb;

    // Main loop over the full K-steps: K-contiguous operands go global -> LDS directly,
    // M/N-contiguous ones through registers (loaded before the MFMAs, written after them).
    auto issue = [&](int kt, T* buf) {
        if (!A_MN) tile_load_direct<T, BM, NW>(A, kt * GEMM_BK, buf, wave, lane);
        else stage2_load<T, BM, NT, true>(sa, A, kt * GEMM_BK, K, tid);
        if (!B_MN) tile_load_direct<T, BN, NW>(B, kt * GEMM_BK, buf + BM * GEMM_BK, wave, lane);
        else stage2_load<T, BN, NT, true>(sb, B, kt * GEMM_BK, K, tid);
    };
    auto commit = [&](T* buf) {
        if (A_MN) stage2_store<T, BM, NT, true>(sa, buf, tid);
        if (B_MN) stage2_store<T, BN, NT, true>(sb, buf + BM * GEMM_BK, tid);
    };
    if (nfull > 0) {
        issue(0, smem);
        commit(smem);
    }
    for (int kt = 0; kt < nfull; ++kt) {
        T* cur = smem + (kt & 1) * BUF;
        T* nxt = smem + ((kt + 1) & 1) * BUF;
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // this wave's direct loads of step kt have landed
        __syncthreads();                                  // everyone's have, and buffer `nxt` is no longer read
        if (kt + 1 < nfull) issue(kt + 1, nxt);
        mma_step<T, WM, WN>(cur, cur + BM * GEMM_BK, wm * WM, wn * WN, lane, acc);
        if (kt + 1 < nfull) commit(nxt);
    }
    if (nfull * GEMM_BK < K) {  // K tail: register path for both operands, zero-filled past K
        T* buf = smem + (nfull & 1) * BUF;
        stage2_load<T, BM, NT, A_MN>(sa, A, nfull * GEMM_BK, K, tid);
        stage2_load<T, BN, NT, B_MN>(sb, B, nfull * GEMM_BK, K, tid);
        stage2_store<T, BM, NT, A_MN>(sa, buf, tid);     // `buf` was last read two steps ago
        stage2_store<T, BN, NT, B_MN>(sb, buf + BM * GEMM_BK, tid);
        __syncthreads();
        mma_step<T, WM, WN>(buf, buf + BM * GEMM_BK, wm * WM, wn * WN, lane, acc);
    }
    __syncthreads();  // every wave is past its last LDS read: the buffers become epilogue staging
    static_assert(gemm2_lds_bytes<T, BM, BN, WAVES_M, WAVES_N>() <= 160 * 1024, "tile configuration exceeds the 160 KB of LDS");
    epilogue_tile<T, TD, WM, WN>(acc, C, D, ldc, ldd, A.origin + wm * WM, B.origin + wn * WN, M, N, alpha, beta, smem, wave, lane);
}

}  // namespace fx
