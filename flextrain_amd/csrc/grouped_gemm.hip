// Expert-grouped GEMMs for the MoE block, gfx950.
//
// The reference runs a Python loop over experts, one cuBLASLt call per GEMM, after
// copying the per-expert row counts to the host and synchronising
// (flextrain/ops/full_moe.py:144-148, :428-466, :545-626).  Here each GEMM family
// is ONE launch whose workgroups find their expert from the counts that are still
// on the device, so no host round trip is needed:
//
//   rows form   D_e[c_e, N]  = alpha * A_e[c_e, K] * op(B[e]) + beta * C_e      (up / down / dgrad)
//   wgrad form  G[e][M, N]   = alpha * A_e[c_e, M]^T * B_e[c_e, N] + beta * G[e]
//
// where rows of expert e are the contiguous range [off_e, off_e + c_e) of the
// expert-sorted buffers and off = exclusive prefix sum of the counts.
#include "gemm_core2.h"
#include "flexhip.h"

namespace fx {

// Workspace layout (int32): [0] number of tiles, [1] E and [2] tile height BM the plan was made
// for, [3 .. E+3] row offsets (E+1 entries), then (expert, first_row_in_expert) pairs, one per
// BM-row tile.  A launch that is given no counts takes the plan as it finds it: the kernels compare
// [1] and [2] with their own E and tile height and do nothing when they differ (a workspace that
// was never planned, or was planned for another shape, must not send them out of bounds), and
// never walk more tiles than the host computed as the worst case.
struct GroupedWs {
    int32_t* ntiles;
    int32_t* offsets;
    int32_t* tiles;
};

static inline GroupedWs split_ws(void* ws, int E) {
    int32_t* p = reinterpret_cast<int32_t*>(ws);
    return GroupedWs{p, p + 3, p + 4 + E};
}

// Number of (row tile, column tile) pairs to process, 0 when the plan is not for (E, BM).
FX_DEV int plan_total(const int32_t* NTILES, int E, int BM, int tiles_n, int max_tiles) {
    if (NTILES[1] != E || (BM != 0 && NTILES[2] != BM)) return 0;
    int nt = NTILES[0];
    nt = nt < 0 ? 0 : (nt > max_tiles ? max_tiles : nt);
    return nt * tiles_n;
}

__global__ __launch_bounds__(256) void grouped_plan_kernel(const int32_t* __restrict__ COUNTS, int E, int BM,
                                                           int32_t* __restrict__ NTILES,
                                                           int32_t* __restrict__ OFFSETS,
                                                           int32_t* __restrict__ TILES) {
    __shared__ int32_t wsum_r[4], wsum_t[4];
    __shared__ int32_t carry_r, carry_t;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    if (threadIdx.x == 0) { carry_r = 0; carry_t = 0; }
    __syncthreads();
    for (int base = 0; base < E; base += 256) {
        const int e = base + threadIdx.x;
        const int32_t c = e < E ? COUNTS[e] : 0;
        const int32_t nt = (c + BM - 1) / BM;
        int32_t ir = c, it = nt;
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) {
            const int32_t orr = __shfl_up(ir, off, 64);
            const int32_t ot = __shfl_up(it, off, 64);
            if (lane >= off) { ir += orr; it += ot; }
        }
        if (lane == 63) { wsum_r[wave] = ir; wsum_t[wave] = it; }
        __syncthreads();
        int32_t br = carry_r, bt = carry_t;
        for (int w = 0; w < wave; ++w) { br += wsum_r[w]; bt += wsum_t[w]; }
        if (e < E) {
            OFFSETS[e] = br + ir - c;
            const int32_t first = bt + it - nt;
            for (int32_t t = 0; t < nt; ++t) {
                TILES[2 * (first + t)] = e;
                TILES[2 * (first + t) + 1] = t * BM;
            }
        }
        __syncthreads();
        if (threadIdx.x == 255) { carry_r = br + ir; carry_t = bt + it; }
        __syncthreads();
    }
    if (threadIdx.x == 0) { OFFSETS[E] = carry_r; NTILES[0] = carry_t; NTILES[1] = E; NTILES[2] = BM; }
}

template <typename T, int BM, int BN, int WAVES_M, int WAVES_N, bool B_MN>
__global__ __launch_bounds__(WAVES_M * WAVES_N * 64) void grouped_rows_kernel(
    const T* __restrict__ A, int64_t lda, const T* __restrict__ B, int64_t ldb, int64_t b_expert_stride,
    const T* C, int64_t ldc, T* D, int64_t ldd, const int32_t* __restrict__ NTILES,
    const int32_t* __restrict__ OFFSETS, const int32_t* __restrict__ TILES, int N, int K, float alpha,
    float beta, int tiles_n, int E, int max_tiles) {
    extern __shared__ __align__(16) unsigned char smem_raw[];
    T* smem = reinterpret_cast<T*>(smem_raw);
    // The grid is sized for the worst case; the live tiles are (row tile, column tile) pairs in
    // expert-major order with the column tile fastest.  Workgroups are dealt round-robin to the 8
    // XCDs: give each XCD a contiguous band of that order, so the workgroups that share an expert's
    // weights and a row tile's activations meet in one L2.
    const int total = plan_total(NTILES, E, BM, tiles_n, max_tiles);
    const int pid = blockIdx.x;
    if (pid >= total) return;
    const int p = xcd_band(pid, total);
    const int tile = p / tiles_n, tn = p % tiles_n;
    const int e = TILES[2 * tile];
    const int m0 = TILES[2 * tile + 1];
    const int64_t row0 = OFFSETS[e];
    const int rows = OFFSETS[e + 1] - OFFSETS[e];
    OperandView<T> a{A + row0 * lda, lda, rows, m0};
    OperandView<T> b{B + (int64_t)e * b_expert_stride, ldb, N, tn * BN};
    const T* c = C ? C + row0 * ldc : nullptr;
    gemm_tile2<T, T, BM, BN, WAVES_M, WAVES_N, false, B_MN>(a, b, c, D + row0 * ldd, ldc, ldd, rows, N, K, alpha, beta, smem);
}

// The same with 32-wide K-steps, three LDS stages and two workgroups per CU (gemm_mainloop32);
// K must be a multiple of 32.
template <typename T, int BM, int BN, int WAVES_M, int WAVES_N, bool B_MN>
__global__ __launch_bounds__(WAVES_M * WAVES_N * 64, 2) void grouped_rows_kernel32(
    const T* __restrict__ A, int64_t lda, const T* __restrict__ B, int64_t ldb, int64_t b_expert_stride,
    const T* C, int64_t ldc, T* D, int64_t ldd, const int32_t* __restrict__ NTILES,
    const int32_t* __restrict__ OFFSETS, const int32_t* __restrict__ TILES, int N, int K, float alpha,
    float beta, int tiles_n, int E, int max_tiles) {
    extern __shared__ __align__(16) unsigned char smem_raw[];
    T* smem = reinterpret_cast<T*>(smem_raw);
    const int total = plan_total(NTILES, E, BM, tiles_n, max_tiles);
    const int pid = blockIdx.x;
    if (pid >= total) return;
    const int p = xcd_band(pid, total);
    const int tile = p / tiles_n, tn = p % tiles_n;
    const int e = TILES[2 * tile];
    const int m0 = TILES[2 * tile + 1];
    const int64_t row0 = OFFSETS[e];
    const int rows = OFFSETS[e + 1] - OFFSETS[e];
    OperandView<T> a{A + row0 * lda, lda, rows, m0};
    OperandView<T> b{B + (int64_t)e * b_expert_stride, ldb, N, tn * BN};
    constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    f32x16_t acc[WM / 32][WN / 32];
    gemm_mainloop32<T, BM, BN, WAVES_M, WAVES_N, false, B_MN>(a, b, K, smem, acc);
    epilogue_tile<T, T, WM, WN>(acc, C ? C + row0 * ldc : nullptr, D + row0 * ldd, ldc, ldd,
                                m0 + (wave / WAVES_N) * WM, tn * BN + (wave % WAVES_N) * WN, rows, N, alpha, beta, smem,
                                wave, lane);
}

// Up projection of every expert with the SwiGLU in the epilogue: the expert's weight holds two
// Nh-row (or Nh-column) halves b2_delta elements apart; P1 / P2 receive the two pre-activation
// halves and ACTO the gated product (see gemm_tile2_glu).
template <typename T, int BM, int BN, int WAVES_M, int WAVES_N, bool B_MN, bool K32 = false>
__global__ __launch_bounds__(WAVES_M * WAVES_N * 64, K32 ? 2 : 1) void grouped_rows_glu_kernel(
    const T* __restrict__ A, int64_t lda, const T* __restrict__ B, int64_t ldb, int64_t b_expert_stride,
    int64_t b2_delta, T* P1, T* P2, int64_t ldp, T* ACTO, int64_t ldact, const int32_t* __restrict__ NTILES,
    const int32_t* __restrict__ OFFSETS, const int32_t* __restrict__ TILES, int Nh, int K, int gate_first,
    int tiles_n, const int32_t* __restrict__ A_ROW_MAP, int a_rows, int E, int max_tiles) {
    extern __shared__ __align__(16) unsigned char smem_raw[];
    T* smem = reinterpret_cast<T*>(smem_raw);
    const int total = plan_total(NTILES, E, BM, tiles_n, max_tiles);
    const int pid = blockIdx.x;
    if (pid >= total) return;
    const int p = xcd_band(pid, total);
    const int tile = p / tiles_n, tn = p % tiles_n;
    const int e = TILES[2 * tile];
    const int m0 = TILES[2 * tile + 1];
    const int64_t row0 = OFFSETS[e];
    const int rows = OFFSETS[e + 1] - OFFSETS[e];
    // A_ROW_MAP: expert-sorted row r is row A_ROW_MAP[r] of A (the token it was routed from): the
    // rows are gathered by the tile loads themselves and no expert-sorted copy of A exists
    OperandView<T> a{A_ROW_MAP ? A : A + row0 * lda, lda, rows, m0};
    if (A_ROW_MAP) { a.row_map = A_ROW_MAP + row0; a.map_rows = a_rows; }
    const T* b1 = B + (int64_t)e * b_expert_stride;
    OperandView<T> b{b1, ldb, Nh, tn * (BN / 2), BN / WAVES_N / 2, b1 + b2_delta};
    gemm_tile2_glu<T, BM, BN, WAVES_M, WAVES_N, B_MN, ACT_SILU, K32>(a, b, P1 + row0 * ldp, P2 + row0 * ldp, ldp,
                                                                     ACTO + row0 * ldact, ldact, rows, Nh, K,
                                                                     gate_first != 0, smem);
}

// ---------------------------------------------------------------- workgroups that walk several tiles
// One workgroup per CU walks the tile list with a stride of the grid size.  Between the K loop of a
// tile and its epilogue it sets up the next tile's loaders and requests that tile's first K-step,
// so the cold start of a tile (table look-ups, first loads: 2-3 us of a 25-70 us tile) runs under
// the epilogue of the one before.  LDS plan (160 KB): [stage 0: 64 KB][32 KB][stage 1: 64 KB]; the
// epilogue stages its bands in the 96 KB behind stage 0, which only the SECOND K-step of the next
// tile overwrites, and that is issued after the barrier that follows the epilogue.
constexpr size_t kWalkLdsBytes = 160 * 1024;

template <typename T>
struct WalkLds {
    static FX_DEV T* buf0(T* smem) { return smem; }
    static FX_DEV T* epi(T* smem) { return smem + 64 * 1024 / sizeof(T); }
    static FX_DEV T* buf1(T* smem) { return smem + 96 * 1024 / sizeof(T); }
};

template <typename T, int BM, int BN, int WAVES_M, int WAVES_N, bool B_MN>
__global__ __launch_bounds__(WAVES_M * WAVES_N * 64) void grouped_rows_walk_kernel(
    const T* __restrict__ A, int64_t lda, const T* __restrict__ B, int64_t ldb, int64_t b_expert_stride,
    const T* C, int64_t ldc, T* D, int64_t ldd, const int32_t* __restrict__ NTILES,
    const int32_t* __restrict__ OFFSETS, const int32_t* __restrict__ TILES, int N, int K, float alpha,
    float beta, int tiles_n, int E, int max_tiles) {
    static_assert((BM + BN) * GEMM_BK * sizeof(T) == 64 * 1024, "the LDS plan assumes 64 KB stages");
    extern __shared__ __align__(16) unsigned char smem_raw[];
    T* smem = reinterpret_cast<T*>(smem_raw);
    constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N;
    const int total = plan_total(NTILES, E, BM, tiles_n, max_tiles);
    int pid = blockIdx.x;
    if (pid >= total) return;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    struct Tile { int m0, tn, rows, e; int64_t row0; };
    auto lookup = [&](int id) {
        const int p = xcd_band(id, total);
        const int tile = p / tiles_n;
        Tile t;
        t.tn = p % tiles_n;
        t.e = TILES[2 * tile];
        t.m0 = TILES[2 * tile + 1];
        t.row0 = OFFSETS[t.e];
        t.rows = OFFSETS[t.e + 1] - OFFSETS[t.e];
        return t;
    };
    auto view_a = [&](const Tile& t) { return OperandView<T>{A + t.row0 * lda, lda, t.rows, t.m0}; };
    auto view_b = [&](const Tile& t) { return OperandView<T>{B + (int64_t)t.e * b_expert_stride, ldb, N, t.tn * BN}; };
    MainLoop2<T, BM, BN, WAVES_M, WAVES_N, false, B_MN> loop;
    Tile cur = lookup(pid);
    OperandView<T> a = view_a(cur), b = view_b(cur);
    loop.begin(a, b, K, WalkLds<T>::buf0(smem));
    bool landed = false;     // from the second tile on, K-step 0 has landed and been published by the epilogue's wait + barrier
    for (;;) {
        const int npid = pid + (int)gridDim.x;
        const bool more = npid < total;
        Tile nxt = cur;
        if (more) nxt = lookup(npid);
        f32x16_t acc[WM / 32][WN / 32];
        loop.finish(a, b, K, WalkLds<T>::buf0(smem), WalkLds<T>::buf1(smem), acc, landed);
        const OperandView<T> a2 = view_a(nxt), b2 = view_b(nxt);
        if (more) loop.begin(a2, b2, K, WalkLds<T>::buf0(smem));
        epilogue_tile<T, T, WM, WN, true>(acc, C ? C + cur.row0 * ldc : nullptr, D + cur.row0 * ldd, ldc, ldd,
                                    cur.m0 + (wave / WAVES_N) * WM, cur.tn * BN + (wave % WAVES_N) * WN, cur.rows, N, alpha,
                                    beta, WalkLds<T>::epi(smem), wave, lane);
        if (!more) break;
        __syncthreads();     // every wave is done with its staging area before stage 1 is written again
        landed = true;
        cur = nxt;
        a = a2;
        b = b2;
        pid = npid;
    }
}

// ---------------------------------------------------------------- dgrad through w_down with the SwiGLU backward in its epilogue
// Steps (a) and (b) of the expert backward (flextrain/ops/full_moe.py:589-600) in one launch:
//   dx_act[r, f] = sum_k dy[r, k] * w_down[e][k, f]                      (rounded to T, never stored)
//   s = sigmoid(gate), silu = gate * s                                   (x_up[r] = [value (F) | gate (F)])
//   dx_up[r, f]     = dx_act * w_r * silu                                (gradient of the value half)
//   dx_up[r, F + f] = dx_act * w_r * value * (s + silu * (1 - s))        (gradient of the gate half)
//   fwd_act[r, f]   = silu * value * w_r
//   dprob[r]        = sum_f dx_act * silu * value
// computed from the ROUNDED dx_act with the element function of the separate kernel
// (moe_swiglu_bwd_elem), so dx_up and fwd_act carry the bits of the two-launch sequence.  The row
// sum crosses column tiles: each wave writes the sum over its own 64 columns to
// PART[r * part_pitch + column_tile * WAVES_N + wave_column] (8-lane tree in a fixed order) and
// dprob_reduce_kernel adds a row's slots in ascending order: no atomics, the same bits every run.
template <typename T, typename TW, int WM, int WN, bool LOADS_LAND>
FX_DEV void epilogue_swiglu_bwd(f32x16_t (&acc)[WM / 32][WN / 32], const T* __restrict__ XUP, int64_t ldx,
                                const TW* __restrict__ SRW, T* __restrict__ DXUP, int64_t lddx, T* __restrict__ ACT,
                                int64_t ldact, float* __restrict__ PART, int part_pitch, int part_slot, int row_base,
                                int col_base, int rows, int F, T* smem, int wave, int lane) {
    constexpr int TM = WM / 32, TN = WN / 32;
    constexpr int PITCH = WN + 4;
    constexpr int GROUPS = WN / 8;
    constexpr int PER_LANE = 32 * GROUPS / 64;
    static_assert(GROUPS == 8, "the row sum below reduces over the 8 lanes that share a staged row");
    typedef typename VecOf<T>::type Pack;
    static_assert(VecOf<T>::N == 8, "2-byte element types only");
    float* stage = reinterpret_cast<float*>(smem) + wave * 32 * PITCH;
    // A band's x_up packs and router weights are requested before the band is staged and used after
    // it is read back (one register set: a second one in flight spills).
    Pack px3[1][PER_LANE], px1[1][PER_LANE];
    float wrow[1][PER_LANE];
    auto request = [&](int band, int set) {
#pragma unroll
        for (int t = 0; t < PER_LANE; ++t) {
            const int id = t * 64 + lane;
            const int row = row_base + band * 32 + id / GROUPS, col = col_base + (id % GROUPS) * 8;
            if (row < rows && col < F) {
                const T* xr = XUP + (int64_t)row * ldx + col;
                px3[set][t] = *reinterpret_cast<const Pack*>(xr);
                px1[set][t] = *reinterpret_cast<const Pack*>(xr + F);
                wrow[set][t] = (float)SRW[row];
            }
        }
    };
#pragma unroll
    for (int i = 0; i < TM; ++i) {
        // lockstep: every lane of the wave has read the previous band back before this one is staged
        request(i, 0);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const f32x4_t q = {acc[i][j][4 * g], acc[i][j][4 * g + 1], acc[i][j][4 * g + 2], acc[i][j][4 * g + 3]};
                *reinterpret_cast<f32x4_t*>(stage + (lane & 31) * PITCH + j * 32 + 8 * g + 4 * (lane >> 5)) = q;
            }
        if (LOADS_LAND && i == TM - 1) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        // lockstep: a wave reads back only what it wrote itself; its LDS accesses complete in order
#pragma unroll
        for (int t = 0; t < PER_LANE; ++t) {
            const int id = t * 64 + lane;
            const int rr = id / GROUPS, cg = id % GROUPS;
            const int row = row_base + i * 32 + rr, col = col_base + cg * 8;
            float part = 0.f;
            if (row < rows && col < F) {
                const float* src = stage + rr * PITCH + cg * 8;
                const f32x4_t lo = *reinterpret_cast<const f32x4_t*>(src), hi = *reinterpret_cast<const f32x4_t*>(src + 4);
                const float w = wrow[0][t];
                float g3[8], g1[8], a[8];
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    const float d = (float)(T)(e < 4 ? lo[e] : hi[e - 4]);      // dx_act as the separate GEMM would have stored it
                    part += moe_swiglu_bwd_elem<false>((float)px3[0][t][e], (float)px1[0][t][e], d, w, 0.f, g3[e],
                                                       g1[e], a[e]);
                }
                T* dst = DXUP + (int64_t)row * lddx + col;
                store_f32<T, 8>(dst, g3);
                store_f32<T, 8>(dst + F, g1);
                if (ACT != nullptr) store_f32<T, 8>(ACT + (int64_t)row * ldact + col, a);
            }
            // the 8 lanes that share a staged row differ in their low three bits
            part += __shfl_xor(part, 1, 64);
            part += __shfl_xor(part, 2, 64);
            part += __shfl_xor(part, 4, 64);
            if (cg == 0 && row < rows) PART[(int64_t)row * part_pitch + part_slot] = part;
        }
    }
}

template <typename T, typename TW, int BM, int BN, int WAVES_M, int WAVES_N, bool B_MN>
__global__ __launch_bounds__(WAVES_M * WAVES_N * 64) void grouped_rows_swiglu_bwd_walk_kernel(
    const T* __restrict__ A, int64_t lda, const T* __restrict__ B, int64_t ldb, int64_t b_expert_stride,
    const T* __restrict__ XUP, int64_t ldx, const TW* __restrict__ SRW, T* __restrict__ DXUP, int64_t lddx,
    T* __restrict__ ACT, int64_t ldact, float* __restrict__ PART, const int32_t* __restrict__ NTILES,
    const int32_t* __restrict__ OFFSETS, const int32_t* __restrict__ TILES, int F, int K, int tiles_n, int E,
    int max_tiles, const int32_t* __restrict__ A_ROW_MAP, int a_rows) {
    static_assert((BM + BN) * GEMM_BK * sizeof(T) == 64 * 1024, "the LDS plan assumes 64 KB stages");
    extern __shared__ __align__(16) unsigned char smem_raw[];
    T* smem = reinterpret_cast<T*>(smem_raw);
    constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N;
    const int total = plan_total(NTILES, E, BM, tiles_n, max_tiles);
    int pid = blockIdx.x;
    if (pid >= total) return;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    struct Tile { int m0, tn, rows, e; int64_t row0; };
    auto lookup = [&](int id) {
        const int p = xcd_band(id, total);
        const int tile = p / tiles_n;
        Tile t;
        t.tn = p % tiles_n;
        t.e = TILES[2 * tile];
        t.m0 = TILES[2 * tile + 1];
        t.row0 = OFFSETS[t.e];
        t.rows = OFFSETS[t.e + 1] - OFFSETS[t.e];
        return t;
    };
    // A_ROW_MAP: expert-sorted row r is row A_ROW_MAP[r] of the unsorted A (gathered by the tile loads)
    auto view_a = [&](const Tile& t) {
        OperandView<T> v{A_ROW_MAP ? A : A + t.row0 * lda, lda, t.rows, t.m0};
        if (A_ROW_MAP) { v.row_map = A_ROW_MAP + t.row0; v.map_rows = a_rows; }
        return v;
    };
    auto view_b = [&](const Tile& t) { return OperandView<T>{B + (int64_t)t.e * b_expert_stride, ldb, F, t.tn * BN}; };
    MainLoop2<T, BM, BN, WAVES_M, WAVES_N, false, B_MN> loop;
    Tile cur = lookup(pid);
    OperandView<T> a = view_a(cur), b = view_b(cur);
    loop.begin(a, b, K, WalkLds<T>::buf0(smem));
    bool landed = false;
    const int part_pitch = tiles_n * WAVES_N;
    for (;;) {
        const int npid = pid + (int)gridDim.x;
        const bool more = npid < total;
        Tile nxt = cur;
        if (more) nxt = lookup(npid);
        f32x16_t acc[WM / 32][WN / 32];
        loop.finish(a, b, K, WalkLds<T>::buf0(smem), WalkLds<T>::buf1(smem), acc, landed);
        const OperandView<T> a2 = view_a(nxt), b2 = view_b(nxt);
        if (more) loop.begin(a2, b2, K, WalkLds<T>::buf0(smem));
        epilogue_swiglu_bwd<T, TW, WM, WN, true>(
            acc, XUP + cur.row0 * ldx, ldx, SRW + cur.row0, DXUP + cur.row0 * lddx, lddx,
            ACT != nullptr ? ACT + cur.row0 * ldact : nullptr, ldact, PART + cur.row0 * part_pitch, part_pitch,
            cur.tn * WAVES_N + wave % WAVES_N, cur.m0 + (wave / WAVES_N) * WM, cur.tn * BN + (wave % WAVES_N) * WN, cur.rows, F,
            WalkLds<T>::epi(smem), wave, lane);
        if (!more) break;
        __syncthreads();
        landed = true;
        cur = nxt;
        a = a2;
        b = b2;
        pid = npid;
    }
}

// dprob[r] = sum of a row's column-slot partial sums, slots ascending.
template <typename TDW>
__global__ __launch_bounds__(256) void dprob_reduce_kernel(const float* __restrict__ PART, int pitch, TDW* __restrict__ DW,
                                                           int64_t rows) {
    const int64_t r = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (r >= rows) return;
    float s = 0.f;
    for (int p = 0; p < pitch; ++p) s += PART[r * pitch + p];
    DW[r] = (TDW)s;
}

// KG: 0 = A and B are expert-sorted; 1 = A, 2 = B is the UNSORTED (src_rows, *) matrix and sorted row r
// of it is row KMAP[r] (the expert-sorted copy of that operand is then never made).
template <typename T, typename TG, int BM, int BN, int WAVES_M, int WAVES_N, int KG>
__global__ __launch_bounds__(WAVES_M * WAVES_N * 64) void grouped_wgrad_walk_kernel(
    const T* __restrict__ A, int64_t lda, const T* __restrict__ B, int64_t ldb, TG* G, int64_t ldg,
    int64_t g_expert_stride, const int32_t* __restrict__ NTILES, const int32_t* __restrict__ OFFSETS, int M, int N,
    float alpha, float beta, int tiles_n, int tiles_per_expert, int total, int E, const int32_t* __restrict__ KMAP,
    int src_rows) {
    static_assert((BM + BN) * GEMM_BK * sizeof(T) == 64 * 1024, "the LDS plan assumes 64 KB stages");
    extern __shared__ __align__(16) unsigned char smem_raw[];
    T* smem = reinterpret_cast<T*>(smem_raw);
    constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N;
    int pid = blockIdx.x;
    if (pid >= total || NTILES[1] != E) return;      // only the row offsets of the plan are used: any tile height serves
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    struct Tile { int e, tm, tn, rows; int64_t row0; };
    auto lookup = [&](int id) {
        const int p = xcd_band(id, total);
        Tile t;
        t.e = p / tiles_per_expert;
        const int q = p % tiles_per_expert;
        if (KG == 2) {          // consecutive tiles share the gathered operand's tile (20 us of 680 at 128 experts x 512 rows)
            const int tiles_m = tiles_per_expert / tiles_n;
            t.tn = q / tiles_m;
            t.tm = q % tiles_m;
        } else {
            t.tm = q / tiles_n;
            t.tn = q % tiles_n;
        }
        t.row0 = OFFSETS[t.e];
        t.rows = OFFSETS[t.e + 1] - OFFSETS[t.e];
        return t;
    };
    auto view_a = [&](const Tile& t) {
        OperandView<T> v{KG == 1 ? A : A + t.row0 * lda, lda, M, t.tm * BM};
        if (KG == 1) { v.k_map = KMAP + t.row0; v.k_ext = t.rows; v.map_rows = src_rows; }
        return v;
    };
    auto view_b = [&](const Tile& t) {
        OperandView<T> v{KG == 2 ? B : B + t.row0 * ldb, ldb, N, t.tn * BN};
        if (KG == 2) { v.k_map = KMAP + t.row0; v.k_ext = t.rows; v.map_rows = src_rows; }
        return v;
    };
    MainLoop2<T, BM, BN, WAVES_M, WAVES_N, true, true, false, true, KG == 1, KG == 2> loop;
    Tile cur = lookup(pid);
    OperandView<T> a = view_a(cur), b = view_b(cur);
    loop.begin(a, b, cur.rows, WalkLds<T>::buf0(smem));
    bool landed = false;
    for (;;) {
        const int npid = pid + (int)gridDim.x;
        const bool more = npid < total;
        Tile nxt = cur;
        if (more) nxt = lookup(npid);
        f32x16_t acc[WM / 32][WN / 32];
        loop.finish(a, b, cur.rows, WalkLds<T>::buf0(smem), WalkLds<T>::buf1(smem), acc, landed);
        const OperandView<T> a2 = view_a(nxt), b2 = view_b(nxt);
        if (more) loop.begin(a2, b2, nxt.rows, WalkLds<T>::buf0(smem));
        if (!(cur.rows == 0 && beta == 1.f)) {   // an expert without rows adds nothing
            TG* g = G + (int64_t)cur.e * g_expert_stride;
            epilogue_tile<T, TG, WM, WN, true>(acc, g, g, ldg, ldg, cur.tm * BM + (wave / WAVES_N) * WM,
                                               cur.tn * BN + (wave % WAVES_N) * WN, M, N, alpha, beta, WalkLds<T>::epi(smem), wave, lane);
        } else {
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // the wait the skipped epilogue would have made
        }
        if (!more) break;
        __syncthreads();
        landed = true;
        cur = nxt;
        a = a2;
        b = b2;
        pid = npid;
    }
}

static inline int cdiv_i(int64_t a, int b) { return (int)((a + b - 1) / b); }

}  // namespace fx

using namespace fx;

// Workgroups of the walking kernels: one per CU of the current device.
static int walk_grid() {
    static int cus[64] = {};
    int dev = 0;
    (void)hipGetDevice(&dev);
    if (dev < 0 || dev >= 64) return 256;
    if (cus[dev] == 0) {
        int n = 0;
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
        cus[dev] = (n / 8) * 8 > 0 ? (n / 8) * 8 : n;      // a multiple of the 8 XCDs keeps a workgroup's tiles on one XCD
    }
    return cus[dev];
}

extern "C" size_t fx_grouped_ws_bytes(int E, int64_t total_rows) {
    if (E <= 0 || total_rows < 0) return 0;
    // smallest row tile is 128: at most total_rows/128 + E tiles
    return sizeof(int32_t) * (size_t)(4 + E + 2 * (total_rows / 128 + E + 1));
}

// Row tile: 256 x 256 (one workgroup per CU, 64-wide K-steps) when experts average 384 rows or
// more, although up to a quarter of such tiles is padding then: at 512 rows per expert it is 10-16 %
// faster than 128-row tiles (up-projection 0.53 -> 0.475 ms on routed counts, 0.575 -> 0.48 ms on
// uniform ones).  Below that, 128-row tiles in a form that lets two workgroups share a CU, so one's
// epilogue overlaps the other's K loop: 128 x 256 with 32-wide K-steps (K a multiple of 32), else
// 128 x 128 with 64-wide ones.
static int rows_bm(int64_t total_rows, int E) { return (total_rows / (E > 0 ? E : 1)) >= 384 ? 256 : 128; }

extern "C" int fx_grouped_plan(const int32_t* counts, int E, int64_t total_rows, void* ws, size_t ws_bytes,
                               hipStream_t stream) {
    if (E <= 0 || total_rows < 0) FX_FAIL("fx_grouped_plan: bad shape");
    if (!counts || !ws || ws_bytes < fx_grouped_ws_bytes(E, total_rows)) FX_FAIL("fx_grouped_plan: null pointer or workspace too small");
    GroupedWs w = split_ws(ws, E);
    grouped_plan_kernel<<<1, 256, 0, stream>>>(counts, E, rows_bm(total_rows, E), w.ntiles, w.offsets, w.tiles);
    FX_CHECK_LAUNCH("fx_grouped_plan");
    return 0;
}

extern "C" int fx_grouped_gemm_rows(const void* A, int64_t lda, const void* B, int64_t ldb,
                                    int64_t b_expert_stride, int trans_b, const void* C, int64_t ldc, void* D,
                                    int64_t ldd, const int32_t* counts, int E, int64_t total_rows, int N, int K,
                                    float alpha, float beta, int dt, void* ws, size_t ws_bytes,
                                    hipStream_t stream) {
    if (E <= 0 || total_rows < 0 || N <= 0 || K <= 0) FX_FAIL("fx_grouped_gemm_rows: bad shape");
    if (total_rows == 0) return 0;
    if (!A || !B || !D) FX_FAIL("fx_grouped_gemm_rows: null pointer");
    if (!ws || ws_bytes < fx_grouped_ws_bytes(E, total_rows)) FX_FAIL("fx_grouped_gemm_rows: workspace too small");
    if (dt != DT_BF16 && dt != DT_F16) FX_FAIL("fx_grouped_gemm_rows: bf16 or fp16 only");
    if (lda >= (1 << 23) || ldb >= (1 << 23)) FX_FAIL("fx_grouped_gemm_rows: leading dimensions must be below 2^23 elements");
    if (!aligned16(A) || !aligned16(B) || !aligned16(D) || (lda & 7) || (ldb & 7) || (K & 7) || (b_expert_stride & 7) ||
        (!trans_b && (N & 7)))
        FX_FAIL("fx_grouped_gemm_rows: operands must be 16-byte aligned with K (and N when B is (K,N)) a multiple of 8");
    if (!C || beta == 0.f) { C = nullptr; beta = 0.f; }
    GroupedWs w = split_ws(ws, E);
    const int BM = rows_bm(total_rows, E);
    if (counts) {    // no counts: the workspace already holds the plan fx_grouped_plan made for them
        grouped_plan_kernel<<<1, 256, 0, stream>>>(counts, E, BM, w.ntiles, w.offsets, w.tiles);
        FX_CHECK_LAUNCH("fx_grouped_gemm_rows(plan)");
    }
    const unsigned max_tiles = (unsigned)(total_rows / BM + E);
#define FX_ROWS(TT, BM_, BN_, WM_, WN_, BMN)                                                              \
    {                                                                                                     \
        auto kern = grouped_rows_kernel<TT, BM_, BN_, WM_, WN_, BMN>;                                     \
        constexpr size_t lds = gemm2_lds_bytes<TT, BM_, BN_, WM_, WN_>();                                 \
        FX_ENSURE_DYNAMIC_LDS(kern, lds);                                                                 \
        const int tiles_n = cdiv_i(N, BN_);                                                               \
        kern<<<dim3(max_tiles * (unsigned)tiles_n), WM_ * WN_ * 64, lds, stream>>>(                       \
            reinterpret_cast<const TT*>(A), lda, reinterpret_cast<const TT*>(B), ldb, b_expert_stride,    \
            reinterpret_cast<const TT*>(C), ldc, reinterpret_cast<TT*>(D), ldd, w.ntiles, w.offsets,      \
            w.tiles, N, K, alpha, beta, tiles_n, E, (int)max_tiles);                                      \
    }
#define FX_ROWS32(TT, BMN)                                                                               \
    {                                                                                                     \
        auto kern = grouped_rows_kernel32<TT, 128, 256, 2, 2, BMN>;                                       \
        constexpr size_t lds = gemm32_lds_bytes<TT, 128, 256, 2, 2>();                                    \
        FX_ENSURE_DYNAMIC_LDS(kern, lds);                                                                 \
        const int tiles_n = cdiv_i(N, 256);                                                               \
        kern<<<dim3(max_tiles * (unsigned)tiles_n), 256, lds, stream>>>(                                  \
            reinterpret_cast<const TT*>(A), lda, reinterpret_cast<const TT*>(B), ldb, b_expert_stride,    \
            reinterpret_cast<const TT*>(C), ldc, reinterpret_cast<TT*>(D), ldd, w.ntiles, w.offsets,      \
            w.tiles, N, K, alpha, beta, tiles_n, E, (int)max_tiles);                                      \
    }
    if (BM == 128 && (K & 31) == 0) {   // small experts: 128 x 256 tiles, 32-wide K-steps, two workgroups per CU
        if (dt == DT_BF16) { if (trans_b) FX_ROWS32(bf16, false) else FX_ROWS32(bf16, true) }
        else { if (trans_b) FX_ROWS32(f16, false) else FX_ROWS32(f16, true) }
        FX_CHECK_LAUNCH("fx_grouped_gemm_rows");
        return 0;
    }
#define FX_ROWS_WALK(TT, BMN)                                                                             \
    {                                                                                                     \
        auto kern = grouped_rows_walk_kernel<TT, 256, 256, 2, 4, BMN>;                                    \
        FX_ENSURE_DYNAMIC_LDS(kern, kWalkLdsBytes);                                                       \
        const int tiles_n = cdiv_i(N, 256);                                                               \
        const unsigned most = max_tiles * (unsigned)tiles_n;                                              \
        const unsigned grid = most < (unsigned)walk_grid() ? most : (unsigned)walk_grid();                \
        kern<<<dim3(grid), 512, kWalkLdsBytes, stream>>>(                                                 \
            reinterpret_cast<const TT*>(A), lda, reinterpret_cast<const TT*>(B), ldb, b_expert_stride,    \
            reinterpret_cast<const TT*>(C), ldc, reinterpret_cast<TT*>(D), ldd, w.ntiles, w.offsets,      \
            w.tiles, N, K, alpha, beta, tiles_n, E, (int)max_tiles);                                      \
    }
#define FX_ROWS_T(TT)                                                                                     \
    if (BM == 256) { if (trans_b) FX_ROWS_WALK(TT, false) else FX_ROWS_WALK(TT, true) }                   \
    else { if (trans_b) FX_ROWS(TT, 128, 128, 2, 2, false) else FX_ROWS(TT, 128, 128, 2, 2, true) }
    if (dt == DT_BF16) { FX_ROWS_T(bf16) } else { FX_ROWS_T(f16) }
#undef FX_ROWS_T
#undef FX_ROWS
    FX_CHECK_LAUNCH("fx_grouped_gemm_rows");
    return 0;
}

extern "C" int fx_grouped_gemm_rows_glu(const void* A, int64_t lda, const void* B, int64_t ldb, int64_t b_expert_stride,
                                        int trans_b, int64_t b2_delta, void* P1, void* P2, int64_t ldp, void* act,
                                        int64_t ldact, const int32_t* counts, int E, int64_t total_rows, int Nh, int K,
                                        int gate_first, int dt, void* ws, size_t ws_bytes, const int32_t* a_row_map,
                                        int64_t a_rows, hipStream_t stream) {
    if (E <= 0 || total_rows < 0 || Nh <= 0 || K <= 0) FX_FAIL("fx_grouped_gemm_rows_glu: bad shape");
    if (total_rows == 0) return 0;
    if (!A || !B || !P1 || !P2 || !act) FX_FAIL("fx_grouped_gemm_rows_glu: null pointer");
    if (!ws || ws_bytes < fx_grouped_ws_bytes(E, total_rows)) FX_FAIL("fx_grouped_gemm_rows_glu: workspace too small");
    if (dt != DT_BF16 && dt != DT_F16) FX_FAIL("fx_grouped_gemm_rows_glu: bf16 or fp16 only");
    if (lda >= (1 << 23) || ldb >= (1 << 23)) FX_FAIL("fx_grouped_gemm_rows_glu: leading dimensions must be below 2^23 elements");
    if (!aligned16(A) || !aligned16(B) || !aligned16(P1) || !aligned16(P2) || !aligned16(act) || (lda & 7) || (ldb & 7) ||
        (ldp & 7) || (ldact & 7) || (K & 63) || (Nh & 7) || (b_expert_stride & 7) || (b2_delta & 7))
        FX_FAIL("fx_grouped_gemm_rows_glu: needs K %% 64 == 0, N %% 8 == 0, strides %% 8 == 0 and 16-byte aligned operands");
    if (a_row_map && (a_rows <= 0 || a_rows > 0x7fffffff || (uint64_t)a_rows * (uint64_t)lda * 2u >= (1ull << 32)))
        FX_FAIL("fx_grouped_gemm_rows_glu: a gathered A must have a_rows > 0 and stay below 4 GB");
    GroupedWs w = split_ws(ws, E);
    const int BM = rows_bm(total_rows, E);
    if (counts) {
        grouped_plan_kernel<<<1, 256, 0, stream>>>(counts, E, BM, w.ntiles, w.offsets, w.tiles);
        FX_CHECK_LAUNCH("fx_grouped_gemm_rows_glu(plan)");
    }
    const unsigned max_tiles = (unsigned)(total_rows / BM + E);
#define FX_GLU(TT, BM_, BN_, WM_, WN_, BMN, K32_)                                                         \
    {                                                                                                     \
        auto kern = grouped_rows_glu_kernel<TT, BM_, BN_, WM_, WN_, BMN, K32_>;                           \
        constexpr size_t lds = gemm2_glu_lds_bytes<TT, BM_, BN_, WM_, WN_, K32_>();                       \
        FX_ENSURE_DYNAMIC_LDS(kern, lds);                                                                 \
        const int tiles_n = cdiv_i(Nh, BN_ / 2);                                                          \
        kern<<<dim3(max_tiles * (unsigned)tiles_n), WM_ * WN_ * 64, lds, stream>>>(                       \
            reinterpret_cast<const TT*>(A), lda, reinterpret_cast<const TT*>(B), ldb, b_expert_stride,    \
            b2_delta, reinterpret_cast<TT*>(P1), reinterpret_cast<TT*>(P2), ldp, reinterpret_cast<TT*>(act), \
            ldact, w.ntiles, w.offsets, w.tiles, Nh, K, gate_first, tiles_n, a_row_map, (int)a_rows, E,   \
            (int)max_tiles);                                                                              \
    }
    // 128-row tiles: 128 x 256 (128 columns of each half) with 32-wide K-steps, two workgroups per CU
#define FX_GLU_T(TT)                                                                                      \
    if (BM == 256) { if (trans_b) FX_GLU(TT, 256, 256, 4, 2, false, false) else FX_GLU(TT, 256, 256, 4, 2, true, false) } \
    else { if (trans_b) FX_GLU(TT, 128, 256, 2, 2, false, true) else FX_GLU(TT, 128, 256, 2, 2, true, true) }
    if (dt == DT_BF16) { FX_GLU_T(bf16) } else { FX_GLU_T(f16) }
#undef FX_GLU_T
#undef FX_GLU
    FX_CHECK_LAUNCH("fx_grouped_gemm_rows_glu");
    return 0;
}

extern "C" int fx_grouped_gemm_wgrad(const void* A, int64_t lda, const void* B, int64_t ldb, void* G, int64_t ldg,
                                     int64_t g_expert_stride, int g_dt, const int32_t* counts, int E,
                                     int64_t total_rows, int M, int N, float alpha, float beta, int dt, void* ws,
                                     size_t ws_bytes, const int32_t* a_row_map, int64_t a_rows,
                                     const int32_t* b_row_map, int64_t b_rows, hipStream_t stream) {
    if (E <= 0 || total_rows < 0 || M <= 0 || N <= 0) FX_FAIL("fx_grouped_gemm_wgrad: bad shape");
    if (!A || !B || !G) FX_FAIL("fx_grouped_gemm_wgrad: null pointer");
    if (!ws || ws_bytes < fx_grouped_ws_bytes(E, total_rows)) FX_FAIL("fx_grouped_gemm_wgrad: workspace too small");
    if (dt != DT_BF16 && dt != DT_F16) FX_FAIL("fx_grouped_gemm_wgrad: bf16 or fp16 only");
    if (lda >= (1 << 23) || ldb >= (1 << 23)) FX_FAIL("fx_grouped_gemm_wgrad: leading dimensions must be below 2^23 elements");
    if (g_dt != dt && !(dt == DT_BF16 && g_dt == DT_F32)) FX_FAIL("fx_grouped_gemm_wgrad: G must match the inputs or be fp32 (bf16 inputs)");
    if (!aligned16(A) || !aligned16(B) || (lda & 7) || (ldb & 7) || (M & 7) || (N & 7))
        FX_FAIL("fx_grouped_gemm_wgrad: operands must be 16-byte aligned with M and N multiples of 8");
    if (a_row_map && b_row_map) FX_FAIL("fx_grouped_gemm_wgrad: at most one operand may be gathered through a row map");
    if (a_row_map && (a_rows <= 0 || a_rows > 0x7fffffff || (uint64_t)a_rows * (uint64_t)lda * 2u >= (1ull << 32)))
        FX_FAIL("fx_grouped_gemm_wgrad: a gathered A must have a_rows > 0 and stay below 4 GB");
    if (b_row_map && (b_rows <= 0 || b_rows > 0x7fffffff || (uint64_t)b_rows * (uint64_t)ldb * 2u >= (1ull << 32)))
        FX_FAIL("fx_grouped_gemm_wgrad: a gathered B must have b_rows > 0 and stay below 4 GB");
    if (total_rows == 0 && (a_row_map || b_row_map)) { a_row_map = nullptr; b_row_map = nullptr; }
    GroupedWs w = split_ws(ws, E);
    if (counts) {    // only the row offsets are used here; the plan is the one every entry point writes for this shape
        grouped_plan_kernel<<<1, 256, 0, stream>>>(counts, E, rows_bm(total_rows, E), w.ntiles, w.offsets, w.tiles);
        FX_CHECK_LAUNCH("fx_grouped_gemm_wgrad(plan)");
    }
    constexpr int BM = 256, BN = 256;
    const int tiles_m = cdiv_i(M, BM), tiles_n = cdiv_i(N, BN);
    const dim3 grid((unsigned)(tiles_m * tiles_n) * (unsigned)E);
    const unsigned grid_w = grid.x < (unsigned)walk_grid() ? grid.x : (unsigned)walk_grid();
    const int32_t* kmap = a_row_map ? a_row_map : b_row_map;
    const int src_rows = (int)(a_row_map ? a_rows : (b_row_map ? b_rows : 0));
#define FX_WG_LAUNCH(TT, TG, KG_)                                                                         \
    {                                                                                                     \
        auto kern = grouped_wgrad_walk_kernel<TT, TG, BM, BN, 2, 4, KG_>;                                 \
        FX_ENSURE_DYNAMIC_LDS(kern, kWalkLdsBytes);                                                       \
        kern<<<dim3(grid_w), 2 * 4 * 64, kWalkLdsBytes, stream>>>(                                        \
            reinterpret_cast<const TT*>(A), lda, reinterpret_cast<const TT*>(B), ldb, reinterpret_cast<TG*>(G), ldg, \
            g_expert_stride, w.ntiles, w.offsets, M, N, alpha, beta, tiles_n, tiles_m * tiles_n,          \
            (int)grid.x, E, kmap, src_rows);                                                              \
    }
#define FX_WG_WALK(TT, TG)                                                                                \
    {                                                                                                     \
        if (a_row_map) FX_WG_LAUNCH(TT, TG, 1)                                                            \
        else if (b_row_map) FX_WG_LAUNCH(TT, TG, 2)                                                       \
        else FX_WG_LAUNCH(TT, TG, 0)                                                                      \
    }
    if (dt == DT_BF16 && g_dt == DT_BF16) FX_WG_WALK(bf16, bf16)
    else if (dt == DT_BF16) FX_WG_WALK(bf16, float)
    else FX_WG_WALK(f16, f16)
#undef FX_WG_WALK
#undef FX_WG_LAUNCH
    FX_CHECK_LAUNCH("fx_grouped_gemm_wgrad");
    return 0;
}

extern "C" int fx_grouped_rows_tile_height(int E, int64_t total_rows) { return rows_bm(total_rows, E); }

extern "C" size_t fx_grouped_swiglu_bwd_ws_bytes(int64_t total_rows, int F) {
    if (total_rows < 0 || F <= 0) return 0;
    return sizeof(float) * (size_t)total_rows * (size_t)(cdiv_i(F, 256) * 4);
}

extern "C" int fx_grouped_gemm_rows_swiglu_bwd(const void* dy, int64_t lddy, const void* w_down, int64_t ldb,
                                               int64_t b_expert_stride, int trans_b, const void* x_up, int64_t ldx,
                                               const void* srw, int srw_dt, void* dx_up, int64_t lddx, void* fwd_act,
                                               int64_t ldact, void* dprob, int dprob_dt, const int32_t* counts, int E,
                                               int64_t total_rows, int F, int K, int dt, void* ws, size_t ws_bytes,
                                               void* part_ws, size_t part_ws_bytes, const int32_t* dy_row_map,
                                               int64_t dy_rows, hipStream_t stream) {
    if (E <= 0 || total_rows < 0 || F <= 0 || K <= 0) FX_FAIL("fx_grouped_gemm_rows_swiglu_bwd: bad shape");
    if (total_rows == 0) return 0;
    if (!dy || !w_down || !x_up || !srw || !dx_up || !dprob) FX_FAIL("fx_grouped_gemm_rows_swiglu_bwd: null pointer");
    if (!ws || ws_bytes < fx_grouped_ws_bytes(E, total_rows)) FX_FAIL("fx_grouped_gemm_rows_swiglu_bwd: workspace too small");
    if (!part_ws || part_ws_bytes < fx_grouped_swiglu_bwd_ws_bytes(total_rows, F) || !aligned16(part_ws))
        FX_FAIL("fx_grouped_gemm_rows_swiglu_bwd: partial-sum workspace missing, misaligned or too small");
    if (dt != DT_BF16 && dt != DT_F16) FX_FAIL("fx_grouped_gemm_rows_swiglu_bwd: bf16 or fp16 only");
    if (srw_dt != dt && srw_dt != DT_F32) FX_FAIL("fx_grouped_gemm_rows_swiglu_bwd: router weights must have the activations' dtype or be fp32");
    if (dprob_dt != dt && dprob_dt != DT_F32) FX_FAIL("fx_grouped_gemm_rows_swiglu_bwd: dprob must have the activations' dtype or be fp32");
    if (rows_bm(total_rows, E) != 256) FX_FAIL("fx_grouped_gemm_rows_swiglu_bwd: needs 256-row tiles (at least 384 rows per expert on average); run the GEMM and fx_swiglu_moe_bwd separately");
    if (lddy >= (1 << 23) || ldb >= (1 << 23)) FX_FAIL("fx_grouped_gemm_rows_swiglu_bwd: leading dimensions must be below 2^23 elements");
    if (!aligned16(dy) || !aligned16(w_down) || !aligned16(x_up) || !aligned16(dx_up) || (fwd_act && !aligned16(fwd_act)) ||
        (lddy & 7) || (ldb & 7) || (ldx & 7) || (lddx & 7) || (fwd_act && (ldact & 7)) || (K & 7) || (F & 7) ||
        (b_expert_stride & 7))
        FX_FAIL("fx_grouped_gemm_rows_swiglu_bwd: operands must be 16-byte aligned with K, F and every row stride a multiple of 8");
    if (dy_row_map && (dy_rows <= 0 || dy_rows > 0x7fffffff || (uint64_t)dy_rows * (uint64_t)lddy * 2u >= (1ull << 32)))
        FX_FAIL("fx_grouped_gemm_rows_swiglu_bwd: a gathered dy must have dy_rows > 0 and stay below 4 GB");
    if (ldx < 2 * (int64_t)F || lddx < 2 * (int64_t)F || (fwd_act && ldact < F)) FX_FAIL("fx_grouped_gemm_rows_swiglu_bwd: x_up / dx_up rows hold 2 F elements, fwd_act rows F");
    GroupedWs w = split_ws(ws, E);
    constexpr int BM = 256;
    if (counts) {
        grouped_plan_kernel<<<1, 256, 0, stream>>>(counts, E, BM, w.ntiles, w.offsets, w.tiles);
        FX_CHECK_LAUNCH("fx_grouped_gemm_rows_swiglu_bwd(plan)");
    }
    const unsigned max_tiles = (unsigned)(total_rows / BM + E);
    const int tiles_n = cdiv_i(F, 256);
    const unsigned most = max_tiles * (unsigned)tiles_n;
    const unsigned grid = most < (unsigned)walk_grid() ? most : (unsigned)walk_grid();
#define FX_SWB(TT, TW, BMN)                                                                               \
    {                                                                                                     \
        auto kern = grouped_rows_swiglu_bwd_walk_kernel<TT, TW, 256, 256, 2, 4, BMN>;                     \
        FX_ENSURE_DYNAMIC_LDS(kern, kWalkLdsBytes);                                                       \
        kern<<<dim3(grid), 512, kWalkLdsBytes, stream>>>(                                                 \
            reinterpret_cast<const TT*>(dy), lddy, reinterpret_cast<const TT*>(w_down), ldb, b_expert_stride, \
            reinterpret_cast<const TT*>(x_up), ldx, reinterpret_cast<const TW*>(srw), reinterpret_cast<TT*>(dx_up), \
            lddx, reinterpret_cast<TT*>(fwd_act), ldact, reinterpret_cast<float*>(part_ws), w.ntiles, w.offsets, \
            w.tiles, F, K, tiles_n, E, (int)max_tiles, dy_row_map, (int)dy_rows);                         \
    }
#define FX_SWB_T(TT)                                                                                      \
    if (srw_dt == DT_F32) { if (trans_b) FX_SWB(TT, float, false) else FX_SWB(TT, float, true) }          \
    else { if (trans_b) FX_SWB(TT, TT, false) else FX_SWB(TT, TT, true) }
    if (dt == DT_BF16) { FX_SWB_T(bf16) } else { FX_SWB_T(f16) }
#undef FX_SWB_T
#undef FX_SWB
    FX_CHECK_LAUNCH("fx_grouped_gemm_rows_swiglu_bwd");
    const unsigned rgrid = (unsigned)((total_rows + 255) / 256);
    const int pitch = tiles_n * 4;
    if (dprob_dt == DT_F32) dprob_reduce_kernel<float><<<rgrid, 256, 0, stream>>>(reinterpret_cast<const float*>(part_ws), pitch, reinterpret_cast<float*>(dprob), total_rows);
    else if (dt == DT_BF16) dprob_reduce_kernel<bf16><<<rgrid, 256, 0, stream>>>(reinterpret_cast<const float*>(part_ws), pitch, reinterpret_cast<bf16*>(dprob), total_rows);
    else dprob_reduce_kernel<f16><<<rgrid, 256, 0, stream>>>(reinterpret_cast<const float*>(part_ws), pitch, reinterpret_cast<f16*>(dprob), total_rows);
    FX_CHECK_LAUNCH("fx_grouped_gemm_rows_swiglu_bwd(reduce)");
    return 0;
}
