// bf16 / fp16 MFMA GEMM building block for gfx950, second generation.
//
//   D[M,N] = alpha * op(A)[M,K] * op(B)[K,N] + beta * C[M,N]       (fp32 accumulate)
//
// A workgroup of WAVES_M x WAVES_N waves owns a BM x BN tile of D and walks K in steps of
// 64.  Each wave owns a (BM/WAVES_M) x (BN/WAVES_N) sub-tile built from
// v_mfma_f32_32x32x16.  Two LDS buffers alternate, so a K-step needs one barrier: while the
// matrix pipe works on buffer t, the loads of step t+1 fill buffer t+1.  Both operand forms go
// from global memory straight into LDS with global_load_lds_dwordx4 (16 bytes per lane, no
// registers in between); a wave instruction fills 1024 contiguous LDS bytes, so the swizzle is
// applied to the global address (a lane fetches the chunk that belongs at its fixed LDS place).
//   K-contiguous in memory (A not transposed, B transposed): LDS row r (an m or n index) holds
//     its 64 k-values as eight 16-byte chunks, chunk c at position c ^ ((r >> 1) & 7); fragments
//     are read with ds_read_b128.  The LDS has 64 banks and serves 16 lanes of a b128 read per
//     cycle: with this swizzle 16 consecutive rows hit 64 distinct banks.
//   M/N-contiguous in memory (A transposed, B not transposed): LDS row k holds the tile's m (or
//     n) values, 16-byte chunk c at position c ^ ((k & 3) << 2); fragments are read with
//     ds_read_b64_tr_b16, which hands lane i of a 16-lane group the i-th element of four rows
//     (source lanes 4j .. 4j+3 give the address of row j): two reads make the 8 consecutive
//     k-values of one m that the MFMA wants, without any transposition in registers.
// Rows / columns outside the matrix are clamped to the last valid ones (their products are
// never stored); a K tail shorter than 64 goes through registers, which zero-fills.
#pragma once
#include <type_traits>

#include "gemm_core.h"

namespace fx {

// Swizzle: chunk c of row r sits at position c ^ swz(r).
FX_DEV int swz(int r) { return (r >> 1) & 7; }


// 16 bytes per lane, global -> LDS; lds_base is wave-uniform, lane l lands at lds_base + 16*l.
// Written as inline assembly on purpose.  With the compiler's builtin for this load, its wait-count
// pass knows that LDS writes are in flight and puts `s_waitcnt vmcnt(0)` in front of every
// ds_read_b64_tr_b16 that follows (it cannot tell that the reads touch the other buffer), which
// exposes the whole global-load latency in every K-step of the transposed-read forms.  The loops
// here wait for these loads themselves (`s_waitcnt vmcnt(n)` before the barrier that publishes a
// buffer), so nothing else may depend on the compiler knowing about them.
//   - the low half of a generic pointer into LDS is the LDS address;
//   - an SALU write of M0 needs one wait state before an LDS-DMA instruction reads it.
FX_DEV void load_to_lds16(const void* gptr, void* lds_base) {
    const unsigned lds_addr = __builtin_amdgcn_readfirstlane((unsigned)(uintptr_t)lds_base);
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" ::"s"(lds_addr), "v"(gptr) : "memory", "m0");
}

// LDS layout of a 64(k) x ROWS M/N-contiguous tile: row k holds ROWS elements, its 16-byte chunk c
// at position c ^ ((k & 3) << 2).
FX_DEV int swz_tr(int k) { return (k & 3) << 2; }

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
            // gathered rows: the tail reads the same (clamped) source rows as the direct loads of the full steps
            const int64_t row = op.row_map != nullptr ? (int64_t)min(max(op.row_map[g], 0), op.map_rows - 1) : (int64_t)g;
            st.v[i] = k < K ? ldg16(op.base + row * op.ld + k) : zero;
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
            if (k < K) {
                const int64_t row = op.k_map != nullptr ? (int64_t)min(max(op.k_map[k], 0), op.map_rows - 1) : (int64_t)k;
                st.v[j] = ldg16(op.base + row * op.ld + g);
            } else {
                st.v[j] = zero;
            }
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

// MFMAs of one 64-wide K-step from LDS tiles As (BM rows or, when A_TR, 64 k-rows of BM) and Bs.
// The fragments of sub-step ks+1 are read from LDS while the MFMAs of sub-step ks run;
// scheduling barriers pin that order, because left alone the scheduler sinks every read to just
// before its first use and the matrix pipe idles for the LDS latency.
template <typename T, int BM, int BN, int WM, int WN, bool A_TR, bool B_TR>
FX_DEV void mma_step(const T* As, const T* Bs, int row_a0, int row_b0, int lane,
                     f32x16_t (&acc)[WM / 32][WN / 32]) {
    constexpr int TM = WM / 32, TN = WN / 32;
    constexpr int KS = GEMM_BK / 16;
    typedef typename Mfma32<T>::frag frag;
    typedef short s16x4_t __attribute__((ext_vector_type(4)));
    typedef __attribute__((address_space(3))) s16x4_t* lds_s16x4_ptr;
    frag af[2][TM], bfv[2][TN];
    // K-contiguous operand: lane reads row (lane & 31), chunk 2*ks + lane/32.
    // Transposed-read operand: lane s of 16-lane group g gives the address of row k = 16*ks + 8*(g/2) + s/4
    // (+4 for the second read), elements 32*i + 16*(g%2) + 4*(s%4) .. +3.
    const int half = lane >> 5;
    const int grp = lane >> 4, sl = lane & 15;
    auto read_k = [&](const T* base, int row0, int ks) {
        const int r = row0 + (lane & 31);
        return *reinterpret_cast<const frag*>(base + r * GEMM_BK + (((ks * 2 + half) ^ swz(r)) << 3));
    };
    auto read_tr = [&](const T* base, int pitch, int col0, int ks) {
        const int n = col0 + 16 * (grp & 1) + 4 * (sl & 3);
        const int k = 16 * ks + 8 * (grp >> 1) + (sl >> 2);       // k & 3 is the same for k and k + 4
        const int off = (((n >> 3) ^ (swz_tr(k) % (pitch / 8))) << 3) + (n & 7);
        const s16x4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)(base + k * pitch + off));
        const s16x4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)(base + (k + 4) * pitch + off));
        typedef short s16x8_t __attribute__((ext_vector_type(8)));
        const s16x8_t both = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
        return __builtin_bit_cast(frag, both);
    };
    // read r of sub-step ks: r < TM is A fragment r, otherwise B fragment r - TM
    auto fetch_one = [&](int ks, int slot, int r) {
        if (r < TM) af[slot][r] = A_TR ? read_tr(As, BM, row_a0 + r * 32, ks) : read_k(As, row_a0 + r * 32, ks);
        else bfv[slot][r - TM] = B_TR ? read_tr(Bs, BN, row_b0 + (r - TM) * 32, ks) : read_k(Bs, row_b0 + (r - TM) * 32, ks);
    };
    constexpr int READS = TM + TN, MFMAS = TM * TN;
#pragma unroll
    for (int r = 0; r < READS; ++r) fetch_one(0, 0, r);
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
        const int cur = ks & 1;
#pragma unroll
        for (int m = 0; m < MFMAS; ++m) {
            const int i = m / TN, j = m % TN;
            __builtin_amdgcn_sched_barrier(0);
            acc[i][j] = Mfma32<T>::run(bfv[cur][j], af[cur][i], acc[i][j]);   // transposed tile: rows = n, columns = m
            if (ks + 1 < KS && m < READS) {
                __builtin_amdgcn_sched_barrier(0);
                fetch_one(ks + 1, cur ^ 1, m);   // issues in the shadow of the MFMA above
            }
        }
        __builtin_amdgcn_sched_barrier(0);
    }
}

// The same MFMA / LDS-read interleave as mma_step, kept as a running pipeline over all the
// sub-steps of the K loop: the fragments live in the object, so the MFMAs of the last sub-step of
// one K-step can run after the workgroup barrier while the first fragments of the next K-step are
// being read.  Without that, every K-step starts with the matrix pipe idle for the LDS latency of
// eight waves' first reads.
// Compile-time index and loop: f(IntC<I>()) for I in [FROM, TO).
template <int M> struct IntC { static constexpr int value = M; };
template <int FROM, int TO, typename F>
FX_DEV void static_for(F&& f) {
    if constexpr (FROM < TO) {
        f(IntC<FROM>());
        static_for<FROM + 1, TO>(f);
    }
}

// Swizzle of a K-contiguous tile whose rows hold BK k-values: 8 chunks per row (BK = 64) or 4 (BK = 32).
template <int BK> FX_DEV int swz_k(int r) { return BK == 64 ? swz(r) : ((r >> 2) & 3); }

template <typename T, int BM, int BN, int WM, int WN, bool A_TR, bool B_TR, int BK = GEMM_BK>
struct MmaPipe {
    static constexpr int TM = WM / 32, TN = WN / 32;
    static constexpr int READS = TM + TN, MFMAS = TM * TN;
    typedef typename Mfma32<T>::frag frag;
    typedef short s16x4_t __attribute__((ext_vector_type(4)));
    typedef short s16x8_t __attribute__((ext_vector_type(8)));
    typedef __attribute__((address_space(3))) s16x4_t* lds_s16x4_ptr;
    static_assert(MFMAS >= READS, "a sub-step must have at least as many MFMAs as fragment reads");
    // one slot of fragments: the operands of one 16-wide sub-step
    struct Slot {
        frag a[TM], b[TN];
    };

    static FX_DEV frag read_k(const T* base, int row0, int ks, int lane) {
        const int r = row0 + (lane & 31);
        return *reinterpret_cast<const frag*>(base + r * BK + (((ks * 2 + (lane >> 5)) ^ swz_k<BK>(r)) << 3));
    }
    static FX_DEV frag read_tr(const T* base, int pitch, int col0, int ks, int lane) {
        const int grp = lane >> 4, sl = lane & 15;
        const int n = col0 + 16 * (grp & 1) + 4 * (sl & 3);
        const int k = 16 * ks + 8 * (grp >> 1) + (sl >> 2);
        const int off = (((n >> 3) ^ (swz_tr(k) % (pitch / 8))) << 3) + (n & 7);
        const s16x4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)(base + k * pitch + off));
        const s16x4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)(base + (k + 4) * pitch + off));
        const s16x8_t both = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
        return __builtin_bit_cast(frag, both);
    }
    // Read R of a sub-step, in the order the MFMAs first use the fragments (A-fragment-major
    // MFMA order): a[0], b[0] .. b[TN-1], a[1] .. a[TM-1].
    template <int R>
    static FX_DEV void fetch_one(Slot& f, const T* As, const T* Bs, int ks, int row_a0, int row_b0, int lane) {
        constexpr bool IS_A = R == 0 || R > TN;
        constexpr int IDX = R == 0 ? 0 : (R <= TN ? R - 1 : R - TN);
        if constexpr (IS_A) f.a[IDX] = A_TR ? read_tr(As, BM, row_a0 + IDX * 32, ks, lane) : read_k(As, row_a0 + IDX * 32, ks, lane);
        else f.b[IDX] = B_TR ? read_tr(Bs, BN, row_b0 + IDX * 32, ks, lane) : read_k(Bs, row_b0 + IDX * 32, ks, lane);
    }
    template <int R = 0>
    static FX_DEV void fetch_all(Slot& f, const T* As, const T* Bs, int ks, int row_a0, int row_b0, int lane) {
        if constexpr (R < READS) {
            fetch_one<R>(f, As, Bs, ks, row_a0, row_b0, lane);
            fetch_all<R + 1>(f, As, Bs, ks, row_a0, row_b0, lane);
        }
    }
    // MFMAs of the sub-step whose fragments sit in `cur`; with FETCH, the fragments of sub-step
    // ks_f of tiles (As_f, Bs_f) are read into `nxt`, one read after each of the first MFMAs.
    // `after(IntC<M>)` runs in the shadow of MFMA M as well (the K loop hangs its global loads there).
    struct Nothing { template <typename I> FX_DEV void operator()(I) const {} };

    template <bool FETCH, int M = 0, typename After = Nothing>
    static FX_DEV void sub(f32x16_t (&acc)[TM][TN], const Slot& cur, Slot& nxt, const T* As_f, const T* Bs_f, int ks_f,
                           int row_a0, int row_b0, int lane, After&& after = After()) {
        if constexpr (M < MFMAS) {
            constexpr int i = M / TN, j = M % TN;
            __builtin_amdgcn_sched_barrier(0);
            acc[i][j] = Mfma32<T>::run(cur.b[j], cur.a[i], acc[i][j]);   // transposed tile: rows = n, columns = m
            if constexpr (FETCH && M < READS) {
                __builtin_amdgcn_sched_barrier(0);
                fetch_one<M>(nxt, As_f, Bs_f, ks_f, row_a0, row_b0, lane);
            }
            __builtin_amdgcn_sched_barrier(0);
            after(IntC<M>());
            sub<FETCH, M + 1>(acc, cur, nxt, As_f, Bs_f, ks_f, row_a0, row_b0, lane, after);
        } else {
            __builtin_amdgcn_sched_barrier(0);
        }
    }
};

// One operand tile's global -> LDS loads as separately issuable instructions.
//
// TileLoader: a wave-uniform 64-bit base (SGPRs, advanced once per K-step) plus loop-invariant
// 32-bit per-lane byte offsets, so issuing an instruction costs no vector ALU work: s_add (LDS
// address), s_mov m0, s_nop, global_load_lds.  With per-lane 64-bit pointers every load carried
// about ten vector instructions between the MFMAs (measured: +3 % with two waves per SIMD, +6-8 %
// with one).  Needs `wave` to be uniform (readfirstlane) and 256 * ld * sizeof(T) < 4 GB.
FX_DEV void load_to_lds16_s(unsigned lane_off, const void* sbase_in, unsigned lds_addr) {
    // the base is wave-uniform by construction; saying so keeps it in scalar registers where the
    // compiler cannot prove it (a no-op where it can)
    const uint64_t u = reinterpret_cast<uint64_t>(sbase_in);
    const void* sbase = reinterpret_cast<const void*>(
        ((uint64_t)(unsigned)__builtin_amdgcn_readfirstlane((int)(unsigned)(u >> 32)) << 32) |
        (uint64_t)(unsigned)__builtin_amdgcn_readfirstlane((int)(unsigned)u));   // the builtin returns a signed int: widen as unsigned
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(lds_addr), "v"(lane_off), "s"(sbase) : "memory", "m0");
}

template <typename T, int ROWS, int NW, bool MN, bool DUAL>
struct TileLoader {
    static constexpr int NI = ROWS / 8 / NW;    // 1 KB instructions per wave: ROWS x 128 bytes in all
    static_assert(ROWS % (8 * NW) == 0, "tile rows must split evenly over the waves");
    static_assert(!(MN && DUAL), "a two-matrix M/N-contiguous tile mixes both matrices inside one instruction");
    unsigned off[NI];
    const T* base;
    const T* base2;
    int64_t step;
    int half;

    FX_DEV void init(const OperandView<T>& op, int wave, int lane) {
        half = op.half;
        if constexpr (!MN) {
            const int rr = lane >> 3, pos = lane & 7;
            const bool gathered = !DUAL && op.row_map != nullptr;      // wave-uniform
#pragma unroll
            for (int j = 0; j < NI; ++j) {
                const int r = (j * NW + wave) * 8 + rr;
                int g = op.origin + (DUAL ? op.dual_index(r) : r);
                g = g < op.ext ? g : op.ext - 1;
                // gathered: the offset is taken from the start of the source matrix (the caller checks
                // that the whole source stays below 4 GB)
                // a map entry outside the source (a mapping that is no permutation, an unwritten entry)
                // must not turn into an address outside it
                const int64_t row = gathered ? (int64_t)min(max(op.row_map[g], 0), op.map_rows - 1) : (int64_t)(g - op.origin);
                off[j] = (unsigned)((row * op.ld + (pos ^ swz(r)) * 8) * (int64_t)sizeof(T));
            }
            base = gathered ? op.base : op.base + (int64_t)op.origin * op.ld;
            base2 = DUAL ? op.base2 + (int64_t)op.origin * op.ld : nullptr;
            step = GEMM_BK;
        } else {
            constexpr int CPR = ROWS / 8, KPI = 64 / CPR;
            static_assert(ROWS == 64 || ROWS == 128 || ROWS == 256, "unsupported tile rows");
            const int kin = lane / CPR, pos = lane % CPR;
#pragma unroll
            for (int j = 0; j < NI; ++j) {
                const int k = (j * NW + wave) * KPI + kin;
                const int c = pos ^ (swz_tr(k) % CPR);
                int g = op.origin + c * 8;
                g = g + 8 <= op.ext ? g : op.ext - 8;
                off[j] = (unsigned)(((int64_t)k * op.ld + (g - op.origin)) * (int64_t)sizeof(T));
            }
            base = op.base + op.origin;
            base2 = nullptr;
            step = (int64_t)GEMM_BK * op.ld;
        }
    }
    // instruction J of the next K-step not yet issued for J (J = 0 .. NI-1 in order)
    template <int J>
    FX_DEV void issue(T* lds, int wave) {
        const unsigned lds_addr = (unsigned)(uintptr_t)(lds + (J * NW + wave) * 512);
        // the rows of one instruction all belong to the same matrix (blocks of `half` >= 8 rows)
        const T* b = (DUAL && ((((J * NW + wave) * 8) & half) != 0)) ? base2 : base;
        load_to_lds16_s(off[J], b, lds_addr);
        if (J == NI - 1) {
            base += step;
            if (DUAL) base2 += step;
        }
    }
};

// The same with per-lane 64-bit source pointers, for the one form whose instructions mix two
// matrices (M/N-contiguous two-matrix tile).
template <typename T, int ROWS, int NW, bool MN, bool DUAL>
struct TileLoaderV {
    static constexpr int NI = ROWS / 8 / NW;
    static_assert(MN && DUAL && ROWS % (8 * NW) == 0 && (ROWS == 64 || ROWS == 128 || ROWS == 256), "see TileLoader");
    const T* src[NI];
    int64_t step;

    FX_DEV void init(const OperandView<T>& op, int wave, int lane) {
        constexpr int CPR = ROWS / 8, KPI = 64 / CPR;
        const int kin = lane / CPR, pos = lane % CPR;
#pragma unroll
        for (int j = 0; j < NI; ++j) {
            const int k = (j * NW + wave) * KPI + kin;
            const int c = pos ^ (swz_tr(k) % CPR);
            const bool second = op.dual_second(c * 8);
            int g = op.origin + op.dual_index(c * 8);
            g = g + 8 <= op.ext ? g : op.ext - 8;
            src[j] = (second ? op.base2 : op.base) + (int64_t)k * op.ld + g;
        }
        step = (int64_t)GEMM_BK * op.ld;
    }
    template <int J>
    FX_DEV void issue(T* lds, int wave) {
        load_to_lds16(src[J], lds + (J * NW + wave) * 512);
        src[J] += step;
    }
};

// M/N-contiguous tile whose k-rows are gathered through OperandView::k_map.  A lane's column offset
// is fixed; its rows change with every K-step, so the byte offsets are rebuilt per step from map
// entries that were requested one step earlier:
//   fetch()    request the map entries of the step after the one about to be issued (clamped to the
//              mapped range, so it may always be called)
//   prepare()  turn the entries on hand into byte offsets; called once per step before its first
//              issue, i.e. right after the K loop's barrier, when no tile load is in flight (the
//              compiler's wait for the entries then costs nothing)
// The whole source must stay below 4 GB (32-bit lane offsets from the operand's base).
template <typename T, int ROWS, int NW>
struct TileLoaderKG {
    static constexpr int NI = ROWS / 8 / NW;
    static constexpr int CPR = ROWS / 8, KPI = 64 / CPR;
    static_assert(ROWS % (8 * NW) == 0 && (ROWS == 64 || ROWS == 128 || ROWS == 256), "see TileLoader");
    unsigned col[NI], roff[NI];
    int nidx[NI];
    const T* base;
    const int32_t* kmap;
    int kpos, kext, map_rows;
    unsigned ld_bytes;

    FX_DEV void fetch() {
#pragma unroll
        for (int j = 0; j < NI; ++j) {
            const int kk = min(kpos + j * NW * KPI, kext - 1);
            nidx[j] = kk >= 0 ? kmap[kk] : 0;       // an empty group has no map entry to read (its map may end the buffer)
        }
        kpos += GEMM_BK;
    }
    FX_DEV void prepare() {
#pragma unroll
        for (int j = 0; j < NI; ++j) roff[j] = col[j] + (unsigned)min(max(nidx[j], 0), map_rows - 1) * ld_bytes;
    }
    FX_DEV void init(const OperandView<T>& op, int wave, int lane) {
        const int kin = lane / CPR, pos = lane % CPR;
#pragma unroll
        for (int j = 0; j < NI; ++j) {
            const int k = (j * NW + wave) * KPI + kin;
            const int c = pos ^ (swz_tr(k) % CPR);
            int g = op.origin + c * 8;
            g = g + 8 <= op.ext ? g : op.ext - 8;
            col[j] = (unsigned)((g - op.origin) * (int)sizeof(T));
        }
        base = op.base + op.origin;
        kmap = op.k_map;
        kext = op.k_ext;
        map_rows = op.map_rows;
        ld_bytes = (unsigned)(op.ld * (int64_t)sizeof(T));
        kpos = wave * KPI + kin;
        fetch();
    }
    template <int J>
    FX_DEV void issue(T* lds, int wave) {
        load_to_lds16_s(roff[J], base, (unsigned)(uintptr_t)(lds + (J * NW + wave) * 512));
    }
};

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

// LOADS_LAND: the caller has requested the first K-step of its next tile before this epilogue; all
// loads issued so far are waited for just before the last band's stores go out (a wait placed after
// the epilogue would also wait for every store to drain, because loads and stores share one counter:
// here the earlier bands' stores have had most of the epilogue to complete).
template <typename T, typename TD, int WM, int WN, bool LOADS_LAND = false, bool NT = false>
FX_DEV void epilogue_tile(f32x16_t (&acc)[WM / 32][WN / 32], const TD* C, TD* D, int64_t ldc, int64_t ldd, int row_base,
                          int col_base, int M, int N, float alpha, float beta, T* smem, int wave, int lane) {
    constexpr int TM = WM / 32, TN = WN / 32;
    constexpr int PITCH = WN + 4;
    constexpr int GROUPS = WN / 8;              // 8-element groups per staged row
    constexpr int PER_LANE = 32 * GROUPS / 64;  // groups per lane per band
    float* stage = reinterpret_cast<float*>(smem) + wave * 32 * PITCH;
    const bool vec_ok = ((ldd & 7) == 0) && ((reinterpret_cast<uintptr_t>(D) & 15u) == 0) &&
                        (beta == 0.f || (((ldc & 7) == 0) && ((reinterpret_cast<uintptr_t>(C) & 15u) == 0)));
    // With beta != 0 the C values of several bands are fetched together before the bands are
    // staged: one exposed memory round trip per group instead of one per band and lane slot (a
    // short-K tile spends as long in its epilogue as in its K loop otherwise).  A group is as many
    // bands as fit 64 registers per lane.
    typedef typename VecOf<TD>::type CV;
    constexpr int CVN = 8 / VecOf<TD>::N;                                   // 16-byte vectors per 8 elements
    constexpr int CB = (CVN == 1 || TM == 1) ? TM : TM / 2;                 // bands per prefetch group
    static_assert(TM % CB == 0, "bands must split evenly into prefetch groups");
    CV cpre[CB][PER_LANE][CVN];
    const bool pre_c = vec_ok && beta != 0.f;
#pragma unroll
    for (int i = 0; i < TM; ++i) {
        // lockstep: every lane of the wave has read the previous band back before this one is staged
        if (pre_c && i % CB == 0) {
#pragma unroll
            for (int b = 0; b < CB; ++b)
#pragma unroll
                for (int t = 0; t < PER_LANE; ++t) {
                    const int id = t * 64 + lane;
                    const int row = row_base + (i + b) * 32 + id / GROUPS, col = col_base + (id % GROUPS) * 8;
                    if (row < M && col + 8 <= N) {
#pragma unroll
                        for (int q = 0; q < CVN; ++q) {
                            const CV* src = reinterpret_cast<const CV*>(C + (int64_t)row * ldc + col + q * VecOf<TD>::N);
                            cpre[b][t][q] = NT ? __builtin_nontemporal_load(src) : *src;
                        }
                    }
                }
        }
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
            if (row >= M || col >= N) continue;
            const float* src = stage + rr * PITCH + cg * 8;
            const f32x4_t lo = *reinterpret_cast<const f32x4_t*>(src), hi = *reinterpret_cast<const f32x4_t*>(src + 4);
            float o[8];
#pragma unroll
            for (int e = 0; e < 4; ++e) { o[e] = alpha * lo[e]; o[4 + e] = alpha * hi[e]; }
            TD* dst = D + (int64_t)row * ldd + col;
            if (vec_ok && col + 8 <= N) {
                if (beta != 0.f) {
#pragma unroll
                    for (int q = 0; q < CVN; ++q)
#pragma unroll
                        for (int e = 0; e < VecOf<TD>::N; ++e)
                            o[q * VecOf<TD>::N + e] += beta * (float)cpre[i % CB][t][q][e];
                }
                store_f32<TD, 8, NT>(dst, o);
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

// K loop of one workgroup tile: leaves the fp32 accumulators of this wave's sub-tile in `acc`
// (transposed MFMA layout, see epilogue_tile).  B_DUAL: the B tile's second half comes from a
// second matrix (OperandView::half); K must then be a multiple of 64.
// ZERO = false: `acc` already holds partial sums and is added to (a product summed over several
// operand pairs, one call per pair; the call ends with a barrier, so the next may start at once).
//
// The loop is an object with two halves so that a workgroup that walks several tiles can request
// the first K-step of its NEXT tile before it runs the epilogue of the current one:
//   begin(A, B, K, buf0)            set up the loaders, issue the loads of K-step 0 into buf0
//   finish(A, B, K, buf0, buf1, acc) issue K-step 1 into buf1, run the K loop, end with a barrier
// Between the two the caller may do anything that leaves buf0 alone and issues no inline-assembly
// loads of its own (compiler-generated loads and stores are fine: the counted waits below only
// assume that loads complete in the order they were issued).
// A_KG / B_KG: that operand (M/N-contiguous) gathers its k-rows through OperandView::k_map.
template <typename T, int BM, int BN, int WAVES_M, int WAVES_N, bool A_MN, bool B_MN, bool B_DUAL = false, bool ZERO = true,
          bool A_KG = false, bool B_KG = false>
struct MainLoop2 {
    static constexpr int NW = WAVES_M * WAVES_N, NT = NW * 64;
    static constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N;
    static constexpr int TM = WM / 32, TN = WN / 32;
    static constexpr int BUF = (BM + BN) * GEMM_BK;
    typedef MmaPipe<T, BM, BN, WM, WN, A_MN, B_MN> Pipe;
    static_assert((!A_KG || A_MN) && (!B_KG || (B_MN && !B_DUAL)), "only M/N-contiguous single-matrix tiles gather k-rows");
    typedef typename std::conditional<A_KG, TileLoaderKG<T, BM, NW>, TileLoader<T, BM, NW, A_MN, false>>::type LoadA;
    typedef typename std::conditional<(B_MN && B_DUAL), TileLoaderV<T, BN, NW, B_MN, B_DUAL>,
                                      typename std::conditional<B_KG, TileLoaderKG<T, BN, NW>,
                                                                TileLoader<T, BN, NW, B_MN, B_DUAL>>::type>::type LoadB;
    static constexpr int LD = LoadA::NI + LoadB::NI;            // load instructions per wave and K-step
    static constexpr int PER = (LD + Pipe::MFMAS - 1) / Pipe::MFMAS;
    static_assert(GEMM_BK == 64, "the pipeline below is written out for four sub-steps per K-step");
    static_assert((size_t)2 * BUF * sizeof(T) <= 160 * 1024, "tile configuration exceeds the 160 KB of LDS");
    LoadA la;
    LoadB lb;
    int wave;

    // instruction IDX of the next K-step into the stage at `buf` (K-steps are issued in order)
    template <int IDX>
    FX_DEV void issue_one(T* buf) {
        if constexpr (IDX == 0) {           // a new step: gathered operands turn their map entries into offsets
            if constexpr (A_KG) la.prepare();
            if constexpr (B_KG) lb.prepare();
        }
        if constexpr (IDX < LoadA::NI) la.template issue<IDX>(buf, wave);
        else if constexpr (IDX < LD) lb.template issue<IDX - LoadA::NI>(buf + BM * GEMM_BK, wave);
        if constexpr (IDX == LD - 1) {      // the step is out: request the entries of the one after
            if constexpr (A_KG) la.fetch();
            if constexpr (B_KG) lb.fetch();
        }
    }
    FX_DEV void issue(T* buf) { static_for<0, LD>([&](auto idx) { issue_one<decltype(idx)::value>(buf); }); }

    FX_DEV void begin(const OperandView<T>& A, const OperandView<T>& B, int K, T* buf0) {
        const int lane = threadIdx.x & 63;
        wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);   // uniform: LDS addresses of the loads stay scalar
        if (K >= GEMM_BK) {
            la.init(A, wave, lane);
            lb.init(B, wave, lane);
            issue(buf0);
        }
    }

    // first_landed: the caller has already waited for the loads of K-step 0 and passed a barrier since
    FX_DEV void finish(const OperandView<T>& A, const OperandView<T>& B, int K, T* buf0, T* buf1, f32x16_t (&acc)[TM][TN],
                       bool first_landed = false) {
        const int tid = threadIdx.x;
        const int lane = tid & 63;
        const int wm = wave / WAVES_N, wn = wave % WAVES_N;
        if (ZERO) {
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j)
#pragma unroll
                    for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;
        }
        const int nfull = K / GEMM_BK;  // K-steps that need no zero fill
        // wave-uniform: does any element of this wave's sub-tile lie inside the matrices?
        const bool live = __builtin_amdgcn_readfirstlane(
            (A.origin + wm * WM < A.ext) && (B_DUAL || B.origin + wn * WN < B.ext));
        auto stage = [&](int kt) { return (kt & 1) ? buf1 : buf0; };
        if (nfull > 0) {
            typename Pipe::Slot f0, f1;
            const int ra = wm * WM, rb = wn * WN;
            // both buffers are free at the start of a tile: the first two K-steps are in flight together
            // and only the first is waited for (short-K tiles spend a visible share of their time here)
            if (nfull > 1) issue(buf1);
            if (!first_landed) {
                if (nfull > 1) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(LD) : "memory");
                else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
                __syncthreads();
            }
            if (!live) {
                // no row (or column) of this wave's sub-tile exists: it keeps loading its share of the
                // stages and meets every barrier of the loop below, and leaves the matrix cores of its
                // SIMD to the wave it shares them with (the last row tile of an expert is mostly this)
                for (int kt = 0; kt + 1 < nfull; ++kt) {
                    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
                    __syncthreads();
                    if (kt + 2 < nfull) issue(stage(kt));
                }
            } else {
            Pipe::fetch_all(f0, buf0, buf0 + BM * GEMM_BK, 0, ra, rb, lane);
            for (int kt = 0; kt + 1 < nfull; ++kt) {
                T* cur = stage(kt);
                T* nxt = stage(kt + 1);
                T* curb = cur + BM * GEMM_BK;
                Pipe::template sub<true>(acc, f0, f1, cur, curb, 1, ra, rb, lane);
                Pipe::template sub<true>(acc, f1, f0, cur, curb, 2, ra, rb, lane);
                Pipe::template sub<true>(acc, f0, f1, cur, curb, 3, ra, rb, lane);
                // Every read of `cur` has been issued.  Once they and this wave's loads of step kt+1 have
                // landed, the barrier makes `nxt` readable and `cur` writable for everyone; the MFMAs of
                // the last sub-step then run while the first fragments of step kt+1 are read and the
                // loads of step kt+2 are issued into `cur`, PER of them after each MFMA (measured 2-3 %
                // faster in every layout than issuing them in one burst after the barrier).
                asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
                __syncthreads();
                const bool more = kt + 2 < nfull;
                Pipe::template sub<true>(acc, f1, f0, nxt, nxt + BM * GEMM_BK, 0, ra, rb, lane, [&](auto m) {
                    constexpr int M = decltype(m)::value;
                    if (more) static_for<M * PER, (M + 1) * PER>([&](auto idx) { issue_one<decltype(idx)::value>(cur); });
                });
            }
            {   // last full K-step: nothing follows it in these buffers
                T* cur = stage(nfull - 1);
                T* curb = cur + BM * GEMM_BK;
                Pipe::template sub<true>(acc, f0, f1, cur, curb, 1, ra, rb, lane);
                Pipe::template sub<true>(acc, f1, f0, cur, curb, 2, ra, rb, lane);
                Pipe::template sub<true>(acc, f0, f1, cur, curb, 3, ra, rb, lane);
                Pipe::template sub<false>(acc, f1, f0, cur, curb, 0, ra, rb, lane);
            }
            }
        }
        if (!B_DUAL && nfull * GEMM_BK < K) {  // K tail: through registers into the K-contiguous layout, zero-filled past K
            Staged2<BM, NT> sa;
            Staged2<BN, NT> sb;
            T* buf = stage(nfull);
            stage2_load<T, BM, NT, A_MN>(sa, A, nfull * GEMM_BK, K, tid);
            stage2_load<T, BN, NT, B_MN>(sb, B, nfull * GEMM_BK, K, tid);
            stage2_store<T, BM, NT, A_MN>(sa, buf, tid);     // `buf` was last read two steps ago
            stage2_store<T, BN, NT, B_MN>(sb, buf + BM * GEMM_BK, tid);
            __syncthreads();
            if (live) mma_step<T, BM, BN, WM, WN, false, false>(buf, buf + BM * GEMM_BK, wm * WM, wn * WN, lane, acc);
        }
        __syncthreads();  // every wave is past its last LDS read: the buffers are free
    }
};

template <typename T, int BM, int BN, int WAVES_M, int WAVES_N, bool A_MN, bool B_MN, bool B_DUAL = false, bool ZERO = true>
FX_DEV void gemm_mainloop2(const OperandView<T>& A, const OperandView<T>& B, int K, T* smem,
                           f32x16_t (&acc)[BM / WAVES_M / 32][BN / WAVES_N / 32]) {
    MainLoop2<T, BM, BN, WAVES_M, WAVES_N, A_MN, B_MN, B_DUAL, ZERO> loop;
    loop.begin(A, B, K, smem);
    loop.finish(A, B, K, smem, smem + loop.BUF, acc);
    static_assert(gemm2_lds_bytes<T, BM, BN, WAVES_M, WAVES_N>() <= 160 * 1024, "tile configuration exceeds the 160 KB of LDS");
}

template <typename T, typename TD, int BM, int BN, int WAVES_M, int WAVES_N, bool A_MN, bool B_MN, bool NT = false>
FX_DEV void gemm_tile2(const OperandView<T>& A, const OperandView<T>& B, const TD* C, TD* D, int64_t ldc,
                       int64_t ldd, int M, int N, int K, float alpha, float beta, T* smem) {
    constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int wm = wave / WAVES_N, wn = wave % WAVES_N;
    f32x16_t acc[WM / 32][WN / 32];
    gemm_mainloop2<T, BM, BN, WAVES_M, WAVES_N, A_MN, B_MN>(A, B, K, smem, acc);
    epilogue_tile<T, TD, WM, WN, false, NT>(acc, C, D, ldc, ldd, A.origin + wm * WM, B.origin + wn * WN, M, N, alpha, beta, smem, wave, lane);
}

// Two GEMMs that share A, fused with the gated activation:
//   P1 = A * op(B1),  P2 = A * op(B2)  (both stored, rounded to T),  ACT = act(gate) * value
// with (gate, value) = (P1, P2) when gate_first, else (P2, P1), evaluated from the ROUNDED P1 / P2
// exactly as a separate activation kernel reading them back would.  The workgroup covers BN/2
// columns of each product.  Needs K % 64 == 0, Nh % 8 == 0, 16-byte aligned rows.
template <typename T, int BM, int BN, int WAVES_M, int WAVES_N, bool A_MN, bool B_MN, bool B_DUAL = false, bool ZERO = true>
FX_DEV void gemm_mainloop32(const OperandView<T>& A, const OperandView<T>& B, int K, T* smem,
                            f32x16_t (&acc)[BM / WAVES_M / 32][BN / WAVES_N / 32]);

// K32: the K loop with 32-wide steps over three stages (K % 32 == 0) instead of 64-wide over two.
//
// Each wave's B rows are WN/2 columns of B1 followed by the same WN/2 columns of B2
// (OperandView::half = WN/2), so a wave holds both pre-activations of its rows x WN/2 columns and
// needs nothing from any other wave.  Per 32-row band it stages the two blocks, rounded to T, in
// its own LDS region and reads them back so that a lane holds 8 consecutive elements of one row of
// each: the activation is computed from the rounded values (as the separate kernel would from
// memory) and the three outputs leave as 16-byte stores, full 128-byte row segments.
template <typename T, int NW, int WN>
constexpr size_t glu_epilogue_lds_bytes() { return (size_t)NW * 2 * 32 * (WN / 2 + 8) * sizeof(T); }

template <typename T, int BM, int BN, int WAVES_M, int WAVES_N, bool B_MN, int ACT, bool K32 = false>
FX_DEV void gemm_tile2_glu(const OperandView<T>& A, const OperandView<T>& B, T* P1, T* P2, int64_t ldp, T* ACTO,
                           int64_t ldact, int M, int Nh, int K, bool gate_first, T* smem) {
    constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N;
    constexpr int TM = WM / 32, TN = WN / 32;
    constexpr int HC = WN / 2;                       // columns of each output per wave
    constexpr int PITCH = HC + 8;                    // staged row pitch in elements: rows stay 16-byte aligned
    constexpr int GROUPS = HC / 8, PER_LANE = 32 * GROUPS / 64;
    static_assert(TN % 2 == 0 && HC % 32 == 0 && (32 * GROUPS) % 64 == 0, "unsupported wave layout for the gated epilogue");
    typedef typename VecOf<T>::type Pack;
    typedef T t4_t __attribute__((ext_vector_type(4)));
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int wm = wave / WAVES_N, wn = wave % WAVES_N;
    f32x16_t acc[TM][TN];
    if constexpr (K32) gemm_mainloop32<T, BM, BN, WAVES_M, WAVES_N, false, B_MN, true>(A, B, K, smem, acc);
    else gemm_mainloop2<T, BM, BN, WAVES_M, WAVES_N, false, B_MN, true>(A, B, K, smem, acc);

    T* st1 = smem + wave * (2 * 32 * PITCH);
    T* st2 = st1 + 32 * PITCH;
    const int row_base = A.origin + wm * WM, col_base = B.origin + wn * HC;
#pragma unroll
    for (int i = 0; i < TM; ++i) {
        // lockstep: every lane of the wave has read the previous band back before this one is staged
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            T* dst = (j < TN / 2 ? st1 : st2) + (lane & 31) * PITCH + (j % (TN / 2)) * 32 + 4 * (lane >> 5);
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const t4_t q = {(T)acc[i][j][4 * g], (T)acc[i][j][4 * g + 1], (T)acc[i][j][4 * g + 2], (T)acc[i][j][4 * g + 3]};
                *reinterpret_cast<t4_t*>(dst + 8 * g) = q;
            }
        }
        // lockstep: a wave reads back only what it wrote itself; its LDS accesses complete in order
#pragma unroll
        for (int t = 0; t < PER_LANE; ++t) {
            const int id = t * 64 + lane;
            const int rr = id / GROUPS, cg = id % GROUPS;
            const int row = row_base + i * 32 + rr, col = col_base + cg * 8;
            if (row < M && col < Nh) {
                const Pack p1 = *reinterpret_cast<const Pack*>(st1 + rr * PITCH + cg * 8);
                const Pack p2 = *reinterpret_cast<const Pack*>(st2 + rr * PITCH + cg * 8);
                Pack y;
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    const float v1 = (float)p1[e], v2 = (float)p2[e];
                    y[e] = (T)(gate_first ? glu_fwd_elem<T, ACT>(v1, v2) : glu_fwd_elem<T, ACT>(v2, v1));
                }
                *reinterpret_cast<Pack*>(P1 + (int64_t)row * ldp + col) = p1;
                *reinterpret_cast<Pack*>(P2 + (int64_t)row * ldp + col) = p2;
                *reinterpret_cast<Pack*>(ACTO + (int64_t)row * ldact + col) = y;
            }
        }
    }
}

// LDS bytes of a workgroup of the gated tile: its K-loop stages or its epilogue staging.
template <typename T, int BM, int BN, int WAVES_M, int WAVES_N, bool K32>
constexpr size_t gemm2_glu_lds_bytes() {
    constexpr size_t tiles = (size_t)(K32 ? 3 * 32 : 2 * GEMM_BK) * (BM + BN) * sizeof(T);
    constexpr size_t epi = glu_epilogue_lds_bytes<T, WAVES_M * WAVES_N, BN / WAVES_N>();
    return tiles > epi ? tiles : epi;
}

// ---------------------------------------------------------------- 32-wide K-steps, three LDS stages
// For problems whose tiles are short-lived (grouped expert GEMMs: K of a few hundred to 2048, a
// large epilogue per tile) the K loop also exists with 32-wide steps: a 128 x 256 (or 256 x 128)
// tile of four waves needs 24 KB per stage, three stages fit the LDS twice per CU, and with at
// most 256 registers per lane two workgroups share a CU: one's epilogue and prologue overlap the
// other's K loop, and the loads of two K-steps are in flight instead of one.
//   K-contiguous tile: LDS row r holds 32 k-values as four 16-byte chunks, chunk c at position
//     c ^ ((r >> 2) & 3) (16 consecutive rows of one chunk column hit 64 distinct banks); a wave
//     instruction covers 16 rows.
//   M/N-contiguous tile: as in the 64-wide form (row k holds the tile's m or n values), 32 rows.
template <typename T, int ROWS, int NW, bool DUAL = false>
FX_DEV void tile32_load_direct(const OperandView<T>& op, int k0, T* lds, int wave, int lane) {
    constexpr int NI = ROWS / 16 / NW;
    static_assert(ROWS % (16 * NW) == 0, "tile rows must split evenly over the waves");
    const int rr = lane >> 2, pos = lane & 3;
#pragma unroll
    for (int j = 0; j < NI; ++j) {
        const int r = (j * NW + wave) * 16 + rr;
        const bool second = DUAL && op.dual_second(r);
        int g = op.origin + (DUAL ? op.dual_index(r) : r);
        g = g < op.ext ? g : op.ext - 1;
        const int c = pos ^ swz_k<32>(r);
        load_to_lds16((second ? op.base2 : op.base) + (int64_t)g * op.ld + k0 + c * 8, lds + (j * NW + wave) * 16 * 32);
    }
}

template <typename T, int ROWS, int NW, bool DUAL = false>
FX_DEV void tile32_load_direct_tr(const OperandView<T>& op, int k0, T* lds, int wave, int lane) {
    constexpr int CPR = ROWS / 8;               // 16-byte chunks per LDS row
    constexpr int KPI = 64 / CPR;               // k-rows per instruction
    constexpr int NI = 32 / KPI / NW;           // instructions per wave
    static_assert((ROWS == 128 || ROWS == 256) && (32 / KPI) % NW == 0, "unsupported tile rows");
    const int kin = lane / CPR, pos = lane % CPR;
#pragma unroll
    for (int j = 0; j < NI; ++j) {
        const int q = j * NW + wave;
        const int k = q * KPI + kin;
        const int c = pos ^ (swz_tr(k) % CPR);
        const bool second = DUAL && op.dual_second(c * 8);
        int g = op.origin + (DUAL ? op.dual_index(c * 8) : c * 8);
        g = g + 8 <= op.ext ? g : op.ext - 8;
        load_to_lds16((second ? op.base2 : op.base) + (int64_t)(k0 + k) * op.ld + g, lds + q * 512);
    }
}

// The 32-wide tiles with a wave-uniform base and 32-bit lane offsets (see TileLoader); the
// M/N-contiguous two-matrix tile keeps the function form above.
template <typename T, int ROWS, int NW, bool MN, bool DUAL>
struct Tile32Loader {
    static constexpr int CPR = ROWS / 8;                      // M/N-contiguous: 16-byte chunks per LDS row
    static constexpr int KPI = 64 / (CPR > 64 ? 64 : CPR);    //                 k-rows per instruction
    static constexpr int NI = MN ? 32 / KPI / NW : ROWS / 16 / NW;
    static_assert(!(MN && DUAL), "a two-matrix M/N-contiguous tile mixes both matrices inside one instruction");
    static_assert(MN ? ((ROWS == 128 || ROWS == 256) && (32 / KPI) % NW == 0) : ROWS % (16 * NW) == 0, "unsupported tile rows");
    unsigned off[NI];
    const T* base;
    const T* base2;
    int64_t step;
    int half;

    FX_DEV void init(const OperandView<T>& op, int wave, int lane) {
        half = op.half;
        if (!MN) {
            const int rr = lane >> 2, pos = lane & 3;
            const bool gathered = !DUAL && op.row_map != nullptr;      // wave-uniform (see TileLoader)
#pragma unroll
            for (int j = 0; j < NI; ++j) {
                const int r = (j * NW + wave) * 16 + rr;
                int g = op.origin + (DUAL ? op.dual_index(r) : r);
                g = g < op.ext ? g : op.ext - 1;
                const int64_t row = gathered ? (int64_t)min(max(op.row_map[g], 0), op.map_rows - 1) : (int64_t)(g - op.origin);
                off[j] = (unsigned)((row * op.ld + (pos ^ swz_k<32>(r)) * 8) * (int64_t)sizeof(T));
            }
            base = gathered ? op.base : op.base + (int64_t)op.origin * op.ld;
            base2 = DUAL ? op.base2 + (int64_t)op.origin * op.ld : nullptr;
            step = 32;
        } else {
            const int kin = lane / CPR, pos = lane % CPR;
#pragma unroll
            for (int j = 0; j < NI; ++j) {
                const int k = (j * NW + wave) * KPI + kin;
                const int c = pos ^ (swz_tr(k) % CPR);
                int g = op.origin + c * 8;
                g = g + 8 <= op.ext ? g : op.ext - 8;
                off[j] = (unsigned)(((int64_t)k * op.ld + (g - op.origin)) * (int64_t)sizeof(T));
            }
            base = op.base + op.origin;
            base2 = nullptr;
            step = (int64_t)32 * op.ld;
        }
    }
    template <int J>
    FX_DEV void issue(T* lds, int wave) {
        const unsigned lds_addr = (unsigned)(uintptr_t)(lds + (J * NW + wave) * 512);
        const T* b = (DUAL && ((((J * NW + wave) * 16) & half) != 0)) ? base2 : base;
        load_to_lds16_s(off[J], b, lds_addr);
        if (J == NI - 1) {
            base += step;
            if (DUAL) base2 += step;
        }
    }
};

template <typename T, int BM, int BN, int WAVES_M, int WAVES_N>
constexpr size_t gemm32_lds_bytes() {
    constexpr size_t tiles = (size_t)3 * (BM + BN) * 32 * sizeof(T);
    constexpr size_t epi = epilogue_lds_bytes<WAVES_M * WAVES_N, BN / WAVES_N>();
    return tiles > epi ? tiles : epi;
}

// K loop with 32-wide steps over three rotating LDS stages; K must be a multiple of 32.
// Leaves the accumulators in `acc` and ends with a barrier (the stages become epilogue staging).
// ZERO = false: `acc` already holds partial sums and is added to.
template <typename T, int BM, int BN, int WAVES_M, int WAVES_N, bool A_MN, bool B_MN, bool B_DUAL, bool ZERO>
FX_DEV void gemm_mainloop32(const OperandView<T>& A, const OperandView<T>& B, int K, T* smem,
                            f32x16_t (&acc)[BM / WAVES_M / 32][BN / WAVES_N / 32]) {
    constexpr int NW = WAVES_M * WAVES_N;
    constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N;
    constexpr int TM = WM / 32, TN = WN / 32;
    constexpr int STAGE = (BM + BN) * 32;
    constexpr int LD = (BM + BN) * 64 / 1024 / NW;      // load instructions per wave per K-step
    static_assert((BM + BN) * 64 % (1024 * NW) == 0, "loads must split evenly over the waves");
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int wm = wave / WAVES_N, wn = wave % WAVES_N;
    if (ZERO) {
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j)
#pragma unroll
                for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;
    }
    const int n = K / 32;
    constexpr bool B_FN = B_MN && B_DUAL;                 // the one tile form without a scalar-base loader
    typedef Tile32Loader<T, BM, NW, A_MN, false> LoadA;
    typedef Tile32Loader<T, BN, NW, B_MN, B_DUAL && !B_FN> LoadB;
    static_assert(LoadA::NI + LoadB::NI == LD, "load instruction count");
    LoadA la;
    LoadB lb;
    la.init(A, wave, lane);
    if constexpr (!B_FN) lb.init(B, wave, lane);
    int kb = 0;                                           // next K-step of the function-form B loader
    // K-steps are issued in order, each exactly once
    auto issue = [&](T* buf) {
        static_for<0, LoadA::NI>([&](auto j) { la.template issue<decltype(j)::value>(buf, wave); });
        if constexpr (B_FN) tile32_load_direct_tr<T, BN, NW, true>(B, (kb++) * 32, buf + BM * 32, wave, lane);
        else static_for<0, LoadB::NI>([&](auto j) { lb.template issue<decltype(j)::value>(buf + BM * 32, wave); });
    };
    if (n > 0) {
        typedef MmaPipe<T, BM, BN, WM, WN, A_MN, B_MN, 32> Pipe;
        typename Pipe::Slot f0, f1;
        const int ra = wm * WM, rb = wn * WN;
        T* cur = smem;
        T* nxt = smem + STAGE;
        T* aft = smem + 2 * STAGE;
        issue(cur);
        if (n > 1) {
            issue(nxt);
            asm volatile("s_waitcnt vmcnt(%0)" ::"n"(LD) : "memory");   // step 0 landed, step 1 may be in flight
        } else {
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        }
        __syncthreads();
        if (n > 2) issue(aft);
        Pipe::fetch_all(f0, cur, cur + BM * 32, 0, ra, rb, lane);
        for (int kt = 0; kt + 1 < n; ++kt) {
            Pipe::template sub<true>(acc, f0, f1, cur, cur + BM * 32, 1, ra, rb, lane);
            // every read of `cur` is issued; step kt+1 must have landed (step kt+2 may still fly)
            if (kt + 2 < n) asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)" ::"n"(LD) : "memory");
            else asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
            __syncthreads();
            if (kt + 3 < n) issue(cur);                  // `cur` is free for everyone now
            Pipe::template sub<true>(acc, f1, f0, nxt, nxt + BM * 32, 0, ra, rb, lane);
            T* t = cur; cur = nxt; nxt = aft; aft = t;
        }
        Pipe::template sub<true>(acc, f0, f1, cur, cur + BM * 32, 1, ra, rb, lane);
        Pipe::template sub<false>(acc, f1, f0, cur, cur, 0, ra, rb, lane);
    }
    __syncthreads();
    static_assert(gemm32_lds_bytes<T, BM, BN, WAVES_M, WAVES_N>() <= 80 * 1024, "two workgroups must fit the LDS of a CU");
}


// ---------------------------------------------------------------- workgroup -> tile maps
// blockIdx.x -> (tile_m, tile_n).  Workgroups are dealt round-robin to the 8 XCDs,
// each with its own L2: give every XCD a contiguous band of tile indices and walk
// the band in groups of GROUP_M tile-rows so concurrently resident workgroups
// share A rows and B columns in L2.
FX_DEV void tile_coords(int pid, int tiles_m, int tiles_n, int& tm, int& tn) {
    const int total = tiles_m * tiles_n;
    constexpr int XCDS = 8;
    int p = pid;
    if (total >= XCDS * 4) {
        const int per = total / XCDS;          // band length; the remainder keeps its order
        const int body = per * XCDS;
        if (pid < body) p = (pid % XCDS) * per + pid / XCDS;
    }
    // 8 tile-rows per group; 4 when the output is very tall (LM-head weight gradient, 501 x 16
    // tiles with K = 8192: 6.96 -> 6.78 ms; at 32 x 16 tiles 4 is 2-3 % slower than 8)
    const int GROUP_M = tiles_m >= 8 * tiles_n ? 4 : 8;
    const int width = GROUP_M * tiles_n;
    const int group = p / width;
    const int first_m = group * GROUP_M;
    const int gsz = (tiles_m - first_m) < GROUP_M ? (tiles_m - first_m) : GROUP_M;
    tm = first_m + (p % width) % gsz;
    tn = (p % width) / gsz;
}

// pid -> position in the logical order: XCD x (= pid % 8) walks positions [x*per, (x+1)*per).
FX_DEV int xcd_band(int pid, int total) {
    constexpr int XCDS = 8;
    if (total < XCDS * 4) return pid;
    const int per = total / XCDS, body = per * XCDS;
    return pid < body ? (pid % XCDS) * per + pid / XCDS : pid;
}

}  // namespace fx
