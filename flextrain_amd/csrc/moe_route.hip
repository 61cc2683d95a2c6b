// MoE routing on gfx950: fused top-k + softmax, the stable expert sort that
// turns (token, slot) pairs into rows of the expert-grouped buffer, and the two
// router backward kernels.
//
// Reference semantics: flextrain/ops/_kernels/moe.py
//   :218-314 fused_topk_softmax_kernel      :317-357 moe_prefix_sum_kernel
//   :360-458 moe_router_gate_bwd_kernel     :461-495 moe_count / moe_map kernels
//   :498-505 moe_copy_counts_kernel         :601-642 load_balance_bwd_kernel
// Expert ids, the index mapping and the per-expert counts are integer results
// and are uniquely determined by those semantics (ties: the smallest expert
// index wins; the sort is stable in flat (token*K + slot) order).
#include <mutex>

#include "common.h"
#include "flexhip.h"

namespace fx {

constexpr float NEG_INF = -__builtin_huge_valf();

// ---------------------------------------------------------------------------
// Top-k + softmax.  LPT lanes share a token; a lane owns NV packs of 8
// consecutive experts, pack v of lane l covering experts (v*LPT + l)*8 .. +7.
// ---------------------------------------------------------------------------
template <int W>
FX_DEV void group_argmax(float& v, int& idx) {
#pragma unroll
    for (int off = W / 2; off > 0; off >>= 1) {
        const float ov = __shfl_xor(v, off, 64);
        const int oi = __shfl_xor(idx, off, 64);
        if (ov > v || (ov == v && oi < idx)) { v = ov; idx = oi; }
    }
}

template <typename TL, typename TW, int LPT, int NV, int MODE>
__global__ __launch_bounds__(256) void topk_softmax_kernel(
    const TL* __restrict__ LOGITS, int32_t* __restrict__ IDS, TW* __restrict__ WTS, int64_t T, int E,
    int K, int BIG) {
    constexpr int TPB = 256 / LPT;  // tokens per workgroup
    constexpr int SLOTS = 8 * NV;
    const int g = threadIdx.x / LPT;
    const int l = threadIdx.x % LPT;
    const int64_t t = (int64_t)blockIdx.x * TPB + g;
    const bool tok_ok = t < T;
    const int64_t tt = tok_ok ? t : 0;  // idle groups shadow token 0, stores masked

    float r[NV][8];
#pragma unroll
    for (int v = 0; v < NV; ++v) {
        const int e0 = (v * LPT + l) * 8;
        if (e0 + 8 <= E && (E & 7) == 0) {
            load_f32<TL, 8>(LOGITS + tt * E + e0, r[v]);
        } else {
#pragma unroll
            for (int j = 0; j < 8; ++j) r[v][j] = (e0 + j < E) ? (float)LOGITS[tt * E + e0 + j] : NEG_INF;
        }
    }
    if (MODE == 1) {
        // stable softmax over all E experts first (moe.py:271-277)
        float mx = NEG_INF;
#pragma unroll
        for (int v = 0; v < NV; ++v)
#pragma unroll
            for (int j = 0; j < 8; ++j) mx = fmaxf(mx, r[v][j]);
        mx = group_max<LPT>(mx);
        float sum = 0.f;
#pragma unroll
        for (int v = 0; v < NV; ++v)
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const int e = (v * LPT + l) * 8 + j;
                r[v][j] = e < E ? expf(r[v][j] - mx) : 0.f;
                sum += r[v][j];
            }
        sum = group_sum<LPT>(sum);
#pragma unroll
        for (int v = 0; v < NV; ++v)
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const int e = (v * LPT + l) * 8 + j;
                r[v][j] = e < E ? r[v][j] / sum : NEG_INF;
            }
    }

    float ex[SLOTS];
#pragma unroll
    for (int s = 0; s < SLOTS; ++s) ex[s] = 0.f;
    float first = 0.f, sum_exp = 0.f;
    for (int k = 0; k < K; ++k) {
        // lane-local best: ascending expert order with strict '>' keeps the
        // smallest index among equal values
        float bv = NEG_INF;
        int bi = BIG;
#pragma unroll
        for (int v = 0; v < NV; ++v)
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const int e = (v * LPT + l) * 8 + j;
                if (e < E && (r[v][j] > bv || bi == BIG)) { bv = r[v][j]; bi = e; }
            }
        group_argmax<LPT>(bv, bi);
        // the selected value goes through the weights buffer's dtype (moe.py:292-293)
        const float stored = round_to<TW>(bv);
        if (MODE == 0) {
            if (k == 0) first = stored;
            const float e = expf(stored - first);
            sum_exp += e;
#pragma unroll
            for (int s = 0; s < SLOTS; ++s)
                if (s == k / LPT && l == k % LPT) ex[s] = e;
        } else {
#pragma unroll
            for (int s = 0; s < SLOTS; ++s)
                if (s == k / LPT && l == k % LPT) ex[s] = bv;
        }
        if (tok_ok && l == 0) IDS[t * K + k] = bi;
#pragma unroll
        for (int v = 0; v < NV; ++v)
#pragma unroll
            for (int j = 0; j < 8; ++j)
                if ((v * LPT + l) * 8 + j == bi) r[v][j] = NEG_INF;
    }
    if (!tok_ok) return;
#pragma unroll
    for (int s = 0; s < SLOTS; ++s) {
        const int k = s * LPT + l;
        if (k < K) WTS[t * K + k] = (TW)(MODE == 0 ? ex[s] / sum_exp : ex[s]);
    }
}

// ---------------------------------------------------------------------------
// Stable counting sort of flat expert ids.
//   phase 1: per-chunk (256 ids) histogram            -> cnt[e][b]
//   phase 2: per-expert exclusive scan over chunks, expert totals and starts
//   phase 3: rank inside the chunk + offsets           -> index_mapping
// ---------------------------------------------------------------------------
constexpr int SORT_CHUNK = 256;

template <typename TI>
__global__ __launch_bounds__(SORT_CHUNK) void sort_hist_kernel(const TI* __restrict__ IDS, int64_t n,
                                                               int E, int NB, int32_t* __restrict__ CNT) {
    extern __shared__ int32_t hist[];
    for (int e = threadIdx.x; e < E; e += SORT_CHUNK) hist[e] = 0;
    __syncthreads();
    const int64_t i = (int64_t)blockIdx.x * SORT_CHUNK + threadIdx.x;
    if (i < n) {
        const int e = (int)IDS[i];
        if (e >= 0 && e < E) atomicAdd(&hist[e], 1);
    }
    __syncthreads();
    for (int e = threadIdx.x; e < E; e += SORT_CHUNK) CNT[(size_t)e * NB + blockIdx.x] = hist[e];
}

// One workgroup per expert: exclusive scan of its NB chunk counts in place, total to TOTAL[e].
__global__ __launch_bounds__(256) void sort_scan_kernel(int32_t* __restrict__ CNT, int NB,
                                                        int32_t* __restrict__ TOTAL) {
    __shared__ int32_t wsum[4];
    __shared__ int32_t carry_s;
    int32_t* row = CNT + (size_t)blockIdx.x * NB;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    if (threadIdx.x == 0) carry_s = 0;
    __syncthreads();
    for (int base = 0; base < NB; base += 256) {
        const int b = base + threadIdx.x;
        const int32_t c = b < NB ? row[b] : 0;
        int32_t inc = c;  // inclusive scan inside the wave
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) {
            const int32_t o = __shfl_up(inc, off, 64);
            if (lane >= off) inc += o;
        }
        if (lane == 63) wsum[wave] = inc;
        __syncthreads();
        int32_t before = carry_s;
        for (int w = 0; w < wave; ++w) before += wsum[w];
        if (b < NB) row[b] = before + inc - c;
        __syncthreads();
        if (threadIdx.x == 255) carry_s = before + inc;
        __syncthreads();
    }
    if (threadIdx.x == 0) TOTAL[blockIdx.x] = carry_s;
}

// Single workgroup: START[e] = sum_{e' < e} TOTAL[e']; optional copies of the totals.
__global__ __launch_bounds__(256) void sort_starts_kernel(const int32_t* __restrict__ TOTAL, int E,
                                                          int32_t* __restrict__ START,
                                                          int32_t* __restrict__ COUNTS_OUT,
                                                          int32_t* __restrict__ COUNTS_HOST) {
    __shared__ int32_t wsum[4];
    __shared__ int32_t carry_s;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    if (threadIdx.x == 0) carry_s = 0;
    __syncthreads();
    for (int base = 0; base < E; base += 256) {
        const int e = base + threadIdx.x;
        const int32_t c = e < E ? TOTAL[e] : 0;
        int32_t inc = c;
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) {
            const int32_t o = __shfl_up(inc, off, 64);
            if (lane >= off) inc += o;
        }
        if (lane == 63) wsum[wave] = inc;
        __syncthreads();
        int32_t before = carry_s;
        for (int w = 0; w < wave; ++w) before += wsum[w];
        if (e < E) {
            START[e] = before + inc - c;
            if (COUNTS_OUT) COUNTS_OUT[e] = c;
            if (COUNTS_HOST) COUNTS_HOST[e] = c;  // zero-copy store into pinned host memory
        }
        __syncthreads();
        if (threadIdx.x == 255) carry_s = before + inc;
        __syncthreads();
    }
}

template <typename TI, typename TO>
__global__ __launch_bounds__(SORT_CHUNK) void sort_map_kernel(const TI* __restrict__ IDS, int64_t n, int E,
                                                              int NB, const int32_t* __restrict__ CNT,
                                                              const int32_t* __restrict__ START,
                                                              TO* __restrict__ MAP) {
    __shared__ int32_t ids[SORT_CHUNK];
    const int64_t i = (int64_t)blockIdx.x * SORT_CHUNK + threadIdx.x;
    const int e = i < n ? (int)IDS[i] : -1;
    ids[threadIdx.x] = e;
    __syncthreads();
    if (i >= n) return;
    if (e < 0 || e >= E) {     // not counted by the histogram: give the pair a row inside the buffers, so that
        MAP[i] = (TO)0;        // a scatter or gather through this map cannot leave them
        return;
    }
    int rank = 0;
    const int4* v = reinterpret_cast<const int4*>(ids);
    const int me = threadIdx.x;
    for (int j4 = 0; j4 * 4 < me; ++j4) {  // earlier elements of the chunk with the same expert
        const int4 q = v[j4];
        rank += (q.x == e) & (j4 * 4 + 0 < me);
        rank += (q.y == e) & (j4 * 4 + 1 < me);
        rank += (q.z == e) & (j4 * 4 + 2 < me);
        rank += (q.w == e) & (j4 * 4 + 3 < me);
    }
    MAP[i] = (TO)(START[e] + CNT[(size_t)e * NB + blockIdx.x] + rank);
}

__global__ __launch_bounds__(256) void copy_i32_kernel(const int32_t* __restrict__ SRC,
                                                       int32_t* __restrict__ DST, int n) {
    for (int i = threadIdx.x; i < n; i += 256) DST[i] = SRC[i];
}

// ---------------------------------------------------------------------------
// Router backward (one wave per token).
// ---------------------------------------------------------------------------
// Row of pair i in the expert-sorted buffers, clamped to them (see load_index in moe_data.hip).
template <typename TI>
FX_DEV int64_t pair_row(const TI* __restrict__ indices, int64_t i, int64_t rows) {
    const int64_t r = (int64_t)indices[i];
    return r < 0 ? 0 : (r < rows ? r : rows - 1);
}

template <typename T, typename TDP, typename TI, int MODE>
__global__ __launch_bounds__(256) void router_gate_bwd_kernel(
    T* __restrict__ DLOGITS, const TDP* __restrict__ DPROBS, const T* __restrict__ PROBS,
    const TI* __restrict__ INDICES, const int32_t* __restrict__ EXPERTS, const T* __restrict__ LOGITS,
    int64_t Tn, int K, int E) {
    const int lane = threadIdx.x & 63;
    const int64_t t = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (t >= Tn) return;
    if (MODE == 0) {
        // dz_k = p_k (dp_k - sum_j p_j dp_j), added into dlogits[t, expert_k]
        float dot = 0.f;
        for (int k = lane; k < K; k += 64)
            dot += (float)DPROBS[pair_row(INDICES, t * K + k, Tn * K)] * (float)PROBS[t * K + k];
        dot = group_sum<64>(dot);
        for (int k = lane; k < K; k += 64) {
            const float p = (float)PROBS[t * K + k];
            const float dp = (float)DPROBS[pair_row(INDICES, t * K + k, Tn * K)];
            const int e = EXPERTS[t * K + k];
            if (e >= 0 && e < E) {
                T* o = DLOGITS + t * E + e;
                *o = (T)((float)*o + round_to<T>(p * (dp - dot)));
            }
        }
    } else {
        // full-E softmax recomputed from the logits (moe.py:418-458)
        float mx = NEG_INF;
        for (int e = lane; e < E; e += 64) mx = fmaxf(mx, (float)LOGITS[t * E + e]);
        mx = group_max<64>(mx);
        float sum = 0.f;
        for (int e = lane; e < E; e += 64) sum += expf((float)LOGITS[t * E + e] - mx);
        sum = group_sum<64>(sum);
        float row_dot = 0.f;
        for (int k = lane; k < K; k += 64) {
            const int e = EXPERTS[t * K + k];
            if (e >= 0 && e < E)
                row_dot += (float)DPROBS[pair_row(INDICES, t * K + k, Tn * K)] * (expf((float)LOGITS[t * E + e] - mx) / sum);
        }
        row_dot = group_sum<64>(row_dot);
        for (int e = lane; e < E; e += 64) {
            const float p = expf((float)LOGITS[t * E + e] - mx) / sum;
            float dz = -p * row_dot;
            for (int k = 0; k < K; ++k)
                if (EXPERTS[t * K + k] == e) dz += (float)DPROBS[pair_row(INDICES, t * K + k, Tn * K)] * p;
            T* o = DLOGITS + t * E + e;
            *o = (T)((float)*o + round_to<T>(dz));
        }
    }
}

// dlogits += scale * p * (f - <f, p>),  p = softmax(logits[t, :]),  f = counts * inv_pairs
template <typename T, typename TD>
__global__ __launch_bounds__(256) void load_balance_bwd_kernel(
    const T* __restrict__ LOGITS, const int32_t* __restrict__ COUNTS, TD* __restrict__ DLOGITS,
    int64_t Tn, int E, float inv_pairs, float scale) {
    const int lane = threadIdx.x & 63;
    const int64_t t = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (t >= Tn) return;
    float mx = NEG_INF;
    for (int e = lane; e < E; e += 64) mx = fmaxf(mx, (float)LOGITS[t * E + e]);
    mx = group_max<64>(mx);
    float sum = 0.f, dot = 0.f;
    for (int e = lane; e < E; e += 64) {
        const float ex = expf((float)LOGITS[t * E + e] - mx);
        sum += ex;
        dot += ex * ((float)COUNTS[e] * inv_pairs);
    }
    sum = group_sum<64>(sum);
    dot = group_sum<64>(dot) / sum;
    for (int e = lane; e < E; e += 64) {
        const float p = expf((float)LOGITS[t * E + e] - mx) / sum;
        const float f = (float)COUNTS[e] * inv_pairs;
        TD* o = DLOGITS + t * E + e;
        *o = (TD)((float)*o + scale * p * (f - dot));
    }
}

template <typename TL, typename TW, int MODE>
static int launch_topk(const void* logits, int32_t* ids, void* wts, int64_t T, int E, int K, hipStream_t s) {
    const TL* L = reinterpret_cast<const TL*>(logits);
    TW* W = reinterpret_cast<TW*>(wts);
    int lpt = 1;
    while (lpt < 64 && lpt * 8 < E) lpt *= 2;
    const int nv = (E + lpt * 8 - 1) / (lpt * 8);
    const int BIG = 1 << 30;
#define FX_TOPK_CASE(L_, V_)                                                                   \
    if (lpt == L_ && nv <= V_) {                                                               \
        constexpr int TPB = 256 / L_;                                                          \
        topk_softmax_kernel<TL, TW, L_, V_, MODE><<<(unsigned)((T + TPB - 1) / TPB), 256, 0, s>>>(L, ids, W, T, E, K, BIG); \
        return 0;                                                                              \
    }
    FX_TOPK_CASE(1, 1) FX_TOPK_CASE(2, 1) FX_TOPK_CASE(4, 1) FX_TOPK_CASE(8, 1) FX_TOPK_CASE(16, 1)
    FX_TOPK_CASE(32, 1) FX_TOPK_CASE(64, 1) FX_TOPK_CASE(64, 2) FX_TOPK_CASE(64, 4)
#undef FX_TOPK_CASE
    return -1;
}

}  // namespace fx

using namespace fx;

extern "C" int fx_topk_softmax(const void* logits, int32_t* ids_out, void* weights_out, int64_t T,
                               int E, int K, int logits_dt, int weights_dt, int mode,
                               hipStream_t stream) {
    if (T < 0 || E <= 0 || K <= 0) FX_FAIL("fx_topk_softmax: bad shape T=%lld E=%d K=%d", (long long)T, E, K);
    if (K > E) FX_FAIL("fx_topk_softmax: top_k (%d) cannot exceed num_experts (%d)", K, E);
    if (E > 2048) FX_FAIL("fx_topk_softmax: at most 2048 experts supported (got %d)", E);
    if (mode != 0 && mode != 1) FX_FAIL("fx_topk_softmax: unknown mode %d", mode);
    if (T == 0) return 0;
    if (!logits || !ids_out || !weights_out) FX_FAIL("fx_topk_softmax: null pointer");
    if (!aligned16(logits)) FX_FAIL("fx_topk_softmax: logits must be 16-byte aligned");
    int rc = -1;
    FX_DISPATCH_DTYPE(logits_dt, TL,
        FX_DISPATCH_DTYPE(weights_dt, TW,
            rc = mode == 0 ? launch_topk<TL, TW, 0>(logits, ids_out, weights_out, T, E, K, stream)
                           : launch_topk<TL, TW, 1>(logits, ids_out, weights_out, T, E, K, stream)));
    if (rc != 0) FX_FAIL("fx_topk_softmax: no kernel for E=%d", E);
    FX_CHECK_LAUNCH("fx_topk_softmax");
    return 0;
}

static inline int sort_chunks(int64_t n) { return (int)((n + SORT_CHUNK - 1) / SORT_CHUNK); }

extern "C" size_t fx_moe_sort_ws_bytes(int64_t n_pairs, int E) {
    if (n_pairs <= 0 || E <= 0) return 0;
    return ((size_t)E * sort_chunks(n_pairs) + 2 * (size_t)E) * sizeof(int32_t);
}

extern "C" int fx_moe_sort(const void* ids, int ids_are_int64, int64_t n_pairs, int E, void* index_out,
                           int index_is_int64, int32_t* counts_out, int32_t* counts_host, void* ws,
                           size_t ws_bytes, hipStream_t stream) {
    if (n_pairs < 0 || E <= 0) FX_FAIL("fx_moe_sort: bad shape n=%lld E=%d", (long long)n_pairs, E);
    if (E * sizeof(int32_t) > 60 * 1024) FX_FAIL("fx_moe_sort: too many experts (%d)", E);
    const int NB = sort_chunks(n_pairs);
    const size_t need = fx_moe_sort_ws_bytes(n_pairs > 0 ? n_pairs : 1, E);
    if (!ws || ws_bytes < need) FX_FAIL("fx_moe_sort: workspace too small (%zu < %zu bytes)", ws_bytes, need);
    if (n_pairs > 0 && (!ids || !index_out)) FX_FAIL("fx_moe_sort: null pointer");
    int32_t* cnt = reinterpret_cast<int32_t*>(ws);
    int32_t* total = cnt + (size_t)E * (NB > 0 ? NB : 1);
    int32_t* start = total + E;
    if (n_pairs > 0) {
        if (ids_are_int64)
            sort_hist_kernel<int64_t><<<NB, SORT_CHUNK, E * sizeof(int32_t), stream>>>(reinterpret_cast<const int64_t*>(ids), n_pairs, E, NB, cnt);
        else
            sort_hist_kernel<int32_t><<<NB, SORT_CHUNK, E * sizeof(int32_t), stream>>>(reinterpret_cast<const int32_t*>(ids), n_pairs, E, NB, cnt);
        FX_CHECK_LAUNCH("fx_moe_sort(hist)");
    }
    sort_scan_kernel<<<E, 256, 0, stream>>>(cnt, NB, total);
    FX_CHECK_LAUNCH("fx_moe_sort(scan)");
    sort_starts_kernel<<<1, 256, 0, stream>>>(total, E, start, counts_out, counts_host);
    FX_CHECK_LAUNCH("fx_moe_sort(starts)");
    if (n_pairs > 0) {
#define FX_MAP(TI, TO) sort_map_kernel<TI, TO><<<NB, SORT_CHUNK, 0, stream>>>(reinterpret_cast<const TI*>(ids), n_pairs, E, NB, cnt, start, reinterpret_cast<TO*>(index_out))
        if (ids_are_int64 && index_is_int64) FX_MAP(int64_t, int64_t);
        else if (ids_are_int64) FX_MAP(int64_t, int32_t);
        else if (index_is_int64) FX_MAP(int32_t, int64_t);
        else FX_MAP(int32_t, int32_t);
#undef FX_MAP
        FX_CHECK_LAUNCH("fx_moe_sort(map)");
    }
    return 0;
}

// ---- the same sort for callers that may not allocate -----------------------------------------
// Callers under HIP graph capture, or in loops that must not touch an allocator, cannot lend a
// workspace sized per call.  This variant keeps the chunk histograms, totals and starts in a
// fixed array in device memory that is part of the loaded code object (one copy per GPU, held
// until the process ends).  The array's name is only a host-side handle: kernels get the
// device address that hipGetSymbolAddress reports for the GPU that is current.
constexpr size_t SORT_STATIC_WORDS = (size_t)2 * 1024 * 1024 + 1024;          // 8 MiB + 4 KiB
static __device__ __align__(256) int32_t scratch[SORT_STATIC_WORDS];

namespace {
constexpr int MAX_DEVICES = 64;
int32_t* g_scratch_ptr[MAX_DEVICES] = {};
std::mutex g_scratch_mutex;

// Device address of `scratch` on the current GPU, resolved once per GPU; nullptr on failure.
int32_t* static_scratch() {
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= MAX_DEVICES) {
        (void)hipGetLastError();
        fprintf(stderr, "flexhip: fx_moe_sort_noalloc: cannot tell the current device\n");
        return nullptr;
    }
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        void* p = nullptr;
        hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !p) {
            (void)hipGetLastError();
            fprintf(stderr, "flexhip: fx_moe_sort_noalloc: hipGetSymbolAddress failed on device %d: %s\n", dev,
                    hipGetErrorString(e));
            return nullptr;
        }
        g_scratch_ptr[dev] = reinterpret_cast<int32_t*>(p);
    }
    return g_scratch_ptr[dev];
}
}  // namespace

extern "C" size_t fx_moe_sort_noalloc_max_words(void) { return SORT_STATIC_WORDS; }

extern "C" int fx_moe_sort_noalloc_init(void) { return static_scratch() ? 0 : -1; }

extern "C" int fx_moe_sort_noalloc(const void* ids, int ids_are_int64, int64_t n_pairs, int E, void* index_out,
                                   int index_is_int64, int32_t* counts_out, int32_t* counts_host,
                                   hipStream_t stream) {
    if (n_pairs < 0 || E <= 0) FX_FAIL("fx_moe_sort_noalloc: bad shape n=%lld E=%d", (long long)n_pairs, E);
    const size_t need = fx_moe_sort_ws_bytes(n_pairs > 0 ? n_pairs : 1, E);
    if (need > SORT_STATIC_WORDS * sizeof(int32_t))
        FX_FAIL("fx_moe_sort_noalloc: %lld pairs over %d experts need %zu bytes of scratch, the built-in array holds "
                "%zu (E * ceil(n / 256) + 2 E <= %zu words); use fx_moe_sort with a workspace",
                (long long)n_pairs, E, need, SORT_STATIC_WORDS * sizeof(int32_t), SORT_STATIC_WORDS);
    int32_t* ws = static_scratch();
    if (!ws) return -1;
    // every word the kernels read was written earlier in the same call (chunk histograms by the
    // histogram kernel, totals by the scan, starts by the starts kernel): nothing needs clearing
    return fx_moe_sort(ids, ids_are_int64, n_pairs, E, index_out, index_is_int64, counts_out, counts_host, ws,
                       SORT_STATIC_WORDS * sizeof(int32_t), stream);
}

extern "C" int fx_copy_i32(const int32_t* src_dev, int32_t* dst, int n, hipStream_t stream) {
    if (n < 0) FX_FAIL("fx_copy_i32: negative count");
    if (n == 0) return 0;
    if (!src_dev || !dst) FX_FAIL("fx_copy_i32: null pointer");
    copy_i32_kernel<<<1, 256, 0, stream>>>(src_dev, dst, n);
    FX_CHECK_LAUNCH("fx_copy_i32");
    return 0;
}

extern "C" int fx_router_gate_bwd(void* dlogits, const void* dprobs, const void* probs, const void* indices,
                                  int indices_are_int64, const int32_t* chosen_experts, const void* logits,
                                  int64_t T, int K, int E, int dt, int dprobs_dt, int mode,
                                  hipStream_t stream) {
    if (T < 0 || K <= 0 || E <= 0) FX_FAIL("fx_router_gate_bwd: bad shape");
    if (mode != 0 && mode != 1) FX_FAIL("fx_router_gate_bwd: unknown mode %d", mode);
    if (T == 0) return 0;
    if (!dlogits || !dprobs || !probs || !indices || !chosen_experts) FX_FAIL("fx_router_gate_bwd: null pointer");
    if (mode == 1 && !logits) FX_FAIL("fx_router_gate_bwd: softmax_then_topk needs the logits");
    const unsigned grid = (unsigned)((T + 3) / 4);
#define FX_RG(TI, M) router_gate_bwd_kernel<TT, TDP, TI, M><<<grid, 256, 0, stream>>>(reinterpret_cast<TT*>(dlogits), reinterpret_cast<const TDP*>(dprobs), reinterpret_cast<const TT*>(probs), reinterpret_cast<const TI*>(indices), chosen_experts, reinterpret_cast<const TT*>(logits), T, K, E)
    FX_DISPATCH_DTYPE(dt, TT,
        FX_DISPATCH_DTYPE(dprobs_dt, TDP,
            if (indices_are_int64) { if (mode == 0) FX_RG(int64_t, 0); else FX_RG(int64_t, 1); }
            else { if (mode == 0) FX_RG(int32_t, 0); else FX_RG(int32_t, 1); }));
#undef FX_RG
    FX_CHECK_LAUNCH("fx_router_gate_bwd");
    return 0;
}

extern "C" int fx_load_balance_bwd(const void* logits, const int32_t* expert_counts, void* dlogits, int64_t T,
                                   int E, int top_k, float scale, int logits_dt, int dlogits_dt,
                                   hipStream_t stream) {
    if (T < 0 || E <= 0 || top_k <= 0) FX_FAIL("fx_load_balance_bwd: bad shape");
    if (T == 0) return 0;
    if (!logits || !expert_counts || !dlogits) FX_FAIL("fx_load_balance_bwd: null pointer");
    const float inv_pairs = 1.0f / ((float)T * (float)top_k);
    const unsigned grid = (unsigned)((T + 3) / 4);
    FX_DISPATCH_DTYPE(logits_dt, TT,
        FX_DISPATCH_DTYPE(dlogits_dt, TD,
            load_balance_bwd_kernel<TT, TD><<<grid, 256, 0, stream>>>(
                reinterpret_cast<const TT*>(logits), expert_counts, reinterpret_cast<TD*>(dlogits), T, E,
                inv_pairs, scale)));
    FX_CHECK_LAUNCH("fx_load_balance_bwd");
    return 0;
}
