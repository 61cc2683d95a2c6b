// RMSNorm forward / recompute / backward for gfx950.
//
// Semantics follow the reference Triton kernels
// (flextrain/ops/_kernels/rmsnorm.py:9-100 fwd, :103-163 recompute,
// :170-274 dx, :279-412 dW) with one structural change: the backward is ONE
// pass over dy/x that produces dx (optionally accumulated into the caller's
// buffer), the re-materialised y, and per-workgroup dW partial sums; a second
// tiny kernel folds the partials in a fixed order, so dW is deterministic (the
// reference's fp32 atomics are not) and dy/x are read once instead of twice.
//
// Layout: X is a contiguous (rows, ncols) matrix.  Per-head normalisation
// (head_dim given) is the same kernel on the (T*H, head_dim) view, because the
// reference requires contiguous X and a single shared (head_dim,) weight.
//
// Thread mapping: LPR lanes cooperate on a row, each lane owns MAXV packs of 8
// consecutive columns, pack v of lane l covering columns (v*LPR + l)*8 .. +7,
// so that a wave's accesses are 1 KiB contiguous (bf16) per pack.
#include "common.h"
#include "flexhip.h"

namespace fx {

template <typename T>
FX_DEV void load8(const T* p, float (&o)[8]) { load_f32<T, 8>(p, o); }
template <typename T>
FX_DEV void store8(T* p, const float (&o)[8]) { store_f32<T, 8>(p, o); }

// Weight pack load with a runtime dtype (wave-uniform branch).
FX_DEV void load_w8(const void* w, int w_dt, int col, float (&o)[8]) {
    if (w_dt == DT_F32) load8<float>(reinterpret_cast<const float*>(w) + col, o);
    else if (w_dt == DT_BF16) load8<bf16>(reinterpret_cast<const bf16*>(w) + col, o);
    else load8<f16>(reinterpret_cast<const f16*>(w) + col, o);
}

// Sum over the LPR lanes that share a row.  For LPR == 256 the row spans four
// consecutive waves and goes through `red` (one float per wave of the block).
template <int LPR>
FX_DEV float row_sum(float v, float* red, int tid) {
    if constexpr (LPR <= 64) {
        return group_sum<LPR>(v);
    } else {
        static_assert(LPR == 256, "row spans 4 waves");
        v = group_sum<64>(v);
        const int wave = tid >> 6;
        __syncthreads();
        if ((tid & 63) == 0) red[wave] = v;
        __syncthreads();
        const int g0 = wave & ~3;
        return (red[g0] + red[g0 + 1]) + (red[g0 + 2] + red[g0 + 3]);
    }
}

// ---------------------------------------------------------------------------
// Forward (and forward-from-saved-rstd).
// ---------------------------------------------------------------------------
template <typename T, int LPR, int MAXV, int THREADS, bool SAVED_RSTD>
__global__ __launch_bounds__(THREADS) void rmsnorm_fwd_kernel(
    const T* X, const void* __restrict__ W, int w_dt, T* Y /* may alias X */,
    float* __restrict__ RSTD, int64_t rows, int ncols, float eps) {
    constexpr int G = THREADS / LPR;  // rows per workgroup
    __shared__ float red[THREADS / 64];
    const int tid = threadIdx.x;
    const int g = tid / LPR;
    const int l = tid % LPR;
    const int64_t row = (int64_t)blockIdx.x * G + g;
    const bool row_ok = row < rows;

    // the weight packs are requested together with the row: fetched after the reduction they
    // would add a second exposed memory round trip to a kernel that lasts two or three
    float x[MAXV][8], w[MAXV][8];
    float ss = 0.f;
#pragma unroll
    for (int v = 0; v < MAXV; ++v) {
        const int col = (v * LPR + l) * 8;
        if (row_ok && col < ncols) {
            load8<T>(X + row * ncols + col, x[v]);
            if (W != nullptr) load_w8(W, w_dt, col, w[v]);
        } else {
#pragma unroll
            for (int j = 0; j < 8; ++j) x[v][j] = 0.f;
        }
        if (!SAVED_RSTD) {
#pragma unroll
            for (int j = 0; j < 8; ++j) ss += x[v][j] * x[v][j];
        }
    }
    float rstd;
    if (SAVED_RSTD) {
        rstd = row_ok ? RSTD[row] : 0.f;
    } else {
        ss = row_sum<LPR>(ss, red, tid);
        rstd = rsqrtf(ss / (float)ncols + eps);
        if (row_ok && l == 0) RSTD[row] = rstd;
    }
#pragma unroll
    for (int v = 0; v < MAXV; ++v) {
        const int col = (v * LPR + l) * 8;
        if (row_ok && col < ncols) {
            float y[8];
            if (W != nullptr) {
#pragma unroll
                for (int j = 0; j < 8; ++j) y[j] = round_to<T>(x[v][j] * rstd) * w[v][j];
            } else {
#pragma unroll
                for (int j = 0; j < 8; ++j) y[j] = x[v][j] * rstd;
            }
            store8<T>(Y + row * ncols + col, y);
        }
    }
}

// Any-shape fallback: one workgroup per row, two passes over the row.
template <typename T, bool SAVED_RSTD>
__global__ __launch_bounds__(256) void rmsnorm_fwd_generic_kernel(
    const T* X, const void* __restrict__ W, int w_dt, T* Y /* may alias X */,
    float* __restrict__ RSTD, int64_t rows, int ncols, float eps) {
    __shared__ float red[4];
    __shared__ float s_rstd;
    const int64_t row = blockIdx.x;
    const T* x = X + row * ncols;
    float rstd;
    if (SAVED_RSTD) {
        rstd = RSTD[row];
    } else {
        float ss = 0.f;
        for (int c = threadIdx.x; c < ncols; c += 256) {
            float v = (float)x[c];
            ss += v * v;
        }
        ss = group_sum<64>(ss);
        if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = ss;
        __syncthreads();
        if (threadIdx.x == 0) {
            float t = (red[0] + red[1]) + (red[2] + red[3]);
            s_rstd = rsqrtf(t / (float)ncols + eps);
            RSTD[row] = s_rstd;
        }
        __syncthreads();
        rstd = s_rstd;
    }
    // In-place safe only per element: every element is re-read by the thread
    // that overwrites it, after the reduction above has finished.
    for (int c = threadIdx.x; c < ncols; c += 256) {
        float v = (float)x[c] * rstd;
        if (W != nullptr) {
            float w = w_dt == DT_F32   ? reinterpret_cast<const float*>(W)[c]
                      : w_dt == DT_BF16 ? (float)reinterpret_cast<const bf16*>(W)[c]
                                        : (float)reinterpret_cast<const f16*>(W)[c];
            v = round_to<T>(v) * w;
        }
        Y[row * ncols + c] = (T)v;
    }
}

// ---------------------------------------------------------------------------
// Backward: dx (+ old dx), optional y, dW partials.
// ---------------------------------------------------------------------------
template <typename T, int LPR, int MAXV, int THREADS>
__global__ __launch_bounds__(THREADS) void rmsnorm_bwd_kernel(
    const T* __restrict__ DY, const T* __restrict__ X, const void* __restrict__ W, int w_dt,
    const float* __restrict__ RSTD, T* __restrict__ DX, int accumulate_dx, T* __restrict__ YOUT,
    float* __restrict__ PARTIAL /* [gridDim.x][ncols] or null */, int64_t rows, int ncols,
    int iters) {
    constexpr int G = THREADS / LPR;
    extern __shared__ float smem[];  // [THREADS/64] reduction slots, then dW fold area
    float* red = smem;
    float* fold = smem + THREADS / 64;
    const int tid = threadIdx.x;
    const int g = tid / LPR;
    const int l = tid % LPR;
    const float inv_n = 1.0f / (float)ncols;
    const bool has_w = W != nullptr;

    float w[MAXV][8];
    float dw[MAXV][8];
#pragma unroll
    for (int v = 0; v < MAXV; ++v) {
        const int col = (v * LPR + l) * 8;
#pragma unroll
        for (int j = 0; j < 8; ++j) { w[v][j] = 1.f; dw[v][j] = 0.f; }
        if (has_w && col < ncols) load_w8(W, w_dt, col, w[v]);
    }

    // Raw 16-byte packs of the NEXT iteration's x, dy and (when accumulating) old dx are requested
    // before the current iteration is reduced, and the old dx together with x and dy rather than
    // after the row reduction: each of those was an exposed memory round trip in a kernel that
    // makes one or two iterations at small token counts.
    typedef typename VecOf<T>::type Pack;
    constexpr int PN = 8 / VecOf<T>::N;     // 16-byte packs per 8 elements
    Pack xr[MAXV][PN], dyr[MAXV][PN], oldr[MAXV][PN];
    auto fetch = [&](int it) {
        const int64_t row = ((int64_t)it * gridDim.x + blockIdx.x) * G + g;
        const bool ok = row < rows;
#pragma unroll
        for (int v = 0; v < MAXV; ++v) {
            const int col = (v * LPR + l) * 8;
            if (ok && col < ncols) {
#pragma unroll
                for (int q = 0; q < PN; ++q) {
                    xr[v][q] = *reinterpret_cast<const Pack*>(X + row * ncols + col + q * VecOf<T>::N);
                    dyr[v][q] = *reinterpret_cast<const Pack*>(DY + row * ncols + col + q * VecOf<T>::N);
                    if (accumulate_dx) oldr[v][q] = *reinterpret_cast<const Pack*>(DX + row * ncols + col + q * VecOf<T>::N);
                }
            }
        }
    };
    constexpr bool AHEAD = MAXV * PN <= 4;  // wider rows of 4-byte elements would spill: they fetch per iteration
    if (AHEAD && iters > 0) fetch(0);
    for (int it = 0; it < iters; ++it) {
        if (!AHEAD) fetch(it);
        const int64_t row = ((int64_t)it * gridDim.x + blockIdx.x) * G + g;
        const bool row_ok = row < rows;
        float x[MAXV][8], dy[MAXV][8];
        Pack old[MAXV][PN];                       // stays packed until it is added
        const float rstd = row_ok ? RSTD[row] : 0.f;
#pragma unroll
        for (int v = 0; v < MAXV; ++v) {
            const int col = (v * LPR + l) * 8;
            const bool ok = row_ok && col < ncols;
#pragma unroll
            for (int q = 0; q < PN; ++q)
#pragma unroll
                for (int e = 0; e < VecOf<T>::N; ++e) {
                    x[v][q * VecOf<T>::N + e] = ok ? (float)xr[v][q][e] : 0.f;
                    dy[v][q * VecOf<T>::N + e] = ok ? (float)dyr[v][q][e] : 0.f;
                }
#pragma unroll
            for (int q = 0; q < PN; ++q) old[v][q] = oldr[v][q];
        }
        if (AHEAD && it + 1 < iters) fetch(it + 1);
        float dot = 0.f;
#pragma unroll
        for (int v = 0; v < MAXV; ++v) {
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const float xh = x[v][j] * rstd;
                dw[v][j] += dy[v][j] * xh;           // unscaled dy (rmsnorm.py:305-307)
                x[v][j] = xh;
                dy[v][j] = dy[v][j] * w[v][j];        // dy_scaled
                dot += xh * dy[v][j];
            }
        }
        dot = row_sum<LPR>(dot, red, tid);
        const float k = dot * inv_n;
#pragma unroll
        for (int v = 0; v < MAXV; ++v) {
            const int col = (v * LPR + l) * 8;
            if (row_ok && col < ncols) {
                float dx[8];
#pragma unroll
                for (int j = 0; j < 8; ++j) dx[j] = rstd * (dy[v][j] - x[v][j] * k);
                if (accumulate_dx) {
#pragma unroll
                    for (int j = 0; j < 8; ++j) dx[j] = (float)old[v][j / VecOf<T>::N][j % VecOf<T>::N] + dx[j];
                }
                store8<T>(DX + row * ncols + col, dx);
                if (YOUT != nullptr) {
                    float y[8];
#pragma unroll
                    for (int j = 0; j < 8; ++j) y[j] = x[v][j] * w[v][j];  // fp32 product (rmsnorm.py:235)
                    store8<T>(YOUT + row * ncols + col, y);
                }
            }
        }
    }

    if (PARTIAL == nullptr) return;
    // Fold the G row-groups' dW registers pairwise through LDS.
    constexpr int PER_GROUP = LPR * MAXV * 8;
#pragma unroll 1
    for (int s = G / 2; s > 0; s >>= 1) {
        __syncthreads();
        if (g >= s && g < 2 * s) {
            float* dst = fold + (size_t)(g - s) * PER_GROUP;
#pragma unroll
            for (int v = 0; v < MAXV; ++v)
#pragma unroll
                for (int j = 0; j < 8; ++j) dst[(v * 8 + j) * LPR + l] = dw[v][j];
        }
        __syncthreads();
        if (g < s) {
            const float* src = fold + (size_t)g * PER_GROUP;
#pragma unroll
            for (int v = 0; v < MAXV; ++v)
#pragma unroll
                for (int j = 0; j < 8; ++j) dw[v][j] += src[(v * 8 + j) * LPR + l];
        }
    }
    if (g == 0) {
        float* out = PARTIAL + (size_t)blockIdx.x * ncols;
#pragma unroll
        for (int v = 0; v < MAXV; ++v) {
            const int col = (v * LPR + l) * 8;
            if (col < ncols) {
                float4* o = reinterpret_cast<float4*>(out + col);
                o[0] = make_float4(dw[v][0], dw[v][1], dw[v][2], dw[v][3]);
                o[1] = make_float4(dw[v][4], dw[v][5], dw[v][6], dw[v][7]);
            }
        }
    }
}

// dW[c] = (accumulate ? dW[c] : 0) + sum_b PARTIAL[b][c], b ascending per slice,
// slices folded in a fixed tree: deterministic for a given launch geometry.
template <typename TDW>
__global__ __launch_bounds__(256) void rmsnorm_dw_reduce_kernel(
    const float* __restrict__ PARTIAL, int nparts, int ncols, TDW* __restrict__ DWOUT,
    int accumulate) {
    __shared__ float sm[8][32];
    const int cl = threadIdx.x & 31;
    const int sl = threadIdx.x >> 5;  // 8 slices of the partial rows
    const int col = blockIdx.x * 32 + cl;
    float acc = 0.f;
    if (col < ncols) {
        // eight independent loads in flight per lane; the additions keep their fixed order
        int b = sl;
        for (; b + 56 < nparts; b += 64) {
            float t[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) t[u] = PARTIAL[(size_t)(b + 8 * u) * ncols + col];
#pragma unroll
            for (int u = 0; u < 8; ++u) acc += t[u];
        }
        for (; b < nparts; b += 8) acc += PARTIAL[(size_t)b * ncols + col];
    }
    sm[sl][cl] = acc;
    __syncthreads();
    if (sl == 0 && col < ncols) {
        float t = ((sm[0][cl] + sm[1][cl]) + (sm[2][cl] + sm[3][cl])) +
                  ((sm[4][cl] + sm[5][cl]) + (sm[6][cl] + sm[7][cl]));
        if (accumulate) t += (float)DWOUT[col];
        DWOUT[col] = (TDW)t;
    }
}

// Any-shape fallback backward: one workgroup per row for dx/y ...
template <typename T>
__global__ __launch_bounds__(256) void rmsnorm_bwd_generic_kernel(
    const T* __restrict__ DY, const T* __restrict__ X, const void* __restrict__ W, int w_dt,
    const float* __restrict__ RSTD, T* __restrict__ DX, int accumulate_dx, T* __restrict__ YOUT,
    int64_t rows, int ncols) {
    __shared__ float red[4];
    __shared__ float s_k;
    const int64_t row = blockIdx.x;
    const T* x = X + row * ncols;
    const T* dy = DY + row * ncols;
    const float rstd = RSTD[row];
    auto wload = [&](int c) -> float {
        if (W == nullptr) return 1.f;
        return w_dt == DT_F32   ? reinterpret_cast<const float*>(W)[c]
               : w_dt == DT_BF16 ? (float)reinterpret_cast<const bf16*>(W)[c]
                                 : (float)reinterpret_cast<const f16*>(W)[c];
    };
    float dot = 0.f;
    for (int c = threadIdx.x; c < ncols; c += 256)
        dot += ((float)x[c] * rstd) * ((float)dy[c] * wload(c));
    dot = group_sum<64>(dot);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = dot;
    __syncthreads();
    if (threadIdx.x == 0) s_k = ((red[0] + red[1]) + (red[2] + red[3])) / (float)ncols;
    __syncthreads();
    const float k = s_k;
    for (int c = threadIdx.x; c < ncols; c += 256) {
        const float xh = (float)x[c] * rstd;
        const float wv = wload(c);
        float dx = rstd * ((float)dy[c] * wv - xh * k);
        if (accumulate_dx) dx = (float)DX[row * ncols + c] + dx;
        DX[row * ncols + c] = (T)dx;
        if (YOUT != nullptr) YOUT[row * ncols + c] = (T)(xh * wv);
    }
}

// ... and one thread per column, rows ascending, for dW.
template <typename T, typename TDW>
__global__ __launch_bounds__(256) void rmsnorm_dw_generic_kernel(
    const T* __restrict__ DY, const T* __restrict__ X, const float* __restrict__ RSTD,
    TDW* __restrict__ DWOUT, int accumulate, int64_t rows, int ncols) {
    const int col = blockIdx.x * 256 + threadIdx.x;
    if (col >= ncols) return;
    float acc = 0.f;
    for (int64_t r = 0; r < rows; ++r)
        acc += (float)DY[r * ncols + col] * ((float)X[r * ncols + col] * RSTD[r]);
    if (accumulate) acc += (float)DWOUT[col];
    DWOUT[col] = (TDW)acc;
}

struct NormCfg { int lpr, maxv; };

static inline bool pick_cfg(int ncols, NormCfg& c) {
    if (ncols % 8 != 0 || ncols > 16384) return false;
    if (ncols <= 128) c = {16, 1};
    else if (ncols <= 256) c = {32, 1};
    else if (ncols <= 512) c = {64, 1};
    else if (ncols <= 1024) c = {64, 2};
    else if (ncols <= 2048) c = {256, 1};
    else if (ncols <= 4096) c = {256, 2};
    else if (ncols <= 8192) c = {256, 4};
    else c = {256, 8};
    return true;
}

// Backward workgroup size per config: wide rows keep many registers per lane,
// so they get fewer waves per workgroup.
static inline int bwd_threads(const NormCfg& c) {
    if (c.maxv == 1) return 1024;
    if (c.maxv <= 4) return 512;     // two packs per lane and the next iteration's requests need 256 registers
    return 256;
}

constexpr int kBwdMaxBlocks = 256;  // one workgroup per CU; bounds the dW partial buffer

static inline int bwd_grid(int64_t rows, int groups) {
    int64_t need = (rows + groups - 1) / groups;
    if (need < 1) need = 1;
    return (int)(need < kBwdMaxBlocks ? need : kBwdMaxBlocks);
}

template <typename T, bool SAVED>
static int launch_fwd(const void* x, const void* w, int w_dt, void* y, float* rstd, int64_t rows,
                      int ncols, float eps, hipStream_t s) {
    NormCfg c;
    const bool vec = pick_cfg(ncols, c) && aligned16(x) && aligned16(y) &&
                     (w == nullptr || aligned16(w));
    const T* X = reinterpret_cast<const T*>(x);
    T* Y = reinterpret_cast<T*>(y);
    if (!vec) {
        rmsnorm_fwd_generic_kernel<T, SAVED><<<dim3((unsigned)rows), 256, 0, s>>>(X, w, w_dt, Y, rstd, rows, ncols, eps);
        return 0;
    }
#define FX_FWD_CASE(L, V)                                                                         \
    if (c.lpr == L && c.maxv == V) {                                                              \
        constexpr int G = 256 / L;                                                                \
        const unsigned grid = (unsigned)((rows + G - 1) / G);                                     \
        rmsnorm_fwd_kernel<T, L, V, 256, SAVED><<<grid, 256, 0, s>>>(X, w, w_dt, Y, rstd, rows, ncols, eps); \
        return 0;                                                                                 \
    }
    FX_FWD_CASE(16, 1) FX_FWD_CASE(32, 1) FX_FWD_CASE(64, 1) FX_FWD_CASE(64, 2)
    FX_FWD_CASE(256, 1) FX_FWD_CASE(256, 2) FX_FWD_CASE(256, 4) FX_FWD_CASE(256, 8)
#undef FX_FWD_CASE
    return -1;
}

template <typename T>
static int launch_bwd(const void* dy, const void* x, const void* w, int w_dt, const float* rstd,
                      void* dx, int acc_dx, void* yout, float* partial, int nblocks, int64_t rows,
                      int ncols, const NormCfg& c, hipStream_t s) {
    const T* DY = reinterpret_cast<const T*>(dy);
    const T* X = reinterpret_cast<const T*>(x);
    T* DX = reinterpret_cast<T*>(dx);
    T* Y = reinterpret_cast<T*>(yout);
#define FX_BWD_CASE(L, V, TH)                                                                     \
    if (c.lpr == L && c.maxv == V) {                                                              \
        constexpr int G = TH / L;                                                                 \
        const int iters = (int)((rows + (int64_t)nblocks * G - 1) / ((int64_t)nblocks * G));      \
        const size_t lds = sizeof(float) * (TH / 64 + (size_t)(G / 2) * L * V * 8);               \
        rmsnorm_bwd_kernel<T, L, V, TH><<<nblocks, TH, lds, s>>>(DY, X, w, w_dt, rstd, DX, acc_dx, Y, partial, rows, ncols, iters); \
        return 0;                                                                                 \
    }
    FX_BWD_CASE(16, 1, 1024) FX_BWD_CASE(32, 1, 1024) FX_BWD_CASE(64, 1, 1024) FX_BWD_CASE(64, 2, 512)
    FX_BWD_CASE(256, 1, 1024) FX_BWD_CASE(256, 2, 512) FX_BWD_CASE(256, 4, 512) FX_BWD_CASE(256, 8, 256)
#undef FX_BWD_CASE
    return -1;
}

}  // namespace fx

using namespace fx;

extern "C" int fx_rmsnorm_fwd(const void* x, const void* w, void* y, float* rstd, int64_t rows,
                              int ncols, float eps, int x_dt, int w_dt, int use_saved_rstd,
                              hipStream_t stream) {
    if (rows < 0 || ncols <= 0) FX_FAIL("fx_rmsnorm_fwd: bad shape rows=%lld ncols=%d", (long long)rows, ncols);
    if (rows == 0) return 0;
    if (!x || !y || !rstd) FX_FAIL("fx_rmsnorm_fwd: null pointer");
    int rc = -1;
    FX_DISPATCH_DTYPE(x_dt, T,
        rc = use_saved_rstd ? launch_fwd<T, true>(x, w, w_dt, y, rstd, rows, ncols, eps, stream)
                            : launch_fwd<T, false>(x, w, w_dt, y, rstd, rows, ncols, eps, stream));
    if (rc != 0) FX_FAIL("fx_rmsnorm_fwd: no kernel for ncols=%d", ncols);
    FX_CHECK_LAUNCH("fx_rmsnorm_fwd");
    return 0;
}

extern "C" size_t fx_rmsnorm_bwd_ws_bytes(int64_t rows, int ncols) {
    NormCfg c;
    if (!pick_cfg(ncols, c)) return 0;
    const int groups = bwd_threads(c) / c.lpr;
    return (size_t)bwd_grid(rows, groups) * (size_t)ncols * sizeof(float);
}

extern "C" int fx_rmsnorm_bwd(const void* dy, const void* x, const void* w, const float* rstd,
                              void* dx, int accumulate_dx, void* dw, int dw_dt, int accumulate_dw,
                              void* y_out, int64_t rows, int ncols, int x_dt, int w_dt,
                              float* ws, size_t ws_bytes, hipStream_t stream) {
    if (rows < 0 || ncols <= 0) FX_FAIL("fx_rmsnorm_bwd: bad shape rows=%lld ncols=%d", (long long)rows, ncols);
    if (rows == 0) return 0;
    if (!dy || !x || !rstd || !dx) FX_FAIL("fx_rmsnorm_bwd: null pointer");
    const bool want_dw = (w != nullptr && dw != nullptr);
    NormCfg c;
    bool vec = pick_cfg(ncols, c) && aligned16(dy) && aligned16(x) && aligned16(dx) &&
               (y_out == nullptr || aligned16(y_out)) && (w == nullptr || aligned16(w));
    if (vec && want_dw) {
        const size_t need = fx_rmsnorm_bwd_ws_bytes(rows, ncols);
        if (ws == nullptr || ws_bytes < need)
            FX_FAIL("fx_rmsnorm_bwd: workspace too small (%zu < %zu bytes)", ws_bytes, need);
    }
    if (!vec) {
        FX_DISPATCH_DTYPE(x_dt, T,
            rmsnorm_bwd_generic_kernel<T><<<dim3((unsigned)rows), 256, 0, stream>>>(
                reinterpret_cast<const T*>(dy), reinterpret_cast<const T*>(x), w, w_dt, rstd,
                reinterpret_cast<T*>(dx), accumulate_dx, reinterpret_cast<T*>(y_out), rows, ncols));
        FX_CHECK_LAUNCH("fx_rmsnorm_bwd(generic dx)");
        if (want_dw) {
            const unsigned grid = (unsigned)((ncols + 255) / 256);
            FX_DISPATCH_DTYPE(x_dt, T,
                FX_DISPATCH_DTYPE(dw_dt, TDW,
                    rmsnorm_dw_generic_kernel<T, TDW><<<grid, 256, 0, stream>>>(
                        reinterpret_cast<const T*>(dy), reinterpret_cast<const T*>(x), rstd,
                        reinterpret_cast<TDW*>(dw), accumulate_dw, rows, ncols)));
            FX_CHECK_LAUNCH("fx_rmsnorm_bwd(generic dw)");
        }
        return 0;
    }
    const int groups = bwd_threads(c) / c.lpr;
    const int nblocks = bwd_grid(rows, groups);
    int rc = -1;
    FX_DISPATCH_DTYPE(x_dt, T,
        rc = launch_bwd<T>(dy, x, w, w_dt, rstd, dx, accumulate_dx, y_out, want_dw ? ws : nullptr,
                           nblocks, rows, ncols, c, stream));
    if (rc != 0) FX_FAIL("fx_rmsnorm_bwd: no kernel for ncols=%d", ncols);
    FX_CHECK_LAUNCH("fx_rmsnorm_bwd");
    if (want_dw) {
        const unsigned grid = (unsigned)((ncols + 31) / 32);
        FX_DISPATCH_DTYPE(dw_dt, TDW,
            rmsnorm_dw_reduce_kernel<TDW><<<grid, 256, 0, stream>>>(
                ws, nblocks, ncols, reinterpret_cast<TDW*>(dw), accumulate_dw));
        FX_CHECK_LAUNCH("fx_rmsnorm_bwd(dw reduce)");
    }
    return 0;
}
