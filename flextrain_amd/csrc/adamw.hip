// Decoupled-weight-decay Adam step on one flat parameter chunk, gfx950.
//
// Update order and fp32 arithmetic follow the reference Triton kernel
// (flextrain/ops/_kernels/adamw.py:34-60):
//   p -= (lr*wd)*p;  m = b1*m + (1-b1)*g;  v = b2*v + (1-b2)*g*g;
//   p -= lr * ((m/bc1) / (sqrt(v/bc2) + eps))
// with bc1/bc2 = 1 - beta^step computed by the host in double and passed as
// fp32.  p, m, v are updated in place in whatever dtype each buffer has.
// An optional extra output receives the updated parameter rounded to bf16 (the
// compute-dtype copy a host-offloaded fp32 master needs); it has no
// counterpart in the reference kernel.
#include "common.h"
#include "flexhip.h"

namespace fx {

constexpr int ADAM_THREADS = 512;  // 512 lanes measured 1.7 % faster than 256 or 1024

struct AdamScalars {
    float lr_wd, lr, beta1, omb1, beta2, omb2, eps, bc1, bc2;
};

FX_DEV void adam_elem(float& p, float g, float& m, float& v, const AdamScalars& a) {
    p = p - a.lr_wd * p;
    m = a.beta1 * m + a.omb1 * g;
    v = a.beta2 * v + a.omb2 * (g * g);
    const float mh = m / a.bc1;
    const float vh = v / a.bc2;
    const float denom = sqrtf(vh) + a.eps;
    p = p - a.lr * (mh / denom);
}

// N consecutive elements of T (N * sizeof(T) = 8 or 16 bytes, address aligned to that) <-> fp32 registers.
template <typename T, int N, bool NT>
FX_DEV void load_n(const T* __restrict__ p, float (&out)[N]) {
    typedef T V __attribute__((ext_vector_type(N)));
    V v;
    if (NT) v = __builtin_nontemporal_load(reinterpret_cast<const V*>(p));
    else v = *reinterpret_cast<const V*>(p);
#pragma unroll
    for (int j = 0; j < N; ++j) out[j] = (float)v[j];
}
template <typename T, int N, bool NT>
FX_DEV void store_n(T* __restrict__ p, const float (&in)[N]) {
    typedef T V __attribute__((ext_vector_type(N)));
    V v;
#pragma unroll
    for (int j = 0; j < N; ++j) v[j] = (T)in[j];
    if (NT) __builtin_nontemporal_store(v, reinterpret_cast<V*>(p));
    else *reinterpret_cast<V*>(p) = v;
}

// A lane owns UNROLL groups of N consecutive elements, N = 4 when any buffer is fp32 (16-byte
// accesses to the fp32 buffers, 8-byte ones to 2-byte buffers) and 8 when all are 2-byte.  Lanes of
// a wave touch consecutive groups, so every load or store instruction of a wave covers one
// contiguous 512- or 1024-byte run (with 8 fp32 elements per lane each instruction would touch
// every other 16 bytes).
template <typename TP, typename TG, typename TS, bool COPY, bool NT, int UNROLL, int N>
__global__ __launch_bounds__(ADAM_THREADS) void adamw_kernel(
    TP* __restrict__ P, const TG* __restrict__ G, TS* __restrict__ M, TS* __restrict__ V,
    bf16* __restrict__ PCOPY, int64_t n, AdamScalars a) {
    const int64_t base = (int64_t)blockIdx.x * ADAM_THREADS * N * UNROLL;
    float p[UNROLL][N], g[UNROLL][N], m[UNROLL][N], v[UNROLL][N];
    bool full[UNROLL];
    // NT (launches that move more than the caches keep): every access is non-temporal.  On the
    // 218 M-parameter chunk that is 5.75-5.8 TB/s against 5.5 TB/s with plain accesses; it only pays
    // with whole-run accesses (when an instruction touched every other 16 bytes, the other halves
    // of the lines were fetched from L2 a second time and non-temporal was the slower variant).
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
        const int64_t off = base + ((int64_t)u * ADAM_THREADS + threadIdx.x) * N;
        full[u] = off + N <= n;
        if (full[u]) {
            load_n<TP, N, NT>(P + off, p[u]);
            load_n<TG, N, NT>(G + off, g[u]);
            load_n<TS, N, NT>(M + off, m[u]);
            load_n<TS, N, NT>(V + off, v[u]);
        }
    }
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
        const int64_t off = base + ((int64_t)u * ADAM_THREADS + threadIdx.x) * N;
        if (full[u]) {
#pragma unroll
            for (int j = 0; j < N; ++j) adam_elem(p[u][j], g[u][j], m[u][j], v[u][j], a);
            store_n<TP, N, NT>(P + off, p[u]);
            store_n<TS, N, NT>(M + off, m[u]);
            store_n<TS, N, NT>(V + off, v[u]);
            if (COPY) store_n<bf16, N, NT>(PCOPY + off, p[u]);
        } else {
            for (int64_t i = off; i < n && i < off + N; ++i) {
                float pp = (float)P[i], gg = (float)G[i], mm = (float)M[i], vv = (float)V[i];
                adam_elem(pp, gg, mm, vv, a);
                P[i] = (TP)pp;
                M[i] = (TS)mm;
                V[i] = (TS)vv;
                if (COPY) PCOPY[i] = (bf16)pp;
            }
        }
    }
}

// flag[0] |= 1 if any element is NaN or +-Inf.
template <typename T>
__global__ __launch_bounds__(256) void nonfinite_kernel(const T* __restrict__ X, int64_t n,
                                                        int* __restrict__ flag) {
    int bad = 0;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (int64_t)gridDim.x * 256) {
        const float v = (float)X[i];
        bad |= !(fabsf(v) <= 3.402823466e38f);
    }
    if (__any(bad) && (threadIdx.x & 63) == 0) atomicOr(flag, 1);
}

template <typename TP, typename TG, typename TS>
static void launch_adamw(void* p, const void* g, void* m, void* v, void* pcopy, int64_t n,
                         const AdamScalars& a, hipStream_t s) {
    TP* P = reinterpret_cast<TP*>(p);
    const TG* G = reinterpret_cast<const TG*>(g);
    TS* M = reinterpret_cast<TS*>(m);
    TS* V = reinterpret_cast<TS*>(v);
    bf16* C = reinterpret_cast<bf16*>(pcopy);
    const bool nt = (size_t)n * (2 * sizeof(TP) + sizeof(TG) + 4 * sizeof(TS)) >= kStreamingBytes;
    constexpr int N = (sizeof(TP) == 4 || sizeof(TG) == 4 || sizeof(TS) == 4) ? 4 : 8;
#define GO(U) { const int64_t per = (int64_t)ADAM_THREADS * N * U; const unsigned grid = (unsigned)((n + per - 1) / per); \
    if (pcopy && nt) adamw_kernel<TP, TG, TS, true, true, U, N><<<grid, ADAM_THREADS, 0, s>>>(P, G, M, V, C, n, a); \
    else if (pcopy) adamw_kernel<TP, TG, TS, true, false, U, N><<<grid, ADAM_THREADS, 0, s>>>(P, G, M, V, C, n, a); \
    else if (nt) adamw_kernel<TP, TG, TS, false, true, U, N><<<grid, ADAM_THREADS, 0, s>>>(P, G, M, V, C, n, a); \
    else adamw_kernel<TP, TG, TS, false, false, U, N><<<grid, ADAM_THREADS, 0, s>>>(P, G, M, V, C, n, a); }
    GO(1)
#undef GO
}

}  // namespace fx

using namespace fx;

extern "C" int fx_adamw_step(void* p, const void* g, void* m, void* v, void* p_bf16_out, int64_t n,
                             int p_dt, int g_dt, int state_dt, float lr, float beta1, float beta2,
                             float eps, float weight_decay, float bias_correction1,
                             float bias_correction2, hipStream_t stream) {
    if (n < 0) FX_FAIL("fx_adamw_step: negative element count");
    if (n == 0) return 0;
    if (!p || !g || !m || !v) FX_FAIL("fx_adamw_step: null pointer");
    if (!aligned16(p) || !aligned16(g) || !aligned16(m) || !aligned16(v) ||
        (p_bf16_out && !aligned16(p_bf16_out)))
        FX_FAIL("fx_adamw_step: buffers must be 16-byte aligned");
    AdamScalars a;
    a.lr_wd = lr * weight_decay;
    a.lr = lr;
    a.beta1 = beta1;
    a.omb1 = 1.0f - beta1;
    a.beta2 = beta2;
    a.omb2 = 1.0f - beta2;
    a.eps = eps;
    a.bc1 = bias_correction1;
    a.bc2 = bias_correction2;
    FX_DISPATCH_DTYPE(p_dt, TP,
        FX_DISPATCH_DTYPE(g_dt, TG,
            FX_DISPATCH_DTYPE(state_dt, TS,
                launch_adamw<TP, TG, TS>(p, g, m, v, p_bf16_out, n, a, stream))));
    FX_CHECK_LAUNCH("fx_adamw_step");
    return 0;
}

extern "C" int fx_nonfinite_flag(const void* x, int64_t n, int dt, int* flag, hipStream_t stream) {
    if (n < 0 || !flag) FX_FAIL("fx_nonfinite_flag: bad arguments");
    if (n == 0) return 0;
    int64_t blocks = (n + 255) / 256;
    if (blocks > 2048) blocks = 2048;
    FX_DISPATCH_DTYPE(dt, T,
        nonfinite_kernel<T><<<(unsigned)blocks, 256, 0, stream>>>(reinterpret_cast<const T*>(x), n, flag));
    FX_CHECK_LAUNCH("fx_nonfinite_flag");
    return 0;
}
