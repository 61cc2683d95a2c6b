// Gated activations (SwiGLU, gated GELU-tanh), forward and backward, gfx950.
//
// out = act(x1) * x3, x1 = gate, x3 = up/value.  Math follows the reference
// Triton kernels: flextrain/ops/_kernels/swiglu.py:9-96 and
// flextrain/ops/_kernels/gelu_tanh_gated.py:55-140.  Pure streaming kernels:
// every lane moves 16 bytes per tensor per access, one pack per lane.
#include "common.h"
#include "flexhip.h"

namespace fx {

template <typename T, int ACT>
FX_DEV void glu_bwd_elem(float x1, float x3, float dout, float& dx1, float& dx3, float& act) {
    if (ACT == ACT_SILU) {
        const float s = fast_sigmoid(x1);
        const float a = x1 * s;
        act = a * x3;
        dx3 = dout * a;
        const float ds = s * (1.0f + x1 * (1.0f - s));
        // The reference multiplies dout*x3 in the storage dtype before the fp32
        // factor (swiglu.py:92); reproduce that one rounding.
        dx1 = round_to<T>(dout * x3) * ds;
    } else {
        const float sq = x1 * x1;
        const float cu = sq * x1;
        const float u = 0.7978845608028654f * (x1 + 0.044715f * cu);
        const float th = 2.0f * fast_sigmoid(2.0f * u) - 1.0f;
        const float opt = 1.0f + th;
        const float g = 0.5f * x1 * opt;
        act = g * x3;
        dx3 = dout * g;
        const float du = 0.7978845608028654f * (1.0f + 3.0f * 0.044715f * sq);
        const float sech = 1.0f - th * th;
        const float dg = 0.5f * opt + 0.5f * x1 * sech * du;
        dx1 = dout * x3 * dg;
    }
}

// Workgroup size and packs of 8 elements per lane, from a sweep at the [8192, 14336] bf16 shape:
// one pack per lane beats two or four; the forward kernel (two input streams) is fastest with
// 512 lanes (6.06 TB/s against 5.68 at 256 x 2), the backward kernel (three input, two or three
// output streams) with 1024 (6.20 TB/s against 5.86).
constexpr int GLU_FWD_THREADS = 512;
constexpr int GLU_BWD_THREADS = 1024;
constexpr int GLU_THREADS = 512;  // SiLU backward
constexpr int GLU_UNROLL = 1;

template <typename T, typename TO, int ACT, bool NT>
__global__ __launch_bounds__(GLU_FWD_THREADS) void glu_fwd_kernel(
    const T* __restrict__ X1, const T* __restrict__ X3, TO* __restrict__ OUT, int64_t n) {
    const int64_t base = ((int64_t)blockIdx.x * GLU_UNROLL) * GLU_FWD_THREADS * 8;
    float a[GLU_UNROLL][8], b[GLU_UNROLL][8];
    bool full[GLU_UNROLL];
#pragma unroll
    for (int u = 0; u < GLU_UNROLL; ++u) {
        const int64_t off = base + ((int64_t)u * GLU_FWD_THREADS + threadIdx.x) * 8;
        full[u] = off + 8 <= n;
        if (full[u]) {
            load_f32<T, 8, NT>(X1 + off, a[u]);
            load_f32<T, 8, NT>(X3 + off, b[u]);
        }
    }
#pragma unroll
    for (int u = 0; u < GLU_UNROLL; ++u) {
        const int64_t off = base + ((int64_t)u * GLU_FWD_THREADS + threadIdx.x) * 8;
        if (full[u]) {
            float o[8];
#pragma unroll
            for (int j = 0; j < 8; ++j) o[j] = glu_fwd_elem<T, ACT>(a[u][j], b[u][j]);
            store_f32<TO, 8, NT>(OUT + off, o);
        } else {
            for (int64_t i = off; i < n && i < off + 8; ++i)
                OUT[i] = (TO)glu_fwd_elem<T, ACT>((float)X1[i], (float)X3[i]);
        }
    }
}

template <typename T, int ACT, bool STORE_ACT, bool NT>
__global__ __launch_bounds__(GLU_BWD_THREADS) void glu_bwd_kernel(
    const T* __restrict__ X1, const T* __restrict__ X3, const T* __restrict__ DOUT,
    T* __restrict__ DX1, T* __restrict__ DX3, T* __restrict__ ACTOUT, int64_t n) {
    const int64_t base = ((int64_t)blockIdx.x * GLU_UNROLL) * GLU_BWD_THREADS * 8;
    float a[GLU_UNROLL][8], b[GLU_UNROLL][8], d[GLU_UNROLL][8];
    bool full[GLU_UNROLL];
#pragma unroll
    for (int u = 0; u < GLU_UNROLL; ++u) {
        const int64_t off = base + ((int64_t)u * GLU_BWD_THREADS + threadIdx.x) * 8;
        full[u] = off + 8 <= n;
        if (full[u]) {
            load_f32<T, 8, NT>(X1 + off, a[u]);
            load_f32<T, 8, NT>(X3 + off, b[u]);
            load_f32<T, 8, NT>(DOUT + off, d[u]);
        }
    }
#pragma unroll
    for (int u = 0; u < GLU_UNROLL; ++u) {
        const int64_t off = base + ((int64_t)u * GLU_BWD_THREADS + threadIdx.x) * 8;
        if (full[u]) {
            float g1[8], g3[8], ac[8];
#pragma unroll
            for (int j = 0; j < 8; ++j)
                glu_bwd_elem<T, ACT>(a[u][j], b[u][j], d[u][j], g1[j], g3[j], ac[j]);
            store_f32<T, 8, NT>(DX1 + off, g1);
            store_f32<T, 8, NT>(DX3 + off, g3);
            if (STORE_ACT) store_f32<T, 8, NT>(ACTOUT + off, ac);
        } else {
            for (int64_t i = off; i < n && i < off + 8; ++i) {
                float g1, g3, ac;
                glu_bwd_elem<T, ACT>((float)X1[i], (float)X3[i], (float)DOUT[i], g1, g3, ac);
                DX1[i] = (T)g1;
                DX3[i] = (T)g3;
                if (STORE_ACT) ACTOUT[i] = (T)ac;
            }
        }
    }
}

// d/dz silu(z) * dout = dout * s * (1 + z * (1 - s)), s = sigmoid(z)  (flextrain/ops/_kernels/silu_bwd.py:16-35).
template <typename T, bool NT>
__global__ __launch_bounds__(GLU_THREADS) void silu_bwd_kernel(const T* Z, const T* DOUT, T* DIN /* may alias Z or DOUT */, int64_t n,
                                                               bool vec) {
    if (vec) {
        const int64_t off = ((int64_t)blockIdx.x * GLU_THREADS + threadIdx.x) * 8;
        if (off + 8 <= n) {
            float z[8], d[8], o[8];
            load_f32<T, 8, NT>(Z + off, z);
            load_f32<T, 8, NT>(DOUT + off, d);
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const float sg = fast_sigmoid(z[j]);
                o[j] = d[j] * (sg * (1.0f + z[j] * (1.0f - sg)));
            }
            store_f32<T, 8, NT>(DIN + off, o);
            return;
        }
        for (int64_t i = off; i < n; ++i) {
            const float zz = (float)Z[i], sg = fast_sigmoid(zz);
            DIN[i] = (T)((float)DOUT[i] * (sg * (1.0f + zz * (1.0f - sg))));
        }
    } else {
        for (int64_t i = ((int64_t)blockIdx.x * GLU_THREADS + threadIdx.x) * 8, e = i + 8; i < n && i < e; ++i) {
            const float zz = (float)Z[i], sg = fast_sigmoid(zz);
            DIN[i] = (T)((float)DOUT[i] * (sg * (1.0f + zz * (1.0f - sg))));
        }
    }
}

// Unaligned-pointer fallback: one element per lane.
template <typename T, typename TO, int ACT>
__global__ __launch_bounds__(256) void glu_fwd_scalar_kernel(const T* X1, const T* X3, TO* OUT, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n) OUT[i] = (TO)glu_fwd_elem<T, ACT>((float)X1[i], (float)X3[i]);
}
template <typename T, int ACT>
__global__ __launch_bounds__(256) void glu_bwd_scalar_kernel(const T* X1, const T* X3, const T* DOUT,
                                                             T* DX1, T* DX3, T* ACTOUT, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n) {
        float g1, g3, ac;
        glu_bwd_elem<T, ACT>((float)X1[i], (float)X3[i], (float)DOUT[i], g1, g3, ac);
        DX1[i] = (T)g1;
        DX3[i] = (T)g3;
        if (ACTOUT) ACTOUT[i] = (T)ac;
    }
}

template <typename T, typename TO, int ACT>
static void launch_glu_fwd(const void* x1, const void* x3, void* out, int64_t n, hipStream_t s) {
    const T* a = reinterpret_cast<const T*>(x1);
    const T* b = reinterpret_cast<const T*>(x3);
    TO* o = reinterpret_cast<TO*>(out);
    if (aligned16(x1) && aligned16(x3) && aligned16(out)) {
        const int64_t per_block = (int64_t)GLU_UNROLL * GLU_FWD_THREADS * 8;
        const unsigned grid = (unsigned)((n + per_block - 1) / per_block);
        if ((size_t)n * (2 * sizeof(T) + sizeof(TO)) >= kStreamingBytes)
            glu_fwd_kernel<T, TO, ACT, true><<<grid, GLU_FWD_THREADS, 0, s>>>(a, b, o, n);
        else
            glu_fwd_kernel<T, TO, ACT, false><<<grid, GLU_FWD_THREADS, 0, s>>>(a, b, o, n);
    } else {
        glu_fwd_scalar_kernel<T, TO, ACT><<<(unsigned)((n + 255) / 256), 256, 0, s>>>(a, b, o, n);
    }
}

template <typename T, int ACT>
static void launch_glu_bwd(const void* x1, const void* x3, const void* dout, void* dx1, void* dx3,
                           void* act, int64_t n, hipStream_t s) {
    const T* a = reinterpret_cast<const T*>(x1);
    const T* b = reinterpret_cast<const T*>(x3);
    const T* d = reinterpret_cast<const T*>(dout);
    T* g1 = reinterpret_cast<T*>(dx1);
    T* g3 = reinterpret_cast<T*>(dx3);
    T* ac = reinterpret_cast<T*>(act);
    if (aligned16(x1) && aligned16(x3) && aligned16(dout) && aligned16(dx1) && aligned16(dx3) &&
        (act == nullptr || aligned16(act))) {
        const int64_t per_block = (int64_t)GLU_UNROLL * GLU_BWD_THREADS * 8;
        const unsigned grid = (unsigned)((n + per_block - 1) / per_block);
        const bool nt = (size_t)n * 5 * sizeof(T) >= kStreamingBytes;
        if (act && nt) glu_bwd_kernel<T, ACT, true, true><<<grid, GLU_BWD_THREADS, 0, s>>>(a, b, d, g1, g3, ac, n);
        else if (act) glu_bwd_kernel<T, ACT, true, false><<<grid, GLU_BWD_THREADS, 0, s>>>(a, b, d, g1, g3, ac, n);
        else if (nt) glu_bwd_kernel<T, ACT, false, true><<<grid, GLU_BWD_THREADS, 0, s>>>(a, b, d, g1, g3, ac, n);
        else glu_bwd_kernel<T, ACT, false, false><<<grid, GLU_BWD_THREADS, 0, s>>>(a, b, d, g1, g3, ac, n);
    } else {
        glu_bwd_scalar_kernel<T, ACT><<<(unsigned)((n + 255) / 256), 256, 0, s>>>(a, b, d, g1, g3, ac, n);
    }
}

}  // namespace fx

using namespace fx;

extern "C" int fx_glu_fwd(const void* x1, const void* x3, void* out, int64_t n, int in_dt,
                          int out_dt, int act, hipStream_t stream) {
    if (n < 0) FX_FAIL("fx_glu_fwd: negative element count");
    if (n == 0) return 0;
    if (!x1 || !x3 || !out) FX_FAIL("fx_glu_fwd: null pointer");
    if (act != ACT_SILU && act != ACT_GELU_TANH) FX_FAIL("fx_glu_fwd: unknown activation %d", act);
    FX_DISPATCH_DTYPE(in_dt, T,
        FX_DISPATCH_DTYPE(out_dt, TO,
            if (act == ACT_SILU) launch_glu_fwd<T, TO, ACT_SILU>(x1, x3, out, n, stream);
            else launch_glu_fwd<T, TO, ACT_GELU_TANH>(x1, x3, out, n, stream)));
    FX_CHECK_LAUNCH("fx_glu_fwd");
    return 0;
}

extern "C" int fx_glu_bwd(const void* x1, const void* x3, const void* dout, void* dx1, void* dx3,
                          void* act_out, int64_t n, int dt, int act, hipStream_t stream) {
    if (n < 0) FX_FAIL("fx_glu_bwd: negative element count");
    if (n == 0) return 0;
    if (!x1 || !x3 || !dout || !dx1 || !dx3) FX_FAIL("fx_glu_bwd: null pointer");
    if (act != ACT_SILU && act != ACT_GELU_TANH) FX_FAIL("fx_glu_bwd: unknown activation %d", act);
    FX_DISPATCH_DTYPE(dt, T,
        if (act == ACT_SILU) launch_glu_bwd<T, ACT_SILU>(x1, x3, dout, dx1, dx3, act_out, n, stream);
        else launch_glu_bwd<T, ACT_GELU_TANH>(x1, x3, dout, dx1, dx3, act_out, n, stream));
    FX_CHECK_LAUNCH("fx_glu_bwd");
    return 0;
}

extern "C" int fx_silu_bwd(const void* z, const void* dout, void* din, int64_t n, int dt, hipStream_t stream) {
    if (n < 0) FX_FAIL("fx_silu_bwd: negative element count");
    if (n == 0) return 0;
    if (!z || !dout || !din) FX_FAIL("fx_silu_bwd: null pointer");
    const bool vec = aligned16(z) && aligned16(dout) && aligned16(din);
    const unsigned grid = (unsigned)((n + (int64_t)GLU_THREADS * 8 - 1) / ((int64_t)GLU_THREADS * 8));
    FX_DISPATCH_DTYPE(dt, T,
        if ((size_t)n * 3 * sizeof(T) >= kStreamingBytes && din != z && din != dout)
            silu_bwd_kernel<T, true><<<grid, GLU_THREADS, 0, stream>>>(reinterpret_cast<const T*>(z), reinterpret_cast<const T*>(dout), reinterpret_cast<T*>(din), n, vec);
        else
            silu_bwd_kernel<T, false><<<grid, GLU_THREADS, 0, stream>>>(reinterpret_cast<const T*>(z), reinterpret_cast<const T*>(dout), reinterpret_cast<T*>(din), n, vec));
    FX_CHECK_LAUNCH("fx_silu_bwd");
    return 0;
}
