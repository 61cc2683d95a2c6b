// MoE data movement and the per-row expert activation, gfx950.
//
// Reference semantics: flextrain/ops/_kernels/moe.py
//   :508-543 moe_scatter_kernel        out[idx[t,k], :] = x[t, :] (* scale[t,k])
//   :546-557 moe_scatter_routing_weights_kernel   out[idx[i]] = w[i]
//   :560-598 moe_gather_kernel         out[t] = residual[t] + sum_k w[t,k] * y[idx[t,k]]  (fp32, k ascending)
//   :29-74   swiglu_fwd_weighted_kernel     packed row [value | gate] -> silu(gate) * value (* w)
//   :77-145  swiglu_bwd_weighted_kernel     and :148-215 the pre-scaled variant
// Rows are moved with 16-byte accesses; one workgroup owns a token (scatter,
// gather) and one wave owns a row (activation), so no cross-wave reduction.
#include "common.h"
#include "flexhip.h"

namespace fx {

// Entry i of an index mapping, clamped to [0, rows): a mapping that is no permutation of the routed
// rows (a caller's own, or one made from expert ids outside the range) moves the wrong rows, never
// an address outside the buffers.
FX_DEV int64_t load_index(const void* idx, int is64, int64_t i, int64_t rows) {
    const int64_t r = is64 ? reinterpret_cast<const int64_t*>(idx)[i] : (int64_t)reinterpret_cast<const int32_t*>(idx)[i];
    return r < 0 ? 0 : (r < rows ? r : rows - 1);
}

// ------------------------------------------------------------------ scatter
template <typename T, typename TS, bool HAS_SCALE>
__global__ __launch_bounds__(256) void moe_scatter_kernel(
    const T* __restrict__ X, T* __restrict__ OUT, const void* __restrict__ IDX, int idx64,
    const TS* __restrict__ SCALE, int64_t Tn, int D, int K, int64_t out_stride, int tok_per_block,
    bool vec) {
    const int tpt = 256 / tok_per_block;
    const int64_t t = (int64_t)blockIdx.x * tok_per_block + threadIdx.x / tpt;
    const int lane = threadIdx.x % tpt;
    if (t >= Tn) return;
    if (vec) {
        for (int c = lane * 8; c < D; c += tpt * 8) {
            float v[8];
            load_f32<T, 8>(X + t * D + c, v);
            for (int k = 0; k < K; ++k) {
                const int64_t row = load_index(IDX, idx64, t * K + k, Tn * K);
                if (HAS_SCALE) {
                    const float s = (float)SCALE[t * K + k];
                    float o[8];
#pragma unroll
                    for (int j = 0; j < 8; ++j) o[j] = v[j] * s;
                    store_f32<T, 8>(OUT + row * out_stride + c, o);
                } else {
                    store_f32<T, 8>(OUT + row * out_stride + c, v);
                }
            }
        }
    } else {
        for (int c = lane; c < D; c += tpt) {
            const float v = (float)X[t * D + c];
            for (int k = 0; k < K; ++k) {
                const int64_t row = load_index(IDX, idx64, t * K + k, Tn * K);
                OUT[row * out_stride + c] = HAS_SCALE ? (T)(v * (float)SCALE[t * K + k]) : X[t * D + c];
            }
        }
    }
}

template <typename T>
__global__ __launch_bounds__(256) void moe_scatter_weights_kernel(const T* __restrict__ W,
                                                                  const void* __restrict__ IDX, int idx64,
                                                                  T* __restrict__ OUT, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n) OUT[load_index(IDX, idx64, i, n)] = W[i];
}

// ------------------------------------------------------------------- gather
template <typename T, typename TW, typename TR, typename TO>
__global__ __launch_bounds__(256) void moe_gather_kernel(
    const T* __restrict__ Y, const void* __restrict__ IDX, int idx64, const TW* __restrict__ W,
    const TR* __restrict__ RES, TO* __restrict__ OUT, int64_t Tn, int D, int K, int tok_per_block,
    bool vec) {
    const int tpt = 256 / tok_per_block;
    const int64_t t = (int64_t)blockIdx.x * tok_per_block + threadIdx.x / tpt;
    const int lane = threadIdx.x % tpt;
    if (t >= Tn) return;
    if (vec) {
        for (int c = lane * 8; c < D; c += tpt * 8) {
            float acc[8];
            if (RES != nullptr) {
                load_f32<TR, 8>(RES + t * D + c, acc);
            } else {
#pragma unroll
                for (int j = 0; j < 8; ++j) acc[j] = 0.f;
            }
            // rows of up to 4 slots are all requested before the first is added (k ascending, as
            // the reference sums): one exposed memory round trip per batch instead of one per slot
            for (int k0 = 0; k0 < K; k0 += 4) {
                float v[4][8], w[4];
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    if (k0 + u < K) {
                        const int64_t row = load_index(IDX, idx64, t * K + k0 + u, Tn * K);
                        load_f32<T, 8>(Y + row * D + c, v[u]);
                        w[u] = W != nullptr ? (float)W[t * K + k0 + u] : 1.f;
                    }
                }
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    if (k0 + u < K) {
                        if (W != nullptr) {
#pragma unroll
                            for (int j = 0; j < 8; ++j) acc[j] += v[u][j] * w[u];
                        } else {
#pragma unroll
                            for (int j = 0; j < 8; ++j) acc[j] += v[u][j];
                        }
                    }
                }
            }
            store_f32<TO, 8>(OUT + t * D + c, acc);
        }
    } else {
        for (int c = lane; c < D; c += tpt) {
            float acc = RES != nullptr ? (float)RES[t * D + c] : 0.f;
            for (int k = 0; k < K; ++k) {
                const int64_t row = load_index(IDX, idx64, t * K + k, Tn * K);
                const float v = (float)Y[row * D + c];
                acc += W != nullptr ? v * (float)W[t * K + k] : v;
            }
            OUT[t * D + c] = (TO)acc;
        }
    }
}

// ---------------------------------------------------- expert SwiGLU, one wave per row
FX_DEV float sigmoidf_(float x) { return 1.0f / (1.0f + expf(-x)); }

template <typename T, typename TW, typename TO>
__global__ __launch_bounds__(256) void swiglu_moe_fwd_kernel(
    const T* __restrict__ X, const TW* __restrict__ W, TO* __restrict__ OUT, int64_t rows, int F,
    int64_t x_stride, int64_t out_stride, bool vec) {
    const int lane = threadIdx.x & 63;
    const int64_t r = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (r >= rows) return;
    const T* xr = X + r * x_stride;
    TO* o = OUT + r * out_stride;
    const float w = W != nullptr ? (float)W[r] : 1.0f;
    if (vec) {
        for (int c = lane * 8; c < F; c += 512) {
            float x3[8], x1[8], y[8];
            load_f32<T, 8>(xr + c, x3);
            load_f32<T, 8>(xr + F + c, x1);
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                y[j] = (x1[j] * sigmoidf_(x1[j])) * x3[j];
                if (W != nullptr) y[j] *= w;
            }
            store_f32<TO, 8>(o + c, y);
        }
    } else {
        for (int c = lane; c < F; c += 64) {
            const float x3 = (float)xr[c], x1 = (float)xr[F + c];
            float y = (x1 * sigmoidf_(x1)) * x3;
            if (W != nullptr) y *= w;
            o[c] = (TO)y;
        }
    }
}

// PRESCALED = false: dout is the plain upstream gradient, the stored activation is
// act * w.  PRESCALED = true: dout already carries w (the kernel divides it back
// out for the w-gradient with 1 / max(1e-8, w)) and the stored activation is unscaled.
template <typename T, typename TW, typename TDW, bool PRESCALED>
__global__ __launch_bounds__(256) void swiglu_moe_bwd_kernel(
    T* __restrict__ DX, TDW* __restrict__ DW, const T* __restrict__ DOUT, const T* __restrict__ X,
    const TW* __restrict__ W, T* __restrict__ ACT, int64_t rows, int F, int64_t dx_stride,
    int64_t dout_stride, int64_t x_stride, int64_t act_stride, bool vec) {
    const int lane = threadIdx.x & 63;
    const int64_t r = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (r >= rows) return;
    const T* xr = X + r * x_stride;
    const T* dr = DOUT + r * dout_stride;
    T* gx = DX + r * dx_stride;
    T* ar = ACT != nullptr ? ACT + r * act_stride : nullptr;
    const float w = (float)W[r];
    const float w_inv = 1.0f / fmaxf(1e-8f, w);
    float dw = 0.f;
    auto elem = [&](float x3, float x1, float d, float& dx3, float& dx1, float& act) {
        dw += moe_swiglu_bwd_elem<PRESCALED>(x3, x1, d, w, w_inv, dx3, dx1, act);
    };
    if (vec) {
        for (int c = lane * 8; c < F; c += 512) {
            float x3[8], x1[8], d[8], g3[8], g1[8], a[8];
            load_f32<T, 8>(xr + c, x3);
            load_f32<T, 8>(xr + F + c, x1);
            load_f32<T, 8>(dr + c, d);
#pragma unroll
            for (int j = 0; j < 8; ++j) elem(x3[j], x1[j], d[j], g3[j], g1[j], a[j]);
            store_f32<T, 8>(gx + c, g3);
            store_f32<T, 8>(gx + F + c, g1);
            if (ar != nullptr) store_f32<T, 8>(ar + c, a);
        }
    } else {
        for (int c = lane; c < F; c += 64) {
            float g3, g1, a;
            elem((float)xr[c], (float)xr[F + c], (float)dr[c], g3, g1, a);
            gx[c] = (T)g3;
            gx[F + c] = (T)g1;
            if (ar != nullptr) ar[c] = (T)a;
        }
    }
    dw = group_sum<64>(dw);
    if (lane == 0) DW[r] = (TDW)dw;
}

static inline int tokens_per_block(int D) {
    int tpb = 1;
    while (tpb < 16 && (D / 8) * tpb * 2 <= 256) tpb *= 2;
    return tpb;
}

}  // namespace fx

using namespace fx;

extern "C" int fx_moe_scatter(const void* x, const void* indices, int indices_are_int64, const void* scales,
                              int scales_dt, void* out, int64_t T, int D, int K, int64_t out_row_stride,
                              int dt, hipStream_t stream) {
    if (T < 0 || D <= 0 || K <= 0) FX_FAIL("fx_moe_scatter: bad shape");
    if (T == 0) return 0;
    if (!x || !indices || !out) FX_FAIL("fx_moe_scatter: null pointer");
    const bool vec = (D % 8 == 0) && (out_row_stride % 8 == 0) && aligned16(x) && aligned16(out);
    const int tpb = tokens_per_block(D);
    const unsigned grid = (unsigned)((T + tpb - 1) / tpb);
    FX_DISPATCH_DTYPE(dt, TT,
        if (scales) {
            FX_DISPATCH_DTYPE(scales_dt, TS,
                moe_scatter_kernel<TT, TS, true><<<grid, 256, 0, stream>>>(
                    reinterpret_cast<const TT*>(x), reinterpret_cast<TT*>(out), indices, indices_are_int64,
                    reinterpret_cast<const TS*>(scales), T, D, K, out_row_stride, tpb, vec));
        } else {
            moe_scatter_kernel<TT, TT, false><<<grid, 256, 0, stream>>>(
                reinterpret_cast<const TT*>(x), reinterpret_cast<TT*>(out), indices, indices_are_int64,
                nullptr, T, D, K, out_row_stride, tpb, vec);
        });
    FX_CHECK_LAUNCH("fx_moe_scatter");
    return 0;
}

namespace fx {
// out[indices[t, k]] = t: the token each expert-sorted row was routed from.
template <typename TI>
__global__ __launch_bounds__(256) void moe_row_sources_kernel(const TI* __restrict__ IND, int64_t n, int K, int32_t* __restrict__ OUT) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    const int64_t r = (int64_t)IND[i];
    if (r >= 0 && r < n) OUT[r] = (int32_t)(i / K);
}
}  // namespace fx

extern "C" int fx_moe_row_sources(const void* indices, int indices_are_int64, int64_t T, int K, int32_t* out,
                                  hipStream_t stream) {
    if (T < 0 || K <= 0) FX_FAIL("fx_moe_row_sources: bad shape");
    if (T == 0) return 0;
    if (!indices || !out) FX_FAIL("fx_moe_row_sources: null pointer");
    const int64_t n = T * K;
    const unsigned grid = (unsigned)((n + 255) / 256);
    if (indices_are_int64)
        moe_row_sources_kernel<int64_t><<<grid, 256, 0, stream>>>(reinterpret_cast<const int64_t*>(indices), n, K, out);
    else
        moe_row_sources_kernel<int32_t><<<grid, 256, 0, stream>>>(reinterpret_cast<const int32_t*>(indices), n, K, out);
    FX_CHECK_LAUNCH("fx_moe_row_sources");
    return 0;
}

extern "C" int fx_moe_scatter_weights(const void* weights, const void* indices, int indices_are_int64,
                                      void* out, int64_t n, int dt, hipStream_t stream) {
    if (n < 0) FX_FAIL("fx_moe_scatter_weights: negative count");
    if (n == 0) return 0;
    if (!weights || !indices || !out) FX_FAIL("fx_moe_scatter_weights: null pointer");
    FX_DISPATCH_DTYPE(dt, TT,
        moe_scatter_weights_kernel<TT><<<(unsigned)((n + 255) / 256), 256, 0, stream>>>(
            reinterpret_cast<const TT*>(weights), indices, indices_are_int64, reinterpret_cast<TT*>(out), n));
    FX_CHECK_LAUNCH("fx_moe_scatter_weights");
    return 0;
}

extern "C" int fx_moe_gather(const void* expert_out, const void* indices, int indices_are_int64,
                             const void* weights, int weights_dt, const void* residual, int residual_dt,
                             void* out, int out_dt, int64_t T, int D, int K, int dt, hipStream_t stream) {
    if (T < 0 || D <= 0 || K <= 0) FX_FAIL("fx_moe_gather: bad shape");
    if (T == 0) return 0;
    if (!expert_out || !indices || !out) FX_FAIL("fx_moe_gather: null pointer");
    const bool vec = (D % 8 == 0) && aligned16(expert_out) && aligned16(out) && (!residual || aligned16(residual));
    const int tpb = tokens_per_block(D);
    const unsigned grid = (unsigned)((T + tpb - 1) / tpb);
    // weights / residual / out follow a small set of dtype combinations; anything
    // mixed beyond "same as expert_out or fp32" is rejected rather than compiled 81 ways.
    auto same_or_f32 = [&](int d) { return d == dt || d == DT_F32; };
    if ((weights && !same_or_f32(weights_dt)) || (residual && !same_or_f32(residual_dt)) || !same_or_f32(out_dt))
        FX_FAIL("fx_moe_gather: weights/residual/out dtype must equal expert_out's or be fp32");
#define FX_GATHER(TW, TR, TO)                                                                      \
    moe_gather_kernel<TT, TW, TR, TO><<<grid, 256, 0, stream>>>(                                   \
        reinterpret_cast<const TT*>(expert_out), indices, indices_are_int64,                       \
        reinterpret_cast<const TW*>(weights), reinterpret_cast<const TR*>(residual),               \
        reinterpret_cast<TO*>(out), T, D, K, tpb, vec)
    FX_DISPATCH_DTYPE(dt, TT, {
        const bool wf = weights && weights_dt == DT_F32 && dt != DT_F32;
        const bool rf = residual && residual_dt == DT_F32 && dt != DT_F32;
        const bool of = out_dt == DT_F32 && dt != DT_F32;
        if (!wf && !rf && !of) FX_GATHER(TT, TT, TT);
        else if (wf && !rf && !of) FX_GATHER(float, TT, TT);
        else if (!wf && rf && !of) FX_GATHER(TT, float, TT);
        else if (!wf && !rf && of) FX_GATHER(TT, TT, float);
        else if (wf && rf && !of) FX_GATHER(float, float, TT);
        else if (wf && !rf && of) FX_GATHER(float, TT, float);
        else if (!wf && rf && of) FX_GATHER(TT, float, float);
        else FX_GATHER(float, float, float);
    });
#undef FX_GATHER
    FX_CHECK_LAUNCH("fx_moe_gather");
    return 0;
}

extern "C" int fx_swiglu_moe_fwd(const void* x, const void* w, int w_dt, void* out, int out_dt, int64_t rows,
                                 int F, int64_t x_row_stride, int64_t out_row_stride, int dt,
                                 hipStream_t stream) {
    if (rows < 0 || F <= 0) FX_FAIL("fx_swiglu_moe_fwd: bad shape");
    if (rows == 0) return 0;
    if (!x || !out) FX_FAIL("fx_swiglu_moe_fwd: null pointer");
    if (out_dt != dt) FX_FAIL("fx_swiglu_moe_fwd: out dtype must match x");
    if (w && w_dt != dt && w_dt != DT_F32) FX_FAIL("fx_swiglu_moe_fwd: w dtype must equal x's or be fp32");
    const bool vec = (F % 8 == 0) && (x_row_stride % 8 == 0) && (out_row_stride % 8 == 0) && aligned16(x) && aligned16(out);
    const unsigned grid = (unsigned)((rows + 3) / 4);
    FX_DISPATCH_DTYPE(dt, TT,
        if (w && w_dt == DT_F32)
            swiglu_moe_fwd_kernel<TT, float, TT><<<grid, 256, 0, stream>>>(reinterpret_cast<const TT*>(x), reinterpret_cast<const float*>(w), reinterpret_cast<TT*>(out), rows, F, x_row_stride, out_row_stride, vec);
        else
            swiglu_moe_fwd_kernel<TT, TT, TT><<<grid, 256, 0, stream>>>(reinterpret_cast<const TT*>(x), reinterpret_cast<const TT*>(w), reinterpret_cast<TT*>(out), rows, F, x_row_stride, out_row_stride, vec));
    FX_CHECK_LAUNCH("fx_swiglu_moe_fwd");
    return 0;
}

extern "C" int fx_swiglu_moe_bwd(void* dx, void* dw, int dw_dt, const void* dout, const void* x, const void* w,
                                 int w_dt, void* fwd_act, int64_t rows, int F, int64_t dx_row_stride,
                                 int64_t dout_row_stride, int64_t x_row_stride, int64_t act_row_stride, int dt,
                                 int prescaled, hipStream_t stream) {
    if (rows < 0 || F <= 0) FX_FAIL("fx_swiglu_moe_bwd: bad shape");
    if (rows == 0) return 0;
    if (!dx || !dw || !dout || !x || !w) FX_FAIL("fx_swiglu_moe_bwd: null pointer");
    if (w_dt != dt && w_dt != DT_F32) FX_FAIL("fx_swiglu_moe_bwd: w dtype must equal x's or be fp32");
    if (dw_dt != dt && dw_dt != DT_F32) FX_FAIL("fx_swiglu_moe_bwd: dw dtype must equal x's or be fp32");
    const bool vec = (F % 8 == 0) && (dx_row_stride % 8 == 0) && (dout_row_stride % 8 == 0) &&
                     (x_row_stride % 8 == 0) && (!fwd_act || act_row_stride % 8 == 0) && aligned16(dx) &&
                     aligned16(dout) && aligned16(x) && (!fwd_act || aligned16(fwd_act));
    const unsigned grid = (unsigned)((rows + 3) / 4);
#define FX_SB(TW, TDW, P)                                                                          \
    swiglu_moe_bwd_kernel<TT, TW, TDW, P><<<grid, 256, 0, stream>>>(                               \
        reinterpret_cast<TT*>(dx), reinterpret_cast<TDW*>(dw), reinterpret_cast<const TT*>(dout),  \
        reinterpret_cast<const TT*>(x), reinterpret_cast<const TW*>(w), reinterpret_cast<TT*>(fwd_act), \
        rows, F, dx_row_stride, dout_row_stride, x_row_stride, act_row_stride, vec)
    FX_DISPATCH_DTYPE(dt, TT, {
        const bool wf = w_dt == DT_F32 && dt != DT_F32;
        const bool df = dw_dt == DT_F32 && dt != DT_F32;
        if (prescaled) {
            if (!wf && !df) FX_SB(TT, TT, true); else if (wf && !df) FX_SB(float, TT, true);
            else if (!wf && df) FX_SB(TT, float, true); else FX_SB(float, float, true);
        } else {
            if (!wf && !df) FX_SB(TT, TT, false); else if (wf && !df) FX_SB(float, TT, false);
            else if (!wf && df) FX_SB(TT, float, false); else FX_SB(float, float, false);
        }
    });
#undef FX_SB
    FX_CHECK_LAUNCH("fx_swiglu_moe_bwd");
    return 0;
}
