// Row softmax, cross-entropy from probabilities, and the fused
// logits -> (loss, dZ) kernel of the LM head, gfx950.
//
// Reference semantics:
//   flextrain/ops/_kernels/softmax.py:13-108        online softmax with temperature; probabilities
//                                                   rounded to the output dtype; first-occurrence
//                                                   argmax (int64) and max probability 1/l (fp32)
//   flextrain/ops/_kernels/cross_entropy.py:14-57   valid = 0 <= label < V; loss = min(-log p[label],
//                                                   max_loss); p[label] -= 1 in place
//   flextrain/nn/loss.py:248-316                    rows whose label is the ignore index (or whose
//                                                   loss_mask is false) get loss 0 and a zero dZ row
// The fused kernel does all of the above in two sweeps over a row of logits and
// takes the loss from the fp32 log-sum-exp, lse - logit[label], instead of from
// probabilities already rounded to bf16.
//
// One workgroup of 1024 lanes owns a row; a lane keeps an online (max, sum)
// pair over its 16-byte packs, pairs are merged through wave shuffles and LDS.
#include "common.h"
#include "flexhip.h"

namespace fx {

constexpr int SM_THREADS = 1024;
constexpr float NEG_INF_F = -__builtin_huge_valf();

struct RowStat {
    float m, l, best;
    int idx;
};

FX_DEV void stat_add(RowStat& s, float x, int i) {
    if (x > s.best) { s.best = x; s.idx = i; }        // strict: the first maximum wins
    if (x > s.m) {
        s.l = s.l * __expf(s.m - x) + 1.0f;
        s.m = x;
    } else if (x > NEG_INF_F) {   // a -inf element adds nothing (and -inf - -inf is NaN)
        s.l += __expf(x - s.m);
    }
}

// Eight consecutive elements at once: one rescale of the running sum per pack instead of a
// data-dependent branch per element (the sweep is otherwise bound by its exponentials).
FX_DEV void stat_add_pack(RowStat& s, const float (&v)[8], int c0) {
    float pm = v[0];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        if (v[j] > s.best) { s.best = v[j]; s.idx = c0 + j; }   // strict: the first maximum wins
        pm = fmaxf(pm, v[j]);
    }
    if (pm > NEG_INF_F) {                 // a pack of -inf adds nothing (and -inf - -inf is NaN)
        const float nm = fmaxf(s.m, pm);
        float acc = 0.f;
#pragma unroll
        for (int j = 0; j < 8; ++j) acc += __expf(v[j] - nm);
        s.l = s.l * __expf(s.m - nm) + acc;
        s.m = nm;
    }
}

FX_DEV void stat_merge(RowStat& a, float m, float l, float best, int idx) {
    if (best > a.best || (best == a.best && idx < a.idx)) { a.best = best; a.idx = idx; }
    const float nm = fmaxf(a.m, m);
    if (nm == NEG_INF_F) { a.l = 0.f; a.m = nm; return; }
    a.l = a.l * __expf(a.m - nm) + l * __expf(m - nm);
    a.m = nm;
}

// All lanes of the workgroup return the row's merged statistics.
FX_DEV RowStat block_stat(RowStat s, float* sm_f, int* sm_i) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        const float m = __shfl_xor(s.m, off, 64), l = __shfl_xor(s.l, off, 64), b = __shfl_xor(s.best, off, 64);
        const int i = __shfl_xor(s.idx, off, 64);
        stat_merge(s, m, l, b, i);
    }
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    constexpr int NW = SM_THREADS / 64;
    __syncthreads();
    if (lane == 0) { sm_f[wave] = s.m; sm_f[NW + wave] = s.l; sm_f[2 * NW + wave] = s.best; sm_i[wave] = s.idx; }
    __syncthreads();
    RowStat r{sm_f[0], sm_f[NW], sm_f[2 * NW], sm_i[0]};
    for (int w = 1; w < NW; ++w) stat_merge(r, sm_f[w], sm_f[NW + w], sm_f[2 * NW + w], sm_i[w]);
    return r;
}

// Final-logit soft cap (flextrain/nn/head.py:273-282): y = cap * tanh(x / cap), rounded to the
// storage type as the reference's in-place buffer is, so that argmax, maximum probability and loss
// see the values a separate capping pass would have left in memory.
template <typename T>
FX_DEV float softcap_value(float x, float cap, float inv_cap) {
    return (float)(T)(cap * tanhf(x * inv_cap));
}

template <typename T, bool CAP = false>
FX_DEV RowStat row_sweep(const T* __restrict__ x, int V, float inv_temp, bool vec, float cap = 0.f) {
    RowStat s{NEG_INF_F, 0.f, NEG_INF_F, 0x7fffffff};
    const float inv_cap = CAP ? 1.0f / cap : 0.f;
    if (vec) {
        for (int c = threadIdx.x * 8; c < V; c += SM_THREADS * 8) {
            float v[8];
            load_f32<T, 8>(x + c, v);
#pragma unroll
            for (int j = 0; j < 8; ++j) v[j] = CAP ? softcap_value<T>(v[j], cap, inv_cap) : v[j] * inv_temp;
            stat_add_pack(s, v, c);
        }
    } else {
        for (int c = threadIdx.x; c < V; c += SM_THREADS)
            stat_add(s, CAP ? softcap_value<T>((float)x[c], cap, inv_cap) : (float)x[c] * inv_temp, c);
    }
    return s;
}

template <typename TI, typename TO>
__global__ __launch_bounds__(SM_THREADS) void softmax_kernel(
    const TI* __restrict__ X, TO* __restrict__ OUT, int64_t* __restrict__ MAX_IDX, float* __restrict__ MAX_VAL,
    int V, int64_t in_stride, int64_t out_stride, float inv_temp, bool vec) {
    __shared__ float sm_f[3 * SM_THREADS / 64];
    __shared__ int sm_i[SM_THREADS / 64];
    const int64_t row = blockIdx.x;
    const TI* x = X + row * in_stride;
    TO* o = OUT + row * out_stride;
    const RowStat st = block_stat(row_sweep<TI>(x, V, inv_temp, vec), sm_f, sm_i);
    const float inv_l = 1.0f / st.l;
    if (threadIdx.x == 0) {
        if (MAX_IDX) MAX_IDX[row] = st.idx;
        if (MAX_VAL) MAX_VAL[row] = inv_l;
    }
    if (vec) {
        for (int c = threadIdx.x * 8; c < V; c += SM_THREADS * 8) {
            float v[8];
            load_f32<TI, 8>(x + c, v);
#pragma unroll
            for (int j = 0; j < 8; ++j) v[j] = __expf(v[j] * inv_temp - st.m) * inv_l;
            store_f32<TO, 8>(o + c, v);
        }
    } else {
        for (int c = threadIdx.x; c < V; c += SM_THREADS) o[c] = (TO)(__expf((float)x[c] * inv_temp - st.m) * inv_l);
    }
}

// Probabilities in, dZ out (in place), one lane per row.
template <typename T, typename TL>
__global__ __launch_bounds__(256) void cross_entropy_kernel(T* __restrict__ P, const TL* __restrict__ LABELS,
                                                            float* __restrict__ LOSS, float* __restrict__ VALID,
                                                            int64_t rows, int V, int64_t stride_t, int64_t stride_v,
                                                            float max_loss) {
    const int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (t >= rows) return;
    const int64_t label = (int64_t)LABELS[t];
    const bool valid = label >= 0 && label < V;
    VALID[t] = valid ? 1.0f : 0.0f;
    float loss = 0.f;
    if (valid) {
        T* p = P + t * stride_t + label * stride_v;
        const float pc = (float)*p;
        loss = fminf(-logf(pc), max_loss);
        *p = (T)(pc - 1.0f);
    }
    LOSS[t] = loss;
}

// Logits in, dZ out (in place or to DZ), fp32 loss from the log-sum-exp.
//   keep  = label != ignore_index  &&  (MASK == null || MASK[t])
//   valid = 0 <= label < V
//   loss  = keep && valid ? min(lse - x[label], max_loss) : 0
//   dZ    = keep ? softmax(x) - (valid ? onehot(label) : 0) : 0
// CAP: the statistics, the loss and the probabilities are those of y = cap * tanh(x / cap), and dZ
// is the gradient at x, i.e. multiplied by dy/dx = 1 - (y / cap)^2 (flextrain/nn/head.py:273-298).
template <typename T, typename TL, bool CAP>
__global__ __launch_bounds__(SM_THREADS) void softmax_ce_kernel(
    const T* X, T* DZ /* may alias X */, const TL* __restrict__ LABELS, const uint8_t* __restrict__ MASK,
    float* __restrict__ LOSS, int64_t* __restrict__ MAX_IDX, float* __restrict__ MAX_VAL, int V, int64_t in_stride,
    int64_t out_stride, int64_t ignore_index, float max_loss, bool vec, float cap) {
    __shared__ float sm_f[3 * SM_THREADS / 64];
    __shared__ int sm_i[SM_THREADS / 64];
    const int64_t row = blockIdx.x;
    const T* x = X + row * in_stride;
    T* o = DZ + row * out_stride;
    const int64_t label = (int64_t)LABELS[row];
    const bool keep = label != ignore_index && (MASK == nullptr || MASK[row] != 0);
    const bool valid = label >= 0 && label < V;
    const RowStat st = block_stat(row_sweep<T, CAP>(x, V, 1.0f, vec, cap), sm_f, sm_i);
    const float inv_l = 1.0f / st.l;
    const float inv_cap = CAP ? 1.0f / cap : 0.f;
    if (threadIdx.x == 0) {
        if (MAX_IDX) MAX_IDX[row] = st.idx;
        if (MAX_VAL) MAX_VAL[row] = inv_l;
        float loss = 0.f;
        if (keep && valid) {
            const float xl = CAP ? softcap_value<T>((float)x[label], cap, inv_cap) : (float)x[label];
            loss = fminf((st.m + logf(st.l)) - xl, max_loss);
        }
        LOSS[row] = loss;
    }
    __syncthreads();  // x[label] is read before any lane overwrites the row in place
    const int hot = (keep && valid) ? (int)label : -1;
    if (vec) {
        for (int c = threadIdx.x * 8; c < V; c += SM_THREADS * 8) {
            float v[8];
            if (keep) {
                load_f32<T, 8>(x + c, v);
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    const float y = CAP ? softcap_value<T>(v[j], cap, inv_cap) : v[j];
                    v[j] = __expf(y - st.m) * inv_l;
                    if (c + j == hot) v[j] -= 1.0f;
                    if (CAP) v[j] *= 1.0f - (y * inv_cap) * (y * inv_cap);
                }
            } else {
#pragma unroll
                for (int j = 0; j < 8; ++j) v[j] = 0.f;
            }
            store_f32<T, 8>(o + c, v);
        }
    } else {
        for (int c = threadIdx.x; c < V; c += SM_THREADS) {
            float v = 0.f;
            if (keep) {
                const float y = CAP ? softcap_value<T>((float)x[c], cap, inv_cap) : (float)x[c];
                v = __expf(y - st.m) * inv_l;
                if (c == hot) v -= 1.0f;
                if (CAP) v *= 1.0f - (y * inv_cap) * (y * inv_cap);
            }
            o[c] = (T)v;
        }
    }
}

// The soft cap as two passes of its own, for loss objects that are not the fused kernel above
// (flextrain/nn/head.py:273-298): forward caps X in place and stores the gate 1 - (y / cap)^2,
// computed from the rounded y, in the storage type; backward multiplies dZ by the gate.
template <typename T>
__global__ __launch_bounds__(256) void softcap_fwd_kernel(T* __restrict__ X, T* __restrict__ GATE, int64_t rows, int V,
                                                          int64_t x_stride, int64_t g_stride, float cap, bool vec) {
    const float inv_cap = 1.0f / cap;
    const int per_row = vec ? V / 8 : V;
    const int64_t total = rows * per_row;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
        const int64_t r = i / per_row;
        const int c = (int)(i % per_row);
        if (vec) {
            float v[8], gt[8];
            load_f32<T, 8>(X + r * x_stride + c * 8, v);
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                v[j] = softcap_value<T>(v[j], cap, inv_cap);
                gt[j] = 1.0f - (v[j] * inv_cap) * (v[j] * inv_cap);
            }
            store_f32<T, 8>(X + r * x_stride + c * 8, v);
            store_f32<T, 8>(GATE + r * g_stride + c * 8, gt);
        } else {
            const float y = softcap_value<T>((float)X[r * x_stride + c], cap, inv_cap);
            X[r * x_stride + c] = (T)y;
            GATE[r * g_stride + c] = (T)(1.0f - (y * inv_cap) * (y * inv_cap));
        }
    }
}

template <typename T>
__global__ __launch_bounds__(256) void softcap_bwd_kernel(T* __restrict__ DZ, const T* __restrict__ GATE, int64_t rows,
                                                          int V, int64_t dz_stride, int64_t g_stride, bool vec) {
    const int per_row = vec ? V / 8 : V;
    const int64_t total = rows * per_row;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
        const int64_t r = i / per_row;
        const int c = (int)(i % per_row);
        if (vec) {
            float v[8], gt[8];
            load_f32<T, 8>(DZ + r * dz_stride + c * 8, v);
            load_f32<T, 8>(GATE + r * g_stride + c * 8, gt);
#pragma unroll
            for (int j = 0; j < 8; ++j) v[j] *= gt[j];
            store_f32<T, 8>(DZ + r * dz_stride + c * 8, v);
        } else {
            DZ[r * dz_stride + c] = (T)((float)DZ[r * dz_stride + c] * (float)GATE[r * g_stride + c]);
        }
    }
}

}  // namespace fx

using namespace fx;

extern "C" int fx_softmax(const void* x, void* out, int64_t* max_idx_out, float* max_val_out, int64_t rows, int V,
                          int64_t in_row_stride, int64_t out_row_stride, float temperature, int in_dt, int out_dt,
                          hipStream_t stream) {
    if (rows < 0 || V <= 0) FX_FAIL("fx_softmax: bad shape");
    if (!(temperature > 0.f)) FX_FAIL("fx_softmax: temperature must be positive");
    if (rows == 0) return 0;
    if (!x || !out) FX_FAIL("fx_softmax: null pointer");
    const bool vec = (V % 8 == 0) && (in_row_stride % 8 == 0) && (out_row_stride % 8 == 0) && aligned16(x) && aligned16(out);
    FX_DISPATCH_DTYPE(in_dt, TI,
        FX_DISPATCH_DTYPE(out_dt, TO,
            softmax_kernel<TI, TO><<<(unsigned)rows, SM_THREADS, 0, stream>>>(
                reinterpret_cast<const TI*>(x), reinterpret_cast<TO*>(out), max_idx_out, max_val_out, V, in_row_stride,
                out_row_stride, 1.0f / temperature, vec)));
    FX_CHECK_LAUNCH("fx_softmax");
    return 0;
}

extern "C" int fx_cross_entropy(void* probs, const void* labels, int labels_are_int64, float* loss_out,
                                float* valid_out, int64_t rows, int V, int64_t stride_t, int64_t stride_v,
                                float max_loss, int dt, hipStream_t stream) {
    if (rows < 0 || V <= 0) FX_FAIL("fx_cross_entropy: bad shape");
    if (rows == 0) return 0;
    if (!probs || !labels || !loss_out || !valid_out) FX_FAIL("fx_cross_entropy: null pointer");
    const unsigned grid = (unsigned)((rows + 255) / 256);
    FX_DISPATCH_DTYPE(dt, TT,
        if (labels_are_int64)
            cross_entropy_kernel<TT, int64_t><<<grid, 256, 0, stream>>>(reinterpret_cast<TT*>(probs), reinterpret_cast<const int64_t*>(labels), loss_out, valid_out, rows, V, stride_t, stride_v, max_loss);
        else
            cross_entropy_kernel<TT, int32_t><<<grid, 256, 0, stream>>>(reinterpret_cast<TT*>(probs), reinterpret_cast<const int32_t*>(labels), loss_out, valid_out, rows, V, stride_t, stride_v, max_loss));
    FX_CHECK_LAUNCH("fx_cross_entropy");
    return 0;
}

extern "C" int fx_softmax_ce(const void* logits, void* dz_out, const void* labels, int labels_are_int64,
                             const uint8_t* loss_mask, float* loss_out, int64_t* max_idx_out, float* max_val_out,
                             int64_t rows, int V, int64_t in_row_stride, int64_t out_row_stride, int64_t ignore_index,
                             float max_loss, float softcap, int dt, hipStream_t stream) {
    if (rows < 0 || V <= 0) FX_FAIL("fx_softmax_ce: bad shape");
    if (!(softcap >= 0.f)) FX_FAIL("fx_softmax_ce: softcap must be 0 (off) or positive");
    if (rows == 0) return 0;
    if (!logits || !dz_out || !labels || !loss_out) FX_FAIL("fx_softmax_ce: null pointer");
    if (rows > 1 && (in_row_stride < V || out_row_stride < V)) FX_FAIL("fx_softmax_ce: a row stride is smaller than the row");
    const bool vec = (V % 8 == 0) && (in_row_stride % 8 == 0) && (out_row_stride % 8 == 0) && aligned16(logits) && aligned16(dz_out);
#define FX_SMCE(TT, TL, CAP_)                                                                                         \
    softmax_ce_kernel<TT, TL, CAP_><<<(unsigned)rows, SM_THREADS, 0, stream>>>(                                        \
        reinterpret_cast<const TT*>(logits), reinterpret_cast<TT*>(dz_out), reinterpret_cast<const TL*>(labels),      \
        loss_mask, loss_out, max_idx_out, max_val_out, V, in_row_stride, out_row_stride, ignore_index, max_loss, vec, \
        softcap)
    FX_DISPATCH_DTYPE(dt, TT,
        if (labels_are_int64) { if (softcap > 0.f) FX_SMCE(TT, int64_t, true); else FX_SMCE(TT, int64_t, false); }
        else { if (softcap > 0.f) FX_SMCE(TT, int32_t, true); else FX_SMCE(TT, int32_t, false); });
#undef FX_SMCE
    FX_CHECK_LAUNCH("fx_softmax_ce");
    return 0;
}

static unsigned flat_grid(int64_t items) {
    const int64_t g = (items + 255) / 256;
    return (unsigned)(g < 1 ? 1 : (g > 65536 ? 65536 : g));
}

extern "C" int fx_softcap_fwd(void* logits, void* gate_out, int64_t rows, int V, int64_t row_stride,
                              int64_t gate_row_stride, float softcap, int dt, hipStream_t stream) {
    if (rows < 0 || V <= 0) FX_FAIL("fx_softcap_fwd: bad shape");
    if (!(softcap > 0.f)) FX_FAIL("fx_softcap_fwd: softcap must be positive");
    if (rows == 0) return 0;
    if (!logits || !gate_out) FX_FAIL("fx_softcap_fwd: null pointer");
    if (rows > 1 && (row_stride < V || gate_row_stride < V)) FX_FAIL("fx_softcap_fwd: a row stride is smaller than the row");
    const bool vec = (V % 8 == 0) && (row_stride % 8 == 0) && (gate_row_stride % 8 == 0) && aligned16(logits) && aligned16(gate_out);
    FX_DISPATCH_DTYPE(dt, TT,
        softcap_fwd_kernel<TT><<<flat_grid(rows * (vec ? V / 8 : V)), 256, 0, stream>>>(
            reinterpret_cast<TT*>(logits), reinterpret_cast<TT*>(gate_out), rows, V, row_stride, gate_row_stride, softcap, vec));
    FX_CHECK_LAUNCH("fx_softcap_fwd");
    return 0;
}

extern "C" int fx_softcap_bwd(void* dz, const void* gate, int64_t rows, int V, int64_t row_stride,
                              int64_t gate_row_stride, int dt, hipStream_t stream) {
    if (rows < 0 || V <= 0) FX_FAIL("fx_softcap_bwd: bad shape");
    if (rows == 0) return 0;
    if (!dz || !gate) FX_FAIL("fx_softcap_bwd: null pointer");
    if (rows > 1 && (row_stride < V || gate_row_stride < V)) FX_FAIL("fx_softcap_bwd: a row stride is smaller than the row");
    const bool vec = (V % 8 == 0) && (row_stride % 8 == 0) && (gate_row_stride % 8 == 0) && aligned16(dz) && aligned16(gate);
    FX_DISPATCH_DTYPE(dt, TT,
        softcap_bwd_kernel<TT><<<flat_grid(rows * (vec ? V / 8 : V)), 256, 0, stream>>>(
            reinterpret_cast<TT*>(dz), reinterpret_cast<const TT*>(gate), rows, V, row_stride, gate_row_stride, vec));
    FX_CHECK_LAUNCH("fx_softcap_bwd");
    return 0;
}
