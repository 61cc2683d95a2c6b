// Rotary position embedding, in place, pair-interleaved channels, gfx950.
//
// Semantics: flextrain/ops/_kernels/rope.py:8-157.  For token t with integer
// position pos and pair index i (< rot_dim/2):  angle = float(pos) * inv_freq[i]
// (fp32), (e, o) = (x[2i], x[2i+1]);
//   forward : (e*c - o*s, e*s + o*c)       backward: (e*c + o*s, -e*s + o*c)
// Q (T,Hq,D) and K (T,Hk,D) are rotated by the same launch.  Channels at or
// beyond rot_dim are left untouched (rot_dim == D is the reference's full
// rotation; smaller values are the partial rotation of
// flextrain/ops/_kernels/rope_partial.py:29-147).
//
// Fast path: unit channel stride and 16-byte aligned head rows.  cos/sin of a
// token are computed once into LDS (D/2 lanes), then every lane rotates packs
// of 8 channels (4 pairs) with one 16-byte load and one 16-byte store.
#include "common.h"
#include "flexhip.h"

namespace fx {

constexpr int ROPE_THREADS = 256;

template <typename T, bool BWD, bool NT>
__global__ __launch_bounds__(ROPE_THREADS) void rope_vec_kernel(
    T* __restrict__ Q, T* __restrict__ K, const int32_t* __restrict__ POS, int64_t stride_pos,
    const float* __restrict__ INV_FREQ, int64_t stride_if, int64_t T_tokens, int Hq, int Hk, int D,
    int rot_dim, int64_t sq_t, int64_t sq_h, int64_t sk_t, int64_t sk_h, int tok_per_block) {
    extern __shared__ float cs[];  // [tok_per_block][rot_dim/2][2]
    const int half = rot_dim >> 1;
    const int tid = threadIdx.x;
    const int64_t tok0 = (int64_t)blockIdx.x * tok_per_block;
    for (int i = tid; i < tok_per_block * half; i += ROPE_THREADS) {
        const int tl = i / half, p = i % half;
        const int64_t t = tok0 + tl;
        float c = 1.f, s = 0.f;
        if (t < T_tokens) {
            const float ang = (float)POS[t * stride_pos] * INV_FREQ[p * stride_if];
            sincosf(ang, &s, &c);
        }
        cs[2 * i] = c;
        cs[2 * i + 1] = BWD ? -s : s;
    }
    __syncthreads();
    const int tpt = ROPE_THREADS / tok_per_block;  // lanes per token
    const int tl = tid / tpt;
    const int lane = tid % tpt;
    const int64_t t = tok0 + tl;
    if (t >= T_tokens) return;
    const int vec_per_head = rot_dim >> 3;  // packs of 8 rotated channels
    const int items = (Hq + Hk) * vec_per_head;
    const float* tcs = cs + (size_t)tl * half * 2;
    auto rotate = [&](int h, int v, const float (&c)[4], const float (&s)[4]) {
        T* p = (h < Hq) ? (Q + t * sq_t + (int64_t)h * sq_h) : (K + t * sk_t + (int64_t)(h - Hq) * sk_h);
        p += v * 8;
        float x[8], y[8];
        load_f32<T, 8, NT>(p, x);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const float e = x[2 * j], o = x[2 * j + 1];
            y[2 * j] = e * c[j] - o * s[j];
            y[2 * j + 1] = e * s[j] + o * c[j];
        }
        store_f32<T, 8, NT>(p, y);
    };
    if (tpt % vec_per_head == 0) {
        // Each lane keeps one pack position for every head: cos/sin stay in registers.
        const int v = lane % vec_per_head;
        float c[4], s[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) { c[j] = tcs[(v * 4 + j) * 2]; s[j] = tcs[(v * 4 + j) * 2 + 1]; }
        const int hstep = tpt / vec_per_head;
        // four heads per round: all loads are issued before the first store, so a lane has up to
        // 64 bytes in flight instead of one load -> rotate -> store chain per head
        for (int h0 = lane / vec_per_head; h0 < Hq + Hk; h0 += 4 * hstep) {
            float x[4][8];
            T* ptr[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int h = h0 + u * hstep;
                ptr[u] = nullptr;
                if (h < Hq + Hk) {
                    ptr[u] = ((h < Hq) ? (Q + t * sq_t + (int64_t)h * sq_h) : (K + t * sk_t + (int64_t)(h - Hq) * sk_h)) + v * 8;
                    load_f32<T, 8, NT>(ptr[u], x[u]);
                }
            }
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                if (ptr[u] == nullptr) continue;
                float y[8];
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const float e = x[u][2 * j], o = x[u][2 * j + 1];
                    y[2 * j] = e * c[j] - o * s[j];
                    y[2 * j + 1] = e * s[j] + o * c[j];
                }
                store_f32<T, 8, NT>(ptr[u], y);
            }
        }
    } else {
        for (int it = lane; it < items; it += tpt) {
            const int h = it / vec_per_head;
            const int v = it % vec_per_head;
            float c[4], s[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) { c[j] = tcs[(v * 4 + j) * 2]; s[j] = tcs[(v * 4 + j) * 2 + 1]; }
            rotate(h, v, c, s);
        }
    }
}

// Arbitrary strides / alignment: one lane per (head, pair).
template <typename T, bool BWD>
__global__ __launch_bounds__(ROPE_THREADS) void rope_generic_kernel(
    T* __restrict__ Q, T* __restrict__ K, const int32_t* __restrict__ POS, int64_t stride_pos,
    const float* __restrict__ INV_FREQ, int64_t stride_if, int Hq, int Hk, int rot_dim,
    int64_t sq_t, int64_t sq_h, int64_t sq_d, int64_t sk_t, int64_t sk_h, int64_t sk_d) {
    const int64_t t = blockIdx.x;
    const int half = rot_dim >> 1;
    const float pos = (float)POS[t * stride_pos];
    const int items = (Hq + Hk) * half;
    for (int it = threadIdx.x; it < items; it += ROPE_THREADS) {
        const int h = it / half, i = it % half;
        float s, c;
        sincosf(pos * INV_FREQ[i * stride_if], &s, &c);
        if (BWD) s = -s;
        T *pe, *po;
        if (h < Hq) {
            pe = Q + t * sq_t + (int64_t)h * sq_h + (int64_t)(2 * i) * sq_d;
            po = pe + sq_d;
        } else {
            pe = K + t * sk_t + (int64_t)(h - Hq) * sk_h + (int64_t)(2 * i) * sk_d;
            po = pe + sk_d;
        }
        const float e = (float)*pe, o = (float)*po;
        *pe = (T)(e * c - o * s);
        *po = (T)(e * s + o * c);
    }
}

static inline bool mult8(int64_t v) { return (v & 7) == 0; }

template <typename T, bool BWD>
static int launch_rope(void* q, void* k, const int32_t* pos, int64_t stride_pos, const float* inv_freq,
                       int64_t stride_if, int64_t T_tokens, int Hq, int Hk, int D, int rot_dim,
                       const int64_t* sq, const int64_t* sk, hipStream_t s) {
    T* Q = reinterpret_cast<T*>(q);
    T* K = reinterpret_cast<T*>(k);
    // 16-byte alignment of every head row: base aligned and strides multiples
    // of 16 bytes (8 two-byte or 4 four-byte elements; use 8 for both).
    bool vec = sq[2] == 1 && mult8(sq[0]) && mult8(sq[1]) && mult8(rot_dim) && aligned16(q);
    if (Hk > 0) vec = vec && sk[2] == 1 && mult8(sk[0]) && mult8(sk[1]) && aligned16(k);
    if (vec) {
        const int items = (Hq + Hk) * (rot_dim >> 3);
        int tpb = 1;
        while (tpb < 16 && items * tpb * 2 <= ROPE_THREADS) tpb *= 2;
        const size_t lds = (size_t)tpb * (rot_dim >> 1) * 2 * sizeof(float);
        const unsigned grid = (unsigned)((T_tokens + tpb - 1) / tpb);
        // the rotation is in place: plain accesses (non-temporal ones slow read-modify-write streams down)
        const bool nt = false;
        if (nt)
            rope_vec_kernel<T, BWD, true><<<grid, ROPE_THREADS, lds, s>>>(
                Q, K, pos, stride_pos, inv_freq, stride_if, T_tokens, Hq, Hk, D, rot_dim, sq[0], sq[1],
                Hk > 0 ? sk[0] : 0, Hk > 0 ? sk[1] : 0, tpb);
        else
            rope_vec_kernel<T, BWD, false><<<grid, ROPE_THREADS, lds, s>>>(
                Q, K, pos, stride_pos, inv_freq, stride_if, T_tokens, Hq, Hk, D, rot_dim, sq[0], sq[1],
                Hk > 0 ? sk[0] : 0, Hk > 0 ? sk[1] : 0, tpb);
    } else {
        rope_generic_kernel<T, BWD><<<(unsigned)T_tokens, ROPE_THREADS, 0, s>>>(
            Q, K, pos, stride_pos, inv_freq, stride_if, Hq, Hk, rot_dim, sq[0], sq[1], sq[2],
            Hk > 0 ? sk[0] : 0, Hk > 0 ? sk[1] : 0, Hk > 0 ? sk[2] : 0);
    }
    return 0;
}

}  // namespace fx

using namespace fx;

extern "C" int fx_rope(void* q, void* k, const int32_t* pos, int64_t stride_pos, const float* inv_freq,
                       int64_t stride_if, int64_t T_tokens, int Hq, int Hk, int D, int rot_dim,
                       const int64_t* q_strides, const int64_t* k_strides, int dt, int backward,
                       hipStream_t stream) {
    if (T_tokens < 0 || Hq < 0 || Hk < 0 || D <= 0) FX_FAIL("fx_rope: bad shape");
    if (rot_dim <= 0 || rot_dim > D || (rot_dim & 1)) FX_FAIL("fx_rope: rot_dim %d invalid for head dim %d", rot_dim, D);
    if (T_tokens == 0 || Hq + Hk == 0) return 0;
    if (!pos || !inv_freq || (Hq > 0 && !q) || (Hk > 0 && !k)) FX_FAIL("fx_rope: null pointer");
    if (!q_strides || (Hk > 0 && !k_strides)) FX_FAIL("fx_rope: missing strides");
    if ((rot_dim >> 1) * 16 * 2 * sizeof(float) > 64 * 1024) FX_FAIL("fx_rope: rot_dim %d too large", rot_dim);
    int64_t sq0[3] = {0, 0, 1};
    if (Hq == 0) q_strides = sq0;
    FX_DISPATCH_DTYPE(dt, T,
        if (backward) launch_rope<T, true>(q, k, pos, stride_pos, inv_freq, stride_if, T_tokens, Hq, Hk, D, rot_dim, q_strides, k_strides, stream);
        else launch_rope<T, false>(q, k, pos, stride_pos, inv_freq, stride_if, T_tokens, Hq, Hk, D, rot_dim, q_strides, k_strides, stream));
    FX_CHECK_LAUNCH("fx_rope");
    return 0;
}
