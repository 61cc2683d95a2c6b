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
// Fast paths: unit channel stride and 16-byte aligned head rows; a lane rotates packs of
// 8 channels (4 pairs) with one 16-byte load and one 16-byte store, all loads of a lane are
// requested before the cos / sin of its tokens are computed (once per token and wave or
// workgroup, shared through LDS), and large launches use non-temporal accesses.
#include "common.h"
#include "flexhip.h"

namespace fx {

constexpr int ROPE_THREADS = 256;

// a / d for 0 <= a < 2^22 and d >= 1, from the reciprocal the host passes in: one multiply, one fix-up.
FX_DEV int div_small(int a, int d, float inv_d) {
    int q = (int)((float)a * inv_d);
    const int r = a - q * d;
    if (r < 0) --q;
    else if (r >= d) ++q;
    return q;
}

// The streaming form.  A workgroup owns `tpw` consecutive tokens and treats their
// tpw * (Hq + Hk) * rot_dim / 8 packs of 8 channels as one flat list: lane l takes packs
// l, l + 256, l + 512, ... so that no lane idles whatever the head count, and requests up to NP
// packs (16 bytes each for 2-byte types) before it touches any of them.  The loads are issued
// FIRST; only then are the tokens' cos / sin computed (tpw * rot_dim / 2 values, one or two per
// lane) into two separate LDS arrays, so the trigonometry runs while the loads are in flight,
// and a lane's four cos and four sin values are one 16-byte LDS read each (lanes of a wave read
// 16 consecutive packs of one token, or the same ones: no bank conflicts).
template <typename T, bool BWD, int NP, bool NT>
__global__ __launch_bounds__(ROPE_THREADS) void rope_flat_kernel(
    T* __restrict__ Q, T* __restrict__ K, const int32_t* __restrict__ POS, int64_t stride_pos,
    const float* __restrict__ INV_FREQ, int64_t stride_if, int64_t T_tokens, int Hq, int rot_dim, int64_t sq_t,
    int64_t sq_h, int64_t sk_t, int64_t sk_h, int tpw, int vph, int items, float inv_items, float inv_vph) {
    extern __shared__ float cs[];
    typedef typename VecOf<T>::type V;
    constexpr int VN = VecOf<T>::N, NV = 8 / VN;
    const int half = rot_dim >> 1;
    float* cosv = cs;
    float* sinv = cs + tpw * half;
    constexpr int nthr = ROPE_THREADS;
    const int tid = threadIdx.x;
    const int64_t tok0 = (int64_t)blockIdx.x * tpw;
    const int ntok = (T_tokens - tok0 < tpw) ? (int)(T_tokens - tok0) : tpw;
    const int total = ntok * items;
    bool have_cs = false;
    for (int base = 0; base < total; base += NP * nthr) {
        V raw[NP][NV];
        T* ptr[NP];
        int cso[NP];
#pragma unroll
        for (int j = 0; j < NP; ++j) {
            const int p = base + j * nthr + tid;
            cso[j] = -1;
            if (p < total) {
                const int tl = div_small(p, items, inv_items);
                const int r = p - tl * items;
                const int h = div_small(r, vph, inv_vph);
                const int v = r - h * vph;
                const int64_t t = tok0 + tl;
                T* src = ((h < Hq) ? (Q + t * sq_t + (int64_t)h * sq_h) : (K + t * sk_t + (int64_t)(h - Hq) * sk_h)) + v * 8;
                ptr[j] = src;
                cso[j] = tl * half + v * 4;
#pragma unroll
                for (int i = 0; i < NV; ++i) {
                    if (NT) raw[j][i] = __builtin_nontemporal_load(reinterpret_cast<const V*>(src + i * VN));
                    else raw[j][i] = *reinterpret_cast<const V*>(src + i * VN);
                }
            }
        }
        if (!have_cs) {       // uniform: every lane of the workgroup runs the same trip count
            for (int i = tid; i < ntok * half; i += nthr) {
                const int tl = i / half, pr = i - tl * half;
                float sn, c;
                sincosf((float)POS[(tok0 + tl) * stride_pos] * INV_FREQ[pr * stride_if], &sn, &c);
                cosv[i] = c;
                sinv[i] = BWD ? -sn : sn;
            }
            __syncthreads();
            have_cs = true;
        }
#pragma unroll
        for (int j = 0; j < NP; ++j) {
            if (cso[j] < 0) continue;
            const float4 c = *reinterpret_cast<const float4*>(cosv + cso[j]);
            const float4 sn = *reinterpret_cast<const float4*>(sinv + cso[j]);
            const float cc[4] = {c.x, c.y, c.z, c.w}, ss[4] = {sn.x, sn.y, sn.z, sn.w};
            float x[8];
#pragma unroll
            for (int i = 0; i < NV; ++i)
#pragma unroll
                for (int e = 0; e < VN; ++e) x[i * VN + e] = (float)raw[j][i][e];
            V out[NV];
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const float e = x[2 * q], o = x[2 * q + 1];
                const float ye = e * cc[q] - o * ss[q], yo = e * ss[q] + o * cc[q];
                out[(2 * q) / VN][(2 * q) % VN] = (T)ye;
                out[(2 * q + 1) / VN][(2 * q + 1) % VN] = (T)yo;
            }
            T* dst = ptr[j];
#pragma unroll
            for (int i = 0; i < NV; ++i) {
                if (NT) __builtin_nontemporal_store(out[i], reinterpret_cast<V*>(dst + i * VN));
                else *reinterpret_cast<V*>(dst + i * VN) = out[i];
            }
        }
    }
}

// The wave-autonomous form: no workgroup barrier at all.  The packs of all tokens form one flat
// list, token-major, cut into chunks of 64 consecutive packs (a whole number of heads of one
// token: the host only takes this path when 64 packs are a whole number of heads and a token a
// whole number of chunks).  A wave takes NP consecutive chunks, requests all its packs first,
// then computes cos / sin of the one or two tokens it touches (lane i: pair i) into its own
// 512-byte LDS slots and reads its four pairs back as two 16-byte LDS loads.
template <typename T, bool BWD, int NP, bool NT>
__global__ __launch_bounds__(ROPE_THREADS) void rope_wave_kernel(
    T* __restrict__ Q, T* __restrict__ K, const int32_t* __restrict__ POS, int64_t stride_pos,
    const float* __restrict__ INV_FREQ, int64_t stride_if, int64_t total_chunks, int cpt, int Hq, int half,
    int64_t sq_t, int64_t sq_h, int64_t sk_t, int64_t sk_h, int vph, int vph_shift) {
    extern __shared__ float cs[];                     // [waves][NP slots][2][64]
    typedef typename VecOf<T>::type V;
    constexpr int VN = VecOf<T>::N, NV = 8 / VN;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    float* mine = cs + (size_t)wave * NP * 128;
    const int64_t c0 = ((int64_t)blockIdx.x * (ROPE_THREADS / 64) + wave) * NP;
    if (c0 >= total_chunks) return;
    const int64_t tok_first = c0 / cpt;
    const int rem_first = (int)(c0 - tok_first * cpt);
    const int v = lane & (vph - 1), hl = lane >> vph_shift, hpc = 64 >> vph_shift;   // heads per chunk
    V raw[NP][NV];
    T* ptr[NP];
    int slot_of[NP];
    int n_slots = 0;
    {
        int64_t tok = tok_first;
        int rem = rem_first;
#pragma unroll
        for (int j = 0; j < NP; ++j) {
            ptr[j] = nullptr;
            slot_of[j] = n_slots;
            if (c0 + j < total_chunks) {
                const int h = rem * hpc + hl;
                T* p = (h < Hq) ? (Q + tok * sq_t + (int64_t)h * sq_h) : (K + tok * sk_t + (int64_t)(h - Hq) * sk_h);
                p += v * 8;
                ptr[j] = p;
#pragma unroll
                for (int i = 0; i < NV; ++i) {
                    if (NT) raw[j][i] = __builtin_nontemporal_load(reinterpret_cast<const V*>(p + i * VN));
                    else raw[j][i] = *reinterpret_cast<const V*>(p + i * VN);
                }
                if (++rem == cpt) { rem = 0; ++tok; ++n_slots; }
            }
        }
        if (rem != 0) ++n_slots;                      // the last token touched was not completed
    }
    // cos / sin of token tok_first + s into slot s (wave-uniform trip count)
    const float f = lane < half ? INV_FREQ[lane * stride_if] : 0.f;
    for (int s = 0; s < n_slots; ++s) {
        float sn, c;
        sincosf((float)POS[(tok_first + s) * stride_pos] * f, &sn, &c);
        mine[s * 128 + lane] = c;
        mine[s * 128 + 64 + lane] = BWD ? -sn : sn;
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
    for (int j = 0; j < NP; ++j) {
        if (ptr[j] == nullptr) continue;
        const float4 c = *reinterpret_cast<const float4*>(mine + slot_of[j] * 128 + v * 4);
        const float4 sn = *reinterpret_cast<const float4*>(mine + slot_of[j] * 128 + 64 + v * 4);
        const float cc[4] = {c.x, c.y, c.z, c.w}, ss[4] = {sn.x, sn.y, sn.z, sn.w};
        float x[8];
#pragma unroll
        for (int i = 0; i < NV; ++i)
#pragma unroll
            for (int e = 0; e < VN; ++e) x[i * VN + e] = (float)raw[j][i][e];
        V out[NV];
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const float e = x[2 * q], o = x[2 * q + 1];
            out[(2 * q) / VN][(2 * q) % VN] = (T)(e * cc[q] - o * ss[q]);
            out[(2 * q + 1) / VN][(2 * q + 1) % VN] = (T)(e * ss[q] + o * cc[q]);
        }
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            if (NT) __builtin_nontemporal_store(out[i], reinterpret_cast<V*>(ptr[j] + i * VN));
            else *reinterpret_cast<V*>(ptr[j] + i * VN) = out[i];
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
    if (vec && (int64_t)(Hq + Hk) * (rot_dim >> 3) > (1 << 18)) vec = false;   // flat pack indices stay below 2^22
    if (vec) {
        // The rotation is in place.  When the launch moves more than the cache can keep anyway, loads and
        // stores are marked non-temporal: on q + k of 8192 tokens x 40 heads x 128 (168 MB moved) that is
        // 29 us against 36 us when the data comes from HBM, and 28 us against 27 us when it is cache-resident.
        const int vph = rot_dim >> 3, items = (Hq + Hk) * vph;
        const bool nt = 2.0 * (double)T_tokens * items * 8 * sizeof(T) >= (double)kStreamingBytes;
        const bool pow2 = (vph & (vph - 1)) == 0;
        if (pow2 && vph <= 64 && items % 64 == 0 && rot_dim <= 128) {
            constexpr int NP = 2;
            int shift = 0;
            while ((1 << shift) < vph) ++shift;
            const int cpt = items / 64;
            const int64_t total_chunks = T_tokens * cpt;
            const int64_t waves = (total_chunks + NP - 1) / NP;
            const unsigned grid = (unsigned)((waves + 3) / 4);
            const size_t lds = 4 * NP * 128 * sizeof(float);
#define FX_ROPE_WV(NT_)                                                                                        \
            rope_wave_kernel<T, BWD, NP, NT_><<<grid, ROPE_THREADS, lds, s>>>(                                 \
                Q, K, pos, stride_pos, inv_freq, stride_if, total_chunks, cpt, Hq, rot_dim >> 1, sq[0], sq[1], \
                Hk > 0 ? sk[0] : 0, Hk > 0 ? sk[1] : 0, vph, shift)
            if (nt) FX_ROPE_WV(true); else FX_ROPE_WV(false);
#undef FX_ROPE_WV
        } else {
            constexpr int NP = 5;
            int tpw = (NP * ROPE_THREADS) / items;            // tokens per workgroup: fill every lane's NP packs
            tpw = tpw < 1 ? 1 : (tpw > 16 ? 16 : tpw);
            const size_t lds = (size_t)tpw * (rot_dim >> 1) * 2 * sizeof(float);
            const unsigned grid = (unsigned)((T_tokens + tpw - 1) / tpw);
#define FX_ROPE_FL(NT_)                                                                                        \
            rope_flat_kernel<T, BWD, NP, NT_><<<grid, ROPE_THREADS, lds, s>>>(                                 \
                Q, K, pos, stride_pos, inv_freq, stride_if, T_tokens, Hq, rot_dim, sq[0], sq[1],               \
                Hk > 0 ? sk[0] : 0, Hk > 0 ? sk[1] : 0, tpw, vph, items, 1.0f / (float)items, 1.0f / (float)vph)
            if (nt) FX_ROPE_FL(true); else FX_ROPE_FL(false);
#undef FX_ROPE_FL
        }
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
