// Shared device helpers for the gfx950 (CDNA4, wave64) kernels.
//
// Element types are the three the C ABI's dtype enum names (0 = fp32, 1 = fp16,
// 2 = bf16; same numbering as the reference GEMM dispatcher,
// helpers/matmul_dispatcher/src/dispatch.cpp:19-21).  All math is done in fp32;
// the helpers here move 16 bytes per lane per access.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stddef.h>
#include <stdio.h>

namespace fx {

typedef __bf16 bf16;
typedef _Float16 f16;

enum : int { DT_F32 = 0, DT_F16 = 1, DT_BF16 = 2 };

constexpr int WAVE = 64;

#define FX_DEV __device__ __forceinline__

// ---------------------------------------------------------------------------
// 16-byte vector packs: VecOf<T>::N elements of T in one global_load_dwordx4.
// ---------------------------------------------------------------------------
template <typename T> struct VecOf;
template <> struct VecOf<float> { static constexpr int N = 4; typedef float type __attribute__((ext_vector_type(4))); };
template <> struct VecOf<bf16>  { static constexpr int N = 8; typedef bf16  type __attribute__((ext_vector_type(8))); };
template <> struct VecOf<f16>   { static constexpr int N = 8; typedef f16   type __attribute__((ext_vector_type(8))); };


// Load/store `N` consecutive elements (N * sizeof(T) must be 16 or 32 bytes and
// the address 16-byte aligned) converting to/from fp32 registers.
// NT = true marks the access non-temporal (streamed once, not kept in L2 /
// last-level cache); measured +8..10 % on large read-once/write-once tensors.
template <typename T, int N, bool NT = false>
FX_DEV void load_f32(const T* __restrict__ p, float (&out)[N]) {
    constexpr int VN = VecOf<T>::N;
    static_assert(N % VN == 0, "N must be a multiple of the 16-byte pack");
    typedef typename VecOf<T>::type V;
#pragma unroll
    for (int i = 0; i < N / VN; ++i) {
        V v;
        if (NT) v = __builtin_nontemporal_load(reinterpret_cast<const V*>(p + i * VN));
        else v = *reinterpret_cast<const V*>(p + i * VN);
#pragma unroll
        for (int j = 0; j < VN; ++j) out[i * VN + j] = (float)v[j];
    }
}

template <typename T, int N, bool NT = false>
FX_DEV void store_f32(T* __restrict__ p, const float (&in)[N]) {
    constexpr int VN = VecOf<T>::N;
    static_assert(N % VN == 0, "N must be a multiple of the 16-byte pack");
    typedef typename VecOf<T>::type V;
#pragma unroll
    for (int i = 0; i < N / VN; ++i) {
        V v;
#pragma unroll
        for (int j = 0; j < VN; ++j) v[j] = (T)in[i * VN + j];
        if (NT) __builtin_nontemporal_store(v, reinterpret_cast<V*>(p + i * VN));
        else *reinterpret_cast<V*>(p + i * VN) = v;
    }
}

// Round an fp32 value to T and back (the reference kernels round at a few
// named points; this reproduces one such rounding).
template <typename T> FX_DEV float round_to(float v) { return (float)(T)v; }

// Gated activations: out = act(x1) * x3 (flextrain/ops/_kernels/swiglu.py:34-39,
// gelu_tanh_gated.py:55-75), shared by the streaming kernels and the fused GEMM epilogue.
enum : int { ACT_SILU = 0, ACT_GELU_TANH = 1 };

FX_DEV float fast_sigmoid(float x) {
    // 1 / (1 + 2^(-x*log2 e)); v_exp_f32 + v_rcp_f32, ~1 ulp each.
    return __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-1.4426950408889634f * x));
}

template <typename T, int ACT>
FX_DEV float glu_fwd_elem(float x1, float x3) {
    if (ACT == ACT_SILU) {
        const float s = fast_sigmoid(x1);
        return (x1 * s) * x3;
    } else {
        const float cu = x1 * x1 * x1;
        const float u = 0.7978845608028654f * (x1 + 0.044715f * cu);
        const float th = 2.0f * fast_sigmoid(2.0f * u) - 1.0f;
        const float g = 0.5f * x1 * (1.0f + th);
        return g * x3;
    }
}

// Backward of the expert SwiGLU for one element (flextrain/ops/_kernels/moe.py:118-145, and the
// pre-scaled variant :189-215), shared by the row kernel and the fused dgrad epilogue so that both
// give the same bits: x3 = value, x1 = gate, d = upstream gradient of the activation, w = the row's
// router weight.  Returns the element's term of the router-weight gradient.
FX_DEV float precise_sigmoid(float x) { return 1.0f / (1.0f + expf(-x)); }

template <bool PRESCALED>
FX_DEV float moe_swiglu_bwd_elem(float x3, float x1, float d, float w, float w_inv, float& dx3, float& dx1, float& act) {
    const float s = precise_sigmoid(x1);
    const float silu = x1 * s;
    const float un = silu * x3;
    const float ds = s + silu * (1.0f - s);
    if (PRESCALED) {
        act = un;
        dx3 = d * silu;
        dx1 = d * x3 * ds;
        return (d * w_inv) * un;
    } else {
        act = un * w;
        const float dsc = d * w;
        dx3 = dsc * silu;
        dx1 = dsc * x3 * ds;
        return d * un;
    }
}

// ---------------------------------------------------------------------------
// Reductions.  `W` lanes (power of two, <= 64) that are contiguous in the wave
// cooperate; every lane of the group ends with the group's sum.
// ---------------------------------------------------------------------------
template <int W>
FX_DEV float group_sum(float v) {
#pragma unroll
    for (int off = W / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    return v;
}
template <int W>
FX_DEV float group_max(float v) {
#pragma unroll
    for (int off = W / 2; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, 64));
    return v;
}

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// Tensors streamed through a kernel exactly once bypass the caches when the
// launch moves more than this many bytes (smaller working sets are likely to be
// consumed from cache by the next kernel).
constexpr size_t kStreamingBytes = (size_t)96 << 20;

inline int elem_size(int dt) { return dt == DT_F32 ? 4 : 2; }

// More than 64 KB of dynamic LDS has to be asked for, once per kernel AND device.  One bit per
// device at each call site; racing host threads at worst repeat the (idempotent) call.
#define FX_ENSURE_DYNAMIC_LDS(kern, bytes)                                                          \
    do {                                                                                           \
        static unsigned long long done__ = 0ull;                                                   \
        int dev__ = 0;                                                                             \
        (void)hipGetDevice(&dev__);                                                                \
        if (dev__ < 0 || dev__ >= 64 || !((done__ >> dev__) & 1ull)) {                             \
            (void)hipFuncSetAttribute(reinterpret_cast<const void*>(kern),                         \
                                      hipFuncAttributeMaxDynamicSharedMemorySize, (int)(bytes));   \
            if (dev__ >= 0 && dev__ < 64) done__ |= 1ull << dev__;                                 \
        }                                                                                          \
    } while (0)

#define FX_CHECK_LAUNCH(name)                                                        \
    do {                                                                             \
        hipError_t e__ = hipGetLastError();                                          \
        if (e__ != hipSuccess) {                                                     \
            fprintf(stderr, "flexhip: %s launch failed: %s\n", name,                 \
                    hipGetErrorString(e__));                                         \
            return -1;                                                               \
        }                                                                            \
    } while (0)

#define FX_FAIL(...)                                                                 \
    do {                                                                             \
        fprintf(stderr, "flexhip: " __VA_ARGS__);                                    \
        fprintf(stderr, "\n");                                                       \
        return -1;                                                                   \
    } while (0)

// Dispatch a callable templated on element type from a runtime dtype enum.
#define FX_DISPATCH_DTYPE(dt, T, ...)                                                \
    switch (dt) {                                                                    \
        case fx::DT_F32:  { typedef float T;    __VA_ARGS__; break; }                \
        case fx::DT_F16:  { typedef fx::f16 T;  __VA_ARGS__; break; }                \
        case fx::DT_BF16: { typedef fx::bf16 T; __VA_ARGS__; break; }                \
        default: FX_FAIL("unsupported dtype enum %d", (int)(dt));                    \
    }

}  // namespace fx
