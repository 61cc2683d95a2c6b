// Types shared by the MFMA GEMM code for gfx950: fragment and accumulator vectors, the
// v_mfma_f32_32x32x16 wrappers, the K-step width and the operand view (the tile code itself is in
// gemm_core2.h).
#pragma once
#include "common.h"

namespace fx {

typedef bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef f16 f16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x16_t __attribute__((ext_vector_type(16)));
typedef unsigned int u32x4_t __attribute__((ext_vector_type(4)));

template <typename T> struct Mfma32;
template <> struct Mfma32<bf16> {
    typedef bf16x8_t frag;
    static FX_DEV f32x16_t run(frag a, frag b, f32x16_t c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
    }
};
template <> struct Mfma32<f16> {
    typedef f16x8_t frag;
    static FX_DEV f32x16_t run(frag a, frag b, f32x16_t c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
    }
};

constexpr int GEMM_BK = 64;
constexpr int GEMM_THREADS = 256;

// One operand of one workgroup tile.
//   base : element pointer to the operand matrix of this problem
//   ld   : leading dimension in elements
//   ext  : extent along the tile's m (or n) axis, rows at or beyond it are never stored
//   origin: first m (or n) index of this tile
template <typename T>
struct OperandView {
    const T* base;
    int64_t ld;
    int ext;
    int origin;
    // Two-matrix tile (loaders instantiated with DUAL): tile rows alternate between the two matrices
    // in blocks of `half` (a power of two): rows [0, half) are indices origin + [0, half) of `base`,
    // rows [half, 2 half) the same indices of `base2` (same ld and extent), rows [2 half, 3 half)
    // indices origin + [half, 2 half) of `base` again, and so on.
    int half = 0;
    const T* base2 = nullptr;
    // Gathered rows (K-contiguous A tiles of the loaders that say so): tile row r is row
    // row_map[origin + r] of `base` instead of row origin + r.
    const int32_t* row_map = nullptr;
    int map_rows = 0;          // rows of `base` a gathered tile may address: map entries are clamped to [0, map_rows)
    // Gathered k-rows (M/N-contiguous tiles of the loaders that say so): k-row k of the operand is row
    // k_map[k] of `base` instead of row k, for k in [0, k_ext).  The expert weight gradients read the
    // unsorted activations that way: their contraction runs over an expert's rows.
    const int32_t* k_map = nullptr;
    int k_ext = 0;
    // tile row -> which matrix, and the index offset from `origin`
    __device__ __forceinline__ bool dual_second(int r) const { return (r & half) != 0; }
    __device__ __forceinline__ int dual_index(int r) const { return ((r & ~(2 * half - 1)) >> 1) + (r & (half - 1)); }
};

FX_DEV u32x4_t ldg16(const void* p) { return *reinterpret_cast<const u32x4_t*>(p); }

}  // namespace fx
