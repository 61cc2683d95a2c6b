// Host stand-in for <hip/hip_runtime.h>: the device code of this package's non-MFMA kernels compiled as
// ordinary C++ and run on the CPU, one workgroup at a time, every GPU lane a cooperative fiber.
//
// What it is for: running the real kernel source (and the real host-side launch code: grid sizes, kernel
// selection, workspace use) against buffers that end at inaccessible guard pages, so that an access one
// element outside any operand kills the test, and comparing results with the CPU oracle.  Test
// infrastructure only: nothing in the package includes it.
//
// Execution model: a launch runs its workgroups in order; a workgroup's lanes are fibers that
// run until they meet a workgroup barrier, a wave-level exchange or their end.  __syncthreads() releases
// when every lane still alive has arrived; wave operations exchange through one slot per lane.  Lanes
// that returned count as arrived (on the GPU their wave either left the barrier's count or carries them
// masked off).  __shared__ variables are statics: one workgroup exists at a time.
#pragma once
#include <algorithm>
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <functional>
#include <vector>

#define __global__
#define __device__
#define __host__
#define __forceinline__ inline
#define __launch_bounds__(...)
#define __shared__ static
#define __align__(n) __attribute__((aligned(n)))
#define HIP_SYMBOL(x) (&(x))

using std::max;
using std::min;

struct dim3 {
    unsigned x, y, z;
    dim3(unsigned a = 1, unsigned b = 1, unsigned c = 1) : x(a), y(b), z(c) {}
};
struct alignas(16) float4 { float x, y, z, w; };
struct alignas(8) float2 { float x, y; };
struct alignas(16) int4 { int x, y, z, w; };
struct alignas(8) uint2 { unsigned x, y; };
struct alignas(16) uint4 { unsigned x, y, z, w; };
inline float4 make_float4(float x, float y, float z, float w) { return float4{x, y, z, w}; }
inline float2 make_float2(float x, float y) { return float2{x, y}; }
inline uint2 make_uint2(unsigned x, unsigned y) { return uint2{x, y}; }
typedef void* hipStream_t;
typedef int hipError_t;
enum { hipSuccess = 0, hipErrorInvalidValue = 1 };
enum { hipFuncAttributeMaxDynamicSharedMemorySize = 8, hipDeviceAttributeMultiprocessorCount = 63 };
inline hipError_t hipGetLastError() { return hipSuccess; }
inline const char* hipGetErrorString(hipError_t e) { return e == 2 ? "stream order violation (host simulation)" : "host simulation"; }
inline hipError_t hipGetDevice(int* d) { *d = 0; return hipSuccess; }
inline hipError_t hipDeviceGetAttribute(int* v, int, int) { *v = 256; return hipSuccess; }
template <typename F> inline hipError_t hipFuncSetAttribute(F, int, int) { return hipSuccess; }
template <typename T> inline hipError_t hipGetSymbolAddress(void** out, T* sym) { *out = (void*)sym; return hipSuccess; }

// Copies, events and pinned memory for the streaming code: everything completes at the call (one of the
// orders the streams allow).  What events and waits still do is bookkeeping: every stream carries a vector
// clock (order.cpp), copies declare the bytes they read and write, and a copy that is not ordered after an
// earlier overlapping access on another stream fails like a failed HIP call.
extern "C" {
uint64_t hostsim_order_snapshot(uint64_t stream);
void hostsim_order_wait(uint64_t stream, uint64_t handle);
int hostsim_order_enqueue(uint64_t stream, const char* what, int n, const uint64_t* lo, const uint64_t* bytes, const int* is_write);
}
enum { hipErrorStreamOrder = 2 };
struct hostsim_event { uint64_t snapshot; };
typedef struct hostsim_event* hipEvent_t;
enum hipMemcpyKind { hipMemcpyHostToDevice = 1, hipMemcpyDeviceToHost = 2, hipMemcpyDeviceToDevice = 3 };
enum { hipEventDisableTiming = 2, hipHostMallocDefault = 0 };
inline hipError_t hostsim_declare(hipStream_t stream, const char* what, const void* read, size_t read_bytes, void* write, size_t write_bytes) {
    const uint64_t lo[2] = {(uint64_t)(uintptr_t)read, (uint64_t)(uintptr_t)write}, bytes[2] = {read_bytes, write_bytes};
    const int is_write[2] = {0, 1};
    return hostsim_order_enqueue((uint64_t)(uintptr_t)stream, what, 2, lo, bytes, is_write) ? hipErrorStreamOrder : hipSuccess;
}
inline hipError_t hipMemcpyAsync(void* dst, const void* src, size_t n, hipMemcpyKind, hipStream_t stream) {
    const hipError_t e = hostsim_declare(stream, "copy", src, n, dst, n);
    memcpy(dst, src, n);
    return e;
}
inline hipError_t hipMemcpy2DAsync(void* dst, size_t dpitch, const void* src, size_t spitch, size_t width, size_t height, hipMemcpyKind,
                                   hipStream_t stream) {
    const hipError_t e = height ? hostsim_declare(stream, "2-D copy", src, (height - 1) * spitch + width, dst, (height - 1) * dpitch + width)
                                : hipSuccess;
    for (size_t r = 0; r < height; ++r) memcpy((char*)dst + r * dpitch, (const char*)src + r * spitch, width);
    return e;
}
inline hipError_t hipEventCreateWithFlags(hipEvent_t* e, unsigned) { *e = new hostsim_event{0}; return hipSuccess; }
inline hipError_t hipEventDestroy(hipEvent_t e) { delete e; return hipSuccess; }
inline hipError_t hipEventRecord(hipEvent_t e, hipStream_t s) { e->snapshot = hostsim_order_snapshot((uint64_t)(uintptr_t)s); return hipSuccess; }
inline hipError_t hipStreamWaitEvent(hipStream_t s, hipEvent_t e, unsigned) { hostsim_order_wait((uint64_t)(uintptr_t)s, e->snapshot); return hipSuccess; }
inline hipError_t hipHostMalloc(void** p, size_t n, unsigned) { *p = malloc(n); return *p ? hipSuccess : hipErrorInvalidValue; }
inline hipError_t hipHostFree(void* p) { free(p); return hipSuccess; }

namespace hostsim {

struct Idx { unsigned x, y, z; };
extern Idx g_thread, g_block;
extern dim3 g_block_dim, g_grid_dim;
extern unsigned char* g_dynamic_lds;

void launch(dim3 grid, dim3 block, size_t lds_bytes, const std::function<void()>& body);
void sync_threads();
void sync_wave();
unsigned lane_slot();                     // index of the running lane's exchange slot
extern uint64_t g_exchange[];             // one 8-byte slot per lane of the workgroup
extern unsigned char g_alive[];           // 1 while the lane has not returned
unsigned flat_thread();

template <typename T>
inline T exchange(T v, int src_lane_in_wave) {
    static_assert(sizeof(T) <= 8, "exchange slot");
    const unsigned me = flat_thread();
    const unsigned wave0 = me & ~63u;
    uint64_t raw = 0;
    memcpy(&raw, &v, sizeof(T));
    g_exchange[me] = raw;
    sync_wave();
    T out = v;
    const unsigned src = wave0 + (unsigned)src_lane_in_wave;
    if (src_lane_in_wave >= 0 && src_lane_in_wave < 64 && src < g_block_dim.x * g_block_dim.y * g_block_dim.z && g_alive[src])
        memcpy(&out, &g_exchange[src], sizeof(T));
    sync_wave();
    return out;
}

}  // namespace hostsim

#define threadIdx hostsim::g_thread
#define blockIdx hostsim::g_block
#define blockDim hostsim::g_block_dim
#define gridDim hostsim::g_grid_dim

inline void __syncthreads() { hostsim::sync_threads(); }
template <typename T> inline T __shfl_xor(T v, int mask, int width = 64) { (void)width; return hostsim::exchange(v, (int)((hostsim::flat_thread() & 63u) ^ (unsigned)mask)); }
template <typename T> inline T __shfl_up(T v, unsigned delta, int width = 64) {
    (void)width;
    const int lane = (int)(hostsim::flat_thread() & 63u);
    return hostsim::exchange(v, lane - (int)delta >= 0 ? lane - (int)delta : lane);
}
template <typename T> inline T __shfl_down(T v, unsigned delta, int width = 64) {
    (void)width;
    const int lane = (int)(hostsim::flat_thread() & 63u);
    return hostsim::exchange(v, lane + (int)delta < 64 ? lane + (int)delta : lane);
}
template <typename T> inline T __shfl(T v, int src, int width = 64) { (void)width; return hostsim::exchange(v, src); }
inline int __any(int pred) {
    const unsigned me = hostsim::flat_thread(), wave0 = me & ~63u;
    const unsigned lanes = hostsim::g_block_dim.x * hostsim::g_block_dim.y * hostsim::g_block_dim.z;
    hostsim::g_exchange[me] = pred != 0;
    hostsim::sync_wave();
    int any = 0;
    for (unsigned l = wave0; l < wave0 + 64 && l < lanes; ++l) any |= hostsim::g_alive[l] && hostsim::g_exchange[l] != 0;
    hostsim::sync_wave();
    return any;
}
template <typename T> inline T atomicAdd(T* p, T v) { T old = *p; *p = old + v; return old; }      // fibers never preempt each other
template <typename T> inline T atomicOr(T* p, T v) { T old = *p; *p = old | v; return old; }
template <typename T> inline T atomicMax(T* p, T v) { T old = *p; *p = std::max(old, v); return old; }

namespace hostsim {
extern float (*g_wave_f32)[64][16];             // [wave][lane][8 of A, 8 of B]: operands published for a matrix instruction

// global_load_lds_dwordx4: lane l of the wave copies 16 bytes from its global address to lds_addr + 16 l.
// The copy is made as LATE as the hardware may make it: it is queued, and lands only when the lane's own
// `s_waitcnt vmcnt(n)` leaves at most n of its loads in flight (oldest first).  A kernel that reads a buffer
// before its counted wait has covered the loads that fill it, or re-uses a buffer that loads are still in
// flight to, computes from stale or overwritten data here and fails its comparison.  (Counting these loads
// alone is the weaker guarantee: other vector memory operations in the window only make the real wait cover
// more.)  Loads never waited for are dropped when the workgroup ends.
struct PendingDma { unsigned lds; const void* src; };
constexpr int kMaxPendingDma = 64;
extern PendingDma g_dma[][kMaxPendingDma];
extern int g_dma_first[], g_dma_count[];
extern int g_dma_eager;     // 1: the other extreme, every copy lands at its issue (a load into a buffer that
                            // lanes scheduled later still have to read then shows as wrong results)
inline void lds_dma16(unsigned lds_addr, const void* gptr) {
    const unsigned me = flat_thread();
    if (g_dma_eager) { memcpy(reinterpret_cast<void*>((uintptr_t)lds_addr + 16u * (me & 63u)), gptr, 16); return; }
    if (g_dma_count[me] == kMaxPendingDma) { fprintf(stderr, "hostsim: more than %d LDS loads in flight in one lane\n", kMaxPendingDma); abort(); }
    g_dma[me][(g_dma_first[me] + g_dma_count[me]++) % kMaxPendingDma] = PendingDma{lds_addr + 16u * (me & 63u), gptr};
}
inline void wait_vmcnt(int n) {
    const unsigned me = flat_thread();
    while (g_dma_count[me] > n) {
        const PendingDma& d = g_dma[me][g_dma_first[me]];
        memcpy(reinterpret_cast<void*>((uintptr_t)d.lds), d.src, 16);
        g_dma_first[me] = (g_dma_first[me] + 1) % kMaxPendingDma;
        --g_dma_count[me];
    }
}

// v_mfma_f32_32x32x16 (bf16 / f16): D = A (32 x 16) * B (16 x 32) + C.  Lane l supplies A[l % 32][8 (l / 32) .. + 7]
// and B[8 (l / 32) .. + 7][l % 32]; register v of lane l is D[8 (v / 4) + 4 (l / 32) + v % 4][l % 32].
template <typename Frag, typename Acc>
inline Acc mfma32x32x16(Frag a, Frag b, Acc c) {
    const unsigned me = flat_thread(), w = me >> 6, l = me & 63u;
    float* mine = g_wave_f32[w][l];
    for (int j = 0; j < 8; ++j) { mine[j] = (float)a[j]; mine[8 + j] = (float)b[j]; }
    sync_wave();
    const float* b_lo = g_wave_f32[w][l % 32] + 8;            // B[0 .. 7][col], B[8 .. 15][col]
    const float* b_hi = g_wave_f32[w][l % 32 + 32] + 8;
    for (int v = 0; v < 16; ++v) {
        const unsigned row = 8u * (v / 4) + 4u * (l / 32) + (unsigned)(v % 4);
        const float* a_lo = g_wave_f32[w][row];
        const float* a_hi = g_wave_f32[w][row + 32];
        float sum = c[v];
        for (int k = 0; k < 8; ++k) sum += a_lo[k] * b_lo[k];
        for (int k = 0; k < 8; ++k) sum += a_hi[k] * b_hi[k];
        c[v] = sum;
    }
    sync_wave();
    return c;
}

// ds_read_b64_tr_b16: inside each group of 16 lanes, lane s receives, for j = 0 .. 3, element s % 4 of the
// 8 bytes that lane 4 j + s / 4 of the group addressed.
template <typename V4>
inline V4 ds_read_tr16(const void* addr) {
    const unsigned me = flat_thread(), group0 = me & ~15u, s = me & 15u;
    g_exchange[me] = (uint64_t)(uintptr_t)addr;
    sync_wave();
    V4 out;
    for (unsigned j = 0; j < 4; ++j) {
        const short* src = reinterpret_cast<const short*>((uintptr_t)g_exchange[group0 + 4 * j + s / 4]);
        out[j] = src[s % 4];
    }
    sync_wave();
    return out;
}

// v_perm_b32: byte i of the result is byte sel[i] of the 8 bytes {hi : lo} (0-3 from lo, 4-7 from hi).
inline unsigned perm_b32(unsigned hi, unsigned lo, unsigned sel) {
    const uint64_t both = ((uint64_t)hi << 32) | lo;
    unsigned out = 0;
    for (int i = 0; i < 4; ++i) out |= (unsigned)((both >> (8 * ((sel >> (8 * i)) & 7))) & 0xff) << (8 * i);
    return out;
}
}  // namespace hostsim

#define __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, x, y, z) hostsim::mfma32x32x16(a, b, c)
#define __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, x, y, z) hostsim::mfma32x32x16(a, b, c)
#define __builtin_amdgcn_ds_read_tr16_b64_v4i16(p) hostsim::ds_read_tr16<short __attribute__((ext_vector_type(4)))>((const void*)(p))
#define __builtin_amdgcn_perm(hi, lo, sel) hostsim::perm_b32(hi, lo, sel)

// gfx950 builtins the kernels use, by their documented meaning
#define __builtin_amdgcn_rcpf(x) (1.0f / (x))
#define __builtin_amdgcn_exp2f(x) exp2f(x)
#define __builtin_amdgcn_readfirstlane(x) (x)          /* only ever applied to wave-uniform values */
#define __builtin_amdgcn_wave_barrier() hostsim::sync_wave()
#define __builtin_amdgcn_fence(...) ((void)0)
#define __builtin_amdgcn_sched_barrier(x) ((void)0)
#define __builtin_amdgcn_s_setprio(x) ((void)0)
inline float rsqrtf(float x) { return 1.0f / sqrtf(x); }
#define __expf(x) expf(x)
#define __logf(x) logf(x)
