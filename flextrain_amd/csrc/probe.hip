// Hardware probes used by the benchmark to put the GEMM numbers in context.
//
// fx_probe_mfma_rate runs nothing but v_mfma_f32_32x32x16_bf16 on every SIMD (one workgroup of four
// waves per CU, 16 independent accumulators per wave, operands kept in registers) and reports the
// achieved rate and the shader clock during the run.  With constant operand data the matrix pipes
// reach the published peak (one MFMA per 32 cycles per SIMD at the maximum clock); with random
// operand data the power management lowers the clock, and the rate measured then is the ceiling a
// GEMM on real data can approach on this machine.  No counterpart in the reference.
#include "common.h"
#include "flexhip.h"

namespace fx {

typedef bf16 probe_bf16x8 __attribute__((ext_vector_type(8)));
typedef float probe_f32x16 __attribute__((ext_vector_type(16)));
typedef unsigned int probe_u32x4 __attribute__((ext_vector_type(4)));

__global__ __launch_bounds__(256) void mfma_rate_kernel(float* __restrict__ sink, int iters, int random_data,
                                                        unsigned long long* __restrict__ clocks) {
    probe_f32x16 acc[16];
#pragma unroll
    for (int i = 0; i < 16; ++i)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[i][v] = 0.f;
    probe_u32x4 r[8];
    unsigned h = threadIdx.x * 2654435761u + blockIdx.x * 40503u + 12345u;
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            h ^= h << 13; h ^= h >> 17; h ^= h << 5;
            // two bf16 values of magnitude 0.5 .. 2 with random sign and mantissa
            const unsigned lo = (h & 0x807fu) | 0x3f80u, hi = ((h >> 16) & 0x807fu) | 0x3f00u;
            r[i][j] = random_data ? (lo | (hi << 16)) : 0x3f803f80u;
        }
    const unsigned long long c0 = __builtin_readcyclecounter(), w0 = wall_clock64();
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int i = 0; i < 16; ++i)
            acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(*reinterpret_cast<probe_bf16x8*>(&r[i & 7]),
                                                             *reinterpret_cast<probe_bf16x8*>(&r[(i * 3 + 1) & 7]),
                                                             acc[i], 0, 0, 0);
    }
    const unsigned long long c1 = __builtin_readcyclecounter(), w1 = wall_clock64();
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < 16; ++i)
#pragma unroll
        for (int v = 0; v < 16; ++v) s += acc[i][v];
    sink[(size_t)blockIdx.x * 256 + threadIdx.x] = s;
    if (threadIdx.x == 0 && blockIdx.x == 0) {
        clocks[0] = c1 - c0;  // shader clock cycles
        clocks[1] = w1 - w0;  // constant-rate wall clock ticks
    }
}

}  // namespace fx

using namespace fx;

extern "C" size_t fx_probe_ws_bytes(void) { return (size_t)1024 * 256 * sizeof(float) + 64; }

extern "C" int fx_probe_mfma_rate(int random_data, int iters, void* ws, size_t ws_bytes, double* flop_out,
                                  hipStream_t stream) {
    if (iters <= 0 || !ws || ws_bytes < fx_probe_ws_bytes() || !flop_out) FX_FAIL("fx_probe_mfma_rate: bad arguments");
    int dev = 0, cus = 0;
    if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess)
        FX_FAIL("fx_probe_mfma_rate: cannot query the device");
    if (cus <= 0 || cus > 1024) FX_FAIL("fx_probe_mfma_rate: unexpected CU count %d", cus);
    unsigned long long* clocks = reinterpret_cast<unsigned long long*>(ws);   // first 16 bytes of ws
    float* sink = reinterpret_cast<float*>(reinterpret_cast<char*>(ws) + 64);
    mfma_rate_kernel<<<cus, 256, 0, stream>>>(sink, iters, random_data, clocks);
    FX_CHECK_LAUNCH("fx_probe_mfma_rate");
    // floating-point operations of the launch: CUs x 4 waves x iters x 16 MFMAs x (2*32*32*16)
    *flop_out = (double)cus * 4.0 * (double)iters * 16.0 * 32768.0;
    return 0;
}
