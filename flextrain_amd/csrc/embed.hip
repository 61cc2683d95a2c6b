// Embedding backward: grad_weight[token] += scale * sum of the grad_output rows that looked the
// token up, gfx950.  Semantics: flextrain/ops/_kernels/embed.py:5-76 (kernel) and :79-122 (wrapper):
// the caller sorts the token ids; position s of the sorted order starts a segment when its token
// differs from the one before it, and the workgroup of that position sums the whole run of equal
// tokens in fp32 (in sorted order), multiplies by scale and adds the result to the weight-gradient
// row, which is read and written in its own dtype.  Positions inside a run exit at once, so no two
// workgroups ever write the same row: no atomics, and the result is reproducible for a given sort.
#include "common.h"
#include "flexhip.h"

namespace fx {

template <typename TG, typename TW, typename TI>
__global__ __launch_bounds__(256) void embedding_bwd_kernel(
    const TG* __restrict__ GO, TW* __restrict__ GW, const TI* __restrict__ SORTED_POS,
    const TI* __restrict__ SORTED_TOK, int64_t T, int D, int64_t go_row, int64_t go_col, int64_t gw_row,
    int64_t gw_col, float scale, int64_t V, bool vec) {
    const int64_t s = blockIdx.x;
    const int64_t tok = (int64_t)SORTED_TOK[s];
    if (s > 0 && (int64_t)SORTED_TOK[s - 1] == tok) return;  // not the first of its run
    if (tok < 0 || tok >= V) return;                          // an id outside the table has no row
    int64_t end = s + 1;
    while (end < T && (int64_t)SORTED_TOK[end] == tok) ++end;
    if (vec) {
        for (int c = threadIdx.x * 8; c < D; c += 256 * 8) {
            float acc[8];
#pragma unroll
            for (int j = 0; j < 8; ++j) acc[j] = 0.f;
            for (int64_t i = s; i < end; ++i) {
                float v[8];
                load_f32<TG, 8>(GO + (int64_t)SORTED_POS[i] * go_row + c, v);
#pragma unroll
                for (int j = 0; j < 8; ++j) acc[j] += v[j];
            }
            float w[8];
            TW* dst = GW + tok * gw_row + c;
            load_f32<TW, 8>(dst, w);
#pragma unroll
            for (int j = 0; j < 8; ++j) w[j] += acc[j] * scale;
            store_f32<TW, 8>(dst, w);
        }
    } else {
        for (int c = threadIdx.x; c < D; c += 256) {
            float acc = 0.f;
            for (int64_t i = s; i < end; ++i) acc += (float)GO[(int64_t)SORTED_POS[i] * go_row + (int64_t)c * go_col];
            TW* dst = GW + tok * gw_row + (int64_t)c * gw_col;
            *dst = (TW)((float)*dst + acc * scale);
        }
    }
}

}  // namespace fx

using namespace fx;

extern "C" int fx_embedding_bwd(const void* grad_out, const void* sorted_pos, const void* sorted_tokens,
                                int indices_are_int64, void* grad_weight, int64_t T, int D, int64_t V,
                                int64_t go_row_stride, int64_t go_col_stride, int64_t gw_row_stride,
                                int64_t gw_col_stride, float scale, int go_dt, int gw_dt, hipStream_t stream) {
    if (T < 0 || D <= 0 || V <= 0) FX_FAIL("fx_embedding_bwd: bad shape");
    if (T == 0) return 0;
    if (!grad_out || !sorted_pos || !sorted_tokens || !grad_weight) FX_FAIL("fx_embedding_bwd: null pointer");
    const bool vec = go_col_stride == 1 && gw_col_stride == 1 && (D % 8) == 0 && (go_row_stride % 8) == 0 &&
                     (gw_row_stride % 8) == 0 && aligned16(grad_out) && aligned16(grad_weight);
#define FX_EMB(TI)                                                                                              \
    FX_DISPATCH_DTYPE(go_dt, TG,                                                                                \
        FX_DISPATCH_DTYPE(gw_dt, TW,                                                                            \
            embedding_bwd_kernel<TG, TW, TI><<<(unsigned)T, 256, 0, stream>>>(                                  \
                reinterpret_cast<const TG*>(grad_out), reinterpret_cast<TW*>(grad_weight),                      \
                reinterpret_cast<const TI*>(sorted_pos), reinterpret_cast<const TI*>(sorted_tokens), T, D,      \
                go_row_stride, go_col_stride, gw_row_stride, gw_col_stride, scale, V, vec)))
    if (indices_are_int64) { FX_EMB(int64_t); } else { FX_EMB(int32_t); }
#undef FX_EMB
    FX_CHECK_LAUNCH("fx_embedding_bwd");
    return 0;
}
