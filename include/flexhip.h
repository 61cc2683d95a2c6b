/* flexhip: C ABI of the MI355X (gfx950) per-layer training compute path.
 *
 * One shared library, libflexhip.so, exports everything below.  Conventions,
 * shared by every entry point unless its comment says otherwise:
 *   - plain pointers and sizes only; device pointers are raw HIP addresses;
 *   - the caller owns every buffer, including scratch ("ws") buffers whose
 *     size the matching *_ws_bytes() function reports; the library never
 *     allocates or frees device memory;
 *   - work is enqueued on the given stream and the call returns without
 *     synchronising;
 *   - dtype enums: 0 = fp32, 1 = fp16, 2 = bf16
 *     (numbering of helpers/matmul_dispatcher/src/dispatch.cpp:19-21);
 *   - return 0 on success, -1 on failure with one line on stderr
 *     (convention of helpers/matmul_dispatcher/src/dispatch.cpp:193-197).
 *
 * Each declaration cites the reference interface it stands in for; paths are
 * relative to the root of als244/flextrain.
 */
#ifndef FLEXHIP_H
#define FLEXHIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#ifndef __HIP__
typedef struct ihipStream_t* hipStream_t;
#endif

#define FX_DT_F32 0
#define FX_DT_F16 1
#define FX_DT_BF16 2

#define FX_ACT_SILU 0
#define FX_ACT_GELU_TANH 1

/* Library identification: returns a static string "flexhip <version> gfx950".  No counterpart in the
 * reference (its kernels are Python functions); lets a binding check what it loaded. */
const char* fx_version(void);

/* ---- RMSNorm ----------------------------------------------------------- */

/* flextrain_rmsnorm_fwd and flextrain_rmsnorm_fwd_recompute
 * (flextrain/ops/_kernels/rmsnorm.py:456-530, :532-583; kernels :9-163).
 * x, y: (rows, ncols) contiguous, same dtype x_dt; y may alias x.  w: (ncols,)
 * of dtype w_dt or NULL.  rstd: fp32 (rows,), written when use_saved_rstd == 0
 * and read when it is 1.  Per-head normalisation is the call with
 * rows = T*H, ncols = head_dim. */
int fx_rmsnorm_fwd(const void* x, const void* w, void* y, float* rstd, int64_t rows, int ncols,
                   float eps, int x_dt, int w_dt, int use_saved_rstd, hipStream_t stream);

/* Scratch bytes fx_rmsnorm_bwd needs for its dW partial sums (0 when the
 * shape takes the unvectorised path).  Replaces the torch.empty partial buffer
 * of flextrain/ops/_kernels/rmsnorm.py:786-789. */
size_t fx_rmsnorm_bwd_ws_bytes(int64_t rows, int ncols);

/* flextrain_rmsnorm_bwd (flextrain/ops/_kernels/rmsnorm.py:585-832; kernels
 * :170-412).  dy, x, dx, y_out share dtype x_dt.  accumulate_dx: dx += result.
 * dw (dtype dw_dt, (ncols,)) is written, or added to when accumulate_dw; pass
 * dw = NULL or w = NULL to skip the weight gradient.  y_out != NULL
 * re-materialises the forward output. */
int fx_rmsnorm_bwd(const void* dy, const void* x, const void* w, const float* rstd, void* dx,
                   int accumulate_dx, void* dw, int dw_dt, int accumulate_dw, void* y_out,
                   int64_t rows, int ncols, int x_dt, int w_dt, float* ws, size_t ws_bytes,
                   hipStream_t stream);

/* ---- Rotary embedding -------------------------------------------------- */

/* flextrain_rope_fwd / flextrain_rope_bwd (flextrain/ops/_kernels/rope.py:207-307;
 * kernels :8-157) and, with rot_dim < D, flextrain_rope_partial_fwd/bwd
 * (flextrain/ops/_kernels/rope_partial.py:29-147).  In place on q (T,Hq,D) and
 * k (T,Hk,D); k may be NULL with Hk = 0.  Strides are in elements, three per
 * tensor (token, head, channel).  pos: int32, element t at pos[t*stride_pos];
 * inv_freq: fp32, pair i at inv_freq[i*stride_if], rot_dim/2 entries. */
int fx_rope(void* q, void* k, const int32_t* pos, int64_t stride_pos, const float* inv_freq,
            int64_t stride_if, int64_t T_tokens, int Hq, int Hk, int D, int rot_dim,
            const int64_t* q_strides, const int64_t* k_strides, int dt, int backward,
            hipStream_t stream);

/* ---- Gated activations ------------------------------------------------- */

/* flextrain_swiglu_fwd (flextrain/ops/_kernels/swiglu.py:103-133) for
 * act = FX_ACT_SILU and flextrain_gelu_tanh_gated_fwd
 * (flextrain/ops/_kernels/gelu_tanh_gated.py:148-170) for FX_ACT_GELU_TANH.
 * out[i] = act(x1[i]) * x3[i] over n contiguous elements. */
int fx_glu_fwd(const void* x1, const void* x3, void* out, int64_t n, int in_dt, int out_dt, int act,
               hipStream_t stream);

/* flextrain_swiglu_bwd (flextrain/ops/_kernels/swiglu.py:136-182) and
 * flextrain_gelu_tanh_gated_bwd (flextrain/ops/_kernels/gelu_tanh_gated.py:173-214).
 * act_out != NULL also stores the recomputed forward output. */
int fx_glu_bwd(const void* x1, const void* x3, const void* dout, void* dx1, void* dx3, void* act_out,
               int64_t n, int dt, int act, hipStream_t stream);

/* flextrain_silu_bwd (flextrain/ops/_kernels/silu_bwd.py:38-67; kernel :16-35):
 * din[i] = dout[i] * s * (1 + z[i] * (1 - s)), s = sigmoid(z[i]); n contiguous elements of dtype dt;
 * din may alias z or dout. */
int fx_silu_bwd(const void* z, const void* dout, void* din, int64_t n, int dt, hipStream_t stream);

/* flextrain_embedding_bwd (flextrain/ops/_kernels/embed.py:79-122; kernel :5-76).  sorted_tokens: the T
 * looked-up ids in ascending order; sorted_pos[s]: the row of grad_out (T, D) that sorted position s
 * came from (both int32, or int64 when indices_are_int64).  grad_weight (V, D) row `token` gets
 * += scale * (fp32 sum of its grad_out rows).  Strides in elements.  Ids outside [0, V) are skipped. */
int fx_embedding_bwd(const void* grad_out, const void* sorted_pos, const void* sorted_tokens, int indices_are_int64,
                     void* grad_weight, int64_t T, int D, int64_t V, int64_t go_row_stride, int64_t go_col_stride,
                     int64_t gw_row_stride, int64_t gw_col_stride, float scale, int go_dt, int gw_dt,
                     hipStream_t stream);

/* ---- AdamW ------------------------------------------------------------- */

/* flextrain_adamw_step (flextrain/ops/_kernels/adamw.py:62-102; kernel :5-60).
 * p (p_dt), m and v (state_dt) are updated in place; g has dtype g_dt.
 * bias_correction{1,2} = 1 - beta^max(1,step), computed by the caller in
 * double.  p_bf16_out, when not NULL, additionally receives bf16(p_new); the
 * reference has no such output (its engine re-casts during the copy back to
 * the host, flextrain/engine/buffers.py:1144-1164). */
int fx_adamw_step(void* p, const void* g, void* m, void* v, void* p_bf16_out, int64_t n, int p_dt,
                  int g_dt, int state_dt, float lr, float beta1, float beta2, float eps,
                  float weight_decay, float bias_correction1, float bias_correction2,
                  hipStream_t stream);

/* The check_error branch of flextrain_adamw_step
 * (flextrain/ops/_kernels/adamw.py:80-83): ORs 1 into *flag (device int32,
 * caller-zeroed) if any element of x is NaN or infinite. */
int fx_nonfinite_flag(const void* x, int64_t n, int dt, int* flag, hipStream_t stream);

/* ---- MoE routing --------------------------------------------------------- */

/* flextrain_fused_topk_softmax (flextrain/ops/_kernels/moe.py:848-943; kernel
 * :218-314).  logits (T,E) contiguous; ids_out int32 (T,K); weights_out (T,K)
 * of dtype weights_dt.  mode 0 = topk_then_softmax, 1 = softmax_then_topk.
 * Ties go to the smallest expert index; slots are in descending value order. */
int fx_topk_softmax(const void* logits, int32_t* ids_out, void* weights_out, int64_t T, int E, int K,
                    int logits_dt, int weights_dt, int mode, hipStream_t stream);

/* Scratch bytes for fx_moe_sort (replaces block_counts / block_accum /
 * total_counts / expert_starts / offsets, flextrain/ops/_kernels/moe.py:679-758). */
size_t fx_moe_sort_ws_bytes(int64_t n_pairs, int E);

/* flextrain_moe_sort (flextrain/ops/_kernels/moe.py:649-783) fused with
 * flextrain_copy_expert_counts (:787-834).  ids: n_pairs = T*K flat expert ids
 * (int32, or int64 when ids_are_int64).  index_out[i] = row of pair i in the
 * expert-grouped order (stable).  counts_out (device, E int32) and counts_host
 * (pinned host memory mapped into the device, E int32) are optional.  An id outside [0, E) is a
 * caller error the reference does not define: here it is not counted and its pair is mapped to
 * row 0, so that scatters and gathers through the map stay inside their buffers. */
int fx_moe_sort(const void* ids, int ids_are_int64, int64_t n_pairs, int E, void* index_out,
                int index_is_int64, int32_t* counts_out, int32_t* counts_host, void* ws, size_t ws_bytes,
                hipStream_t stream);

/* No counterpart in the reference.  fx_moe_sort for callers that cannot allocate device memory or
 * lend a workspace sized per call: code under HIP graph capture, tight serving loops, harnesses
 * that forbid allocation.  Same arguments and results as fx_moe_sort without `ws`: the chunk
 * histograms, totals and starts live in a fixed device array inside the library (8 MiB + 4 KiB per
 * GPU, held until the process ends).  Limit: E * ceil(n_pairs / 256) + 2 * E <=
 * fx_moe_sort_noalloc_max_words() (= 2 * 1024 * 1024 + 1024, e.g. 1 Mi pairs over 512 experts);
 * larger problems return -1 with a message.  Calls no allocator.  All calls on one GPU share that
 * GPU's array: calls that overlap on one GPU (different streams, or threads) race; calls on one
 * stream are ordered and need nothing cleared between them.  fx_moe_sort_noalloc_init() resolves
 * the array's device address for the current GPU ahead of time (it is otherwise resolved on the
 * first call on each GPU, which must then happen outside graph capture). */
size_t fx_moe_sort_noalloc_max_words(void);
int fx_moe_sort_noalloc_init(void);
int fx_moe_sort_noalloc(const void* ids, int ids_are_int64, int64_t n_pairs, int E, void* index_out,
                        int index_is_int64, int32_t* counts_out, int32_t* counts_host, hipStream_t stream);

/* flextrain_copy_expert_counts (flextrain/ops/_kernels/moe.py:787-834; kernel
 * :498-505): a kernel copies n int32 from device memory to dst, which may be
 * pinned host memory (zero-copy store). */
int fx_copy_i32(const int32_t* src_dev, int32_t* dst, int n, hipStream_t stream);

/* flextrain_moe_router_gate_bwd (flextrain/ops/_kernels/moe.py:1527-1655;
 * kernel :360-458).  dlogits (T,E) is accumulated into.  dprobs is indexed
 * through indices (T,K); probs (T,K); logits (T,E) only for mode 1. */
int fx_router_gate_bwd(void* dlogits, const void* dprobs, const void* probs, const void* indices,
                       int indices_are_int64, const int32_t* chosen_experts, const void* logits, int64_t T,
                       int K, int E, int dt, int dprobs_dt, int mode, hipStream_t stream);

/* flextrain_load_balance_bwd (flextrain/ops/_kernels/moe.py:1658-1745; kernel
 * :601-642).  dlogits += scale * p * (f - <f,p>), f = counts / (T*top_k);
 * scale = alpha*E/tokens_per_step is computed by the caller. */
int fx_load_balance_bwd(const void* logits, const int32_t* expert_counts, void* dlogits, int64_t T, int E,
                        int top_k, float scale, int logits_dt, int dlogits_dt, hipStream_t stream);

/* ---- MoE data movement and expert activation ----------------------------- */

/* flextrain_moe_scatter (flextrain/ops/_kernels/moe.py:946-1050; kernel :508-543).
 * x (T,D) contiguous; out row r starts at out + r*out_row_stride; scales (T,K)
 * optional, in original (token, slot) order. */
int fx_moe_scatter(const void* x, const void* indices, int indices_are_int64, const void* scales,
                   int scales_dt, void* out, int64_t T, int D, int K, int64_t out_row_stride, int dt,
                   hipStream_t stream);

/* The token every expert-sorted row came from: out[indices[t, k]] = t for the (T, K) mapping that
 * fx_moe_sort wrote (the inverse of flextrain/ops/_kernels/moe.py:649-834's index mapping, which the
 * reference never needs because it always materialises the sorted copy).  out has T*K entries. */
int fx_moe_row_sources(const void* indices, int indices_are_int64, int64_t T, int K, int32_t* out,
                       hipStream_t stream);

/* flextrain_moe_scatter_routing_weights (flextrain/ops/_kernels/moe.py:1053-1127). */
int fx_moe_scatter_weights(const void* weights, const void* indices, int indices_are_int64, void* out,
                           int64_t n, int dt, hipStream_t stream);

/* flextrain_moe_gather (flextrain/ops/_kernels/moe.py:1130-1271; kernel :560-598).
 * expert_out (T*K,D) contiguous; weights (T,K) and residual (T,D) optional;
 * fp32 accumulation, residual first, k ascending. */
int fx_moe_gather(const void* expert_out, const void* indices, int indices_are_int64, const void* weights,
                  int weights_dt, const void* residual, int residual_dt, void* out, int out_dt, int64_t T,
                  int D, int K, int dt, hipStream_t stream);

/* flextrain_swiglu_moe_fwd (flextrain/ops/_kernels/moe.py:1274-1320; kernel :29-74).
 * x rows are packed [value (F) | gate (F)]; w (rows,) optional. */
int fx_swiglu_moe_fwd(const void* x, const void* w, int w_dt, void* out, int out_dt, int64_t rows, int F,
                      int64_t x_row_stride, int64_t out_row_stride, int dt, hipStream_t stream);

/* flextrain_swiglu_moe_bwd and flextrain_swiglu_moe_bwd_prescaled
 * (flextrain/ops/_kernels/moe.py:1323-1524; kernels :77-215).  dx rows are
 * packed [d value | d gate]; dw (rows,) receives sum_F dout*act; fwd_act optional. */
int fx_swiglu_moe_bwd(void* dx, void* dw, int dw_dt, const void* dout, const void* x, const void* w, int w_dt,
                      void* fwd_act, int64_t rows, int F, int64_t dx_row_stride, int64_t dout_row_stride,
                      int64_t x_row_stride, int64_t act_row_stride, int dt, int prescaled, hipStream_t stream);

/* ---- Softmax / cross-entropy ------------------------------------------------ */

/* flextrain_softmax (flextrain/ops/_kernels/softmax.py:111-215; kernel :13-108).
 * out = softmax(x / temperature) per row, stored in out_dt.  max_idx_out
 * (int64, first occurrence) and max_val_out (fp32, = 1/sum) are optional. */
int fx_softmax(const void* x, void* out, int64_t* max_idx_out, float* max_val_out, int64_t rows, int V,
               int64_t in_row_stride, int64_t out_row_stride, float temperature, int in_dt, int out_dt,
               hipStream_t stream);

/* flextrain_cross_entropy_loss (flextrain/ops/_kernels/cross_entropy.py:61-134;
 * kernel :14-57).  probs is overwritten with dZ = P - onehot(label);
 * loss_out[t] = min(-log P[t,label], max_loss), 0 for labels outside [0,V);
 * valid_out[t] = 1/0. */
int fx_cross_entropy(void* probs, const void* labels, int labels_are_int64, float* loss_out, float* valid_out,
                     int64_t rows, int V, int64_t stride_t, int64_t stride_v, float max_loss, int dt,
                     hipStream_t stream);

/* CrossEntropyLoss.compute (flextrain/nn/loss.py:248-316) as one kernel: logits in,
 * dZ out (dz_out may alias logits), per-row fp32 loss from the log-sum-exp
 * (lse - logit[label], clamped to max_loss), rows with label == ignore_index or a
 * zero loss_mask byte get loss 0 and a zero dZ row.  loss_mask (one byte per row),
 * max_idx_out and max_val_out are optional.
 * softcap > 0 folds the final-logit soft cap of flextrain/nn/head.py:273-298 into both
 * sweeps: statistics, loss, argmax and probabilities are those of
 * y = softcap * tanh(logit / softcap) (rounded to the storage type), and dZ is the gradient
 * at the uncapped logit, (softmax(y) - onehot) * (1 - (y / softcap)^2).  0 = no cap. */
int fx_softmax_ce(const void* logits, void* dz_out, const void* labels, int labels_are_int64,
                  const uint8_t* loss_mask, float* loss_out, int64_t* max_idx_out, float* max_val_out, int64_t rows,
                  int V, int64_t in_row_stride, int64_t out_row_stride, int64_t ignore_index, float max_loss,
                  float softcap, int dt, hipStream_t stream);

/* The soft cap as passes of its own, for loss objects other than the fused kernel
 * (flextrain/nn/head.py:276-282 and :295-297): fx_softcap_fwd caps logits in place and writes
 * gate = 1 - (y / softcap)^2 in the storage type; fx_softcap_bwd multiplies dz by gate. */
int fx_softcap_fwd(void* logits, void* gate_out, int64_t rows, int V, int64_t row_stride, int64_t gate_row_stride,
                   float softcap, int dt, hipStream_t stream);
int fx_softcap_bwd(void* dz, const void* gate, int64_t rows, int V, int64_t row_stride, int64_t gate_row_stride,
                   int dt, hipStream_t stream);

/* ---- Expert-grouped GEMMs -------------------------------------------------- */

/* Scratch bytes for the grouped GEMM entry points (plan header, row offsets, tile list).  No counterpart
 * in the reference, whose per-expert loop (flextrain/ops/full_moe.py:428-626) slices on the host: here the
 * offsets and tiles are built on the device from the counts, and the caller lends the memory. */
size_t fx_grouped_ws_bytes(int E, int64_t total_rows);

/* Row offsets and tile list of one routing, made once and shared by several grouped launches: a
 * grouped entry point called with counts == NULL takes the plan its workspace already holds instead
 * of making it again.  Only a plan written by fx_grouped_plan, or by a grouped entry point that was
 * given counts, for the SAME E and total_rows may be reused that way (every entry point writes the
 * same plan for a given shape).  The plan records the E and the tile height it was made for; a
 * launch that finds another E or tile height there does nothing, and no launch walks more tiles
 * than total_rows and E allow, so a stale or unplanned workspace cannot send a kernel out of
 * bounds, but its output is then left unwritten.  With the per-expert loop of
 * flextrain/ops/full_moe.py:428-626 in mind: the counts are read once per pass over the experts,
 * not once per GEMM. */
int fx_grouped_plan(const int32_t* counts, int E, int64_t total_rows, void* ws, size_t ws_bytes, hipStream_t stream);

/* The per-expert GEMMs of swiglu_expert_loop_fwd / _bwd / _recompute_x_up
 * (flextrain/ops/full_moe.py:428-466, :589-601, :613-616, :661-676) as one launch:
 *   D_e[c_e, N] = alpha * A_e[c_e, K] * op(B[e]) + beta * C_e
 * for every expert e, rows [off_e, off_e + c_e) of the expert-sorted buffers A, C, D.
 * counts: E int32 readable by the device (device memory or pinned host memory).
 * B[e] = B + e * b_expert_stride; trans_b = 1: B[e] stored (N,K) (x @ w.T);
 * trans_b = 0: B[e] stored (K,N).  C may be NULL.  dt: fp16 or bf16. */
int fx_grouped_gemm_rows(const void* A, int64_t lda, const void* B, int64_t ldb, int64_t b_expert_stride,
                         int trans_b, const void* C, int64_t ldc, void* D, int64_t ldd, const int32_t* counts,
                         int E, int64_t total_rows, int N, int K, float alpha, float beta, int dt, void* ws,
                         size_t ws_bytes, hipStream_t stream);

/* The per-expert weight-gradient GEMMs (flextrain/ops/full_moe.py:602-611, :617-626):
 *   G[e][M, N] = alpha * A_e[c_e, M]^T * B_e[c_e, N] + beta * G[e],  G[e] = G + e * g_expert_stride.
 * g_dt may be fp32 for bf16 inputs.
 * a_row_map / b_row_map (optional, at most one; total_rows entries from fx_moe_row_sources): that
 * operand is then the UNSORTED (a_rows or b_rows, M or N) activation matrix and its expert-sorted row
 * r is row map[r] of it: the tile loads gather the rows along the contraction, and the scatter launch
 * of flextrain/ops/moe_backend.py:440-452 with its expert-sorted copy is not needed for this product.
 * rows * ld * 2 bytes must stay below 4 GB; map entries are clamped to the source's rows. */
int fx_grouped_gemm_wgrad(const void* A, int64_t lda, const void* B, int64_t ldb, void* G, int64_t ldg,
                          int64_t g_expert_stride, int g_dt, const int32_t* counts, int E, int64_t total_rows,
                          int M, int N, float alpha, float beta, int dt, void* ws, size_t ws_bytes,
                          const int32_t* a_row_map, int64_t a_rows, const int32_t* b_row_map, int64_t b_rows,
                          hipStream_t stream);

/* The expert up-projection with the SwiGLU fused into its epilogue: one launch for the GEMM of
 * flextrain/ops/full_moe.py:428-447 and the activation kernel that follows it (:448-455).
 * B[e] holds two halves of Nh rows (trans_b = 1, (2*Nh, K) row-major) or Nh columns (trans_b = 0),
 * b2_delta elements apart.  P1 / P2 (row stride ldp) receive the two pre-activation halves,
 * act (rows, Nh) = silu(gate) * value with gate = P1 when gate_first else P2, computed from the
 * rounded P values.  Needs K % 64 == 0 and Nh % 8 == 0.
 * a_row_map (optional, total_rows entries from fx_moe_row_sources): expert-sorted row r of the
 * product is row a_row_map[r] of A, which then is the UNSORTED (a_rows, K) activation matrix: the
 * tile loads gather the rows, and the scatter launch of flextrain/ops/full_moe.py:131-141 with its
 * expert-sorted copy of the activations is not needed for this product.  a_rows * lda * 2 bytes
 * must stay below 4 GB; map entries are clamped to [0, a_rows), so a map that is not a permutation
 * gives wrong rows, never an access outside A.  Without a map A is the expert-sorted
 * (total_rows, K) matrix. */
int fx_grouped_gemm_rows_glu(const void* A, int64_t lda, const void* B, int64_t ldb, int64_t b_expert_stride,
                             int trans_b, int64_t b2_delta, void* P1, void* P2, int64_t ldp, void* act,
                             int64_t ldact, const int32_t* counts, int E, int64_t total_rows, int Nh, int K,
                             int gate_first, int dt, void* ws, size_t ws_bytes, const int32_t* a_row_map,
                             int64_t a_rows, hipStream_t stream);

/* Steps (a) and (b) of the expert backward (flextrain/ops/full_moe.py:589-600: the dgrad GEMM through
 * w_down, then the weighted SwiGLU backward of flextrain/ops/_kernels/moe.py:77-145) as one launch
 * plus a small reduction: dx_act = dy_e @ op(w_down[e]) is rounded to the storage type in the
 * epilogue and never stored;
 *   dx_up[r] = [dx_act * w_r * silu(gate) | dx_act * w_r * value * dsilu(gate)]   (rows of 2 F)
 *   fwd_act[r] = silu(gate) * value * w_r                                         (rows of F; may be NULL)
 *   dprob[r] = sum_f dx_act * silu(gate) * value
 * with x_up[r] = [value (F) | gate (F)] the saved pre-activation and srw[r] = w_r the router weight
 * of expert-sorted row r.  dx_up and fwd_act carry the bits of fx_grouped_gemm_rows followed by
 * fx_swiglu_moe_bwd; dprob is summed in a fixed order (per-wave column slots in part_ws, then a
 * reduction), reproducible from run to run but not in the order of that kernel.
 * K = d_model, F = expert width; trans_b as fx_grouped_gemm_rows (w_down stored (E, d, F): 0).
 * part_ws: fx_grouped_swiglu_bwd_ws_bytes(total_rows, F) bytes, 16-byte aligned.
 * Needs the 256-row tile form (fx_grouped_rows_tile_height(E, total_rows) == 256), K, F and all
 * row strides multiples of 8.
 * dy_row_map (optional): dy is then the UNSORTED (dy_rows, K) upstream gradient and expert-sorted row
 * r is row dy_row_map[r] of it, gathered by the tile loads (as a_row_map of fx_grouped_gemm_rows_glu). */
int fx_grouped_rows_tile_height(int E, int64_t total_rows);
size_t fx_grouped_swiglu_bwd_ws_bytes(int64_t total_rows, int F);
int fx_grouped_gemm_rows_swiglu_bwd(const void* dy, int64_t lddy, const void* w_down, int64_t ldb,
                                    int64_t b_expert_stride, int trans_b, const void* x_up, int64_t ldx,
                                    const void* srw, int srw_dt, void* dx_up, int64_t lddx, void* fwd_act,
                                    int64_t ldact, void* dprob, int dprob_dt, const int32_t* counts, int E,
                                    int64_t total_rows, int F, int K, int dt, void* ws, size_t ws_bytes, void* part_ws,
                                    size_t part_ws_bytes, const int32_t* dy_row_map, int64_t dy_rows,
                                    hipStream_t stream);

/* Gate and up projections of the dense gated FFN with the activation in the epilogue: replaces the
 * two matmuls and the gated-activation launch of flextrain/nn/blocks/ffn_dense.py:130-146.
 *   P1 = A @ op(B1), P2 = A @ op(B2) (both (M, Nh), row stride ldp), act = f(gate) * value
 * with (gate, value) = (P1, P2) when gate_first, else (P2, P1); activation 0 = SiLU,
 * 1 = GELU-tanh.  trans_b = 1: B are (Nh, K) row-major; 0: (K, Nh) row-major; both share ldb.
 * Needs K % 64 == 0 and Nh % 8 == 0. */
int fx_gemm_dual_glu(const void* A, int64_t lda, const void* B1, const void* B2, int64_t ldb, int trans_b,
                     void* P1, void* P2, int64_t ldp, void* act, int64_t ldact, int M, int Nh, int K,
                     int gate_first, int activation, int dt, hipStream_t stream);

/* Up to FX_GEMM_MAX_SEGMENTS products that share op(A), as one launch:
 *   D[i] (M, N[i]) = alpha * op(A) * op(B[i]) + beta * C[i],   i = 0 .. nseg-1.
 * Replaces back-to-back dispatcher calls whose outputs are each too small to fill the GPU: the key
 * and value projections of flextrain/nn/blocks/attention.py:424-463 and their weight gradients
 * (attention.py:712-775).  trans_a / trans_b as in dispatch_matmul (1 = the operand is stored
 * transposed, i.e. column-major); every B[i] has the same form and its own ldb[i]; C and D are
 * row-major with strides ldc[i] / ldd[i], C (or ldc) may be NULL when beta is 0.  bf16 or fp16,
 * outputs of the input type; operands 16-byte aligned with contiguous axes and leading dimensions
 * multiples of 8 (anything else is an error: the caller falls back to separate calls). */
#define FX_GEMM_MAX_SEGMENTS 4
int fx_gemm_segments(const void* A, int64_t lda, int trans_a, int nseg, const void* const* B,
                     const int64_t* ldb, int trans_b, const void* const* C, const int64_t* ldc,
                     void* const* D, const int64_t* ldd, int M, const int* N, int K, float alpha,
                     float beta, int dt, hipStream_t stream);

/* A sum of up to FX_GEMM_MAX_SEGMENTS products into one output, as one launch:
 *   D (M, N) = alpha * sum_i op(A[i]) * op(B[i]) + beta * C,   op(A[i]): M x K[i], op(B[i]): K[i] x N.
 * Replaces chains of dispatcher calls with beta = 1 into the same output: dq Wq^T + dk Wk^T + dv Wv^T
 * of flextrain/nn/blocks/attention.py:712-775 and dx1 W1^T + dx3 W3^T of
 * flextrain/nn/blocks/ffn_dense.py:193-235.  The sum is formed in fp32 and rounded once.  trans_a /
 * trans_b as in dispatch_matmul, shared by all products; lda[i] / ldb[i] per product.  bf16 or fp16
 * inputs, output of the input type or fp32 (bf16 inputs); operands 16-byte aligned, K[i],
 * contiguous axes and leading dimensions multiples of 8 (anything else is an error: the caller
 * falls back to separate calls). */
int fx_gemm_ksum(int nseg, const void* const* A, const int64_t* lda, int trans_a, const void* const* B,
                 const int64_t* ldb, int trans_b, const int* K, const void* C, int64_t ldc, void* D,
                 int64_t ldd, int M, int N, float alpha, float beta, int dt, int d_dt, hipStream_t stream);

/* ---- GEMM dispatcher (verbatim ABI of the reference helper) --------------- */

/* helpers/matmul_dispatcher/src/dispatch.h:12-35.  D = alpha*op(A)*op(B) + beta*C,
 * row-major storage, fp32 accumulation.  trans_a = 0: A is (M,K) with row
 * stride lda; trans_a = 1: A is stored (K,M) with row stride lda.  trans_b = 0:
 * B is (K,N) with row stride ldb; trans_b = 1: B is stored (N,K).  C may be 0
 * (treated as beta = 0) and may alias D.  M, N or K == 0 returns 0 without
 * doing anything.  The workspace (device memory, 16-byte aligned; the reference
 * lends cuBLASLt 64 MiB) is used for fp32 partial sums when a problem with few
 * output tiles and a long K is split along K; without one such problems run
 * unsplit.  A context is not thread-safe; use one per stream, as the reference does. */
typedef struct DispatchContext DispatchContext;
DispatchContext* create_dispatcher(int round_multiple, int max_algos);
void destroy_dispatcher(DispatchContext* ctx);
/* out_stats[7] = {algos_saved, calls, hits, total_ns, hash_ns, lookup_ns, driver_ns}. */
void get_stats(DispatchContext* ctx, uint64_t* out_stats);
int dispatch_matmul(DispatchContext* ctx, intptr_t stream_ptr, int M, int N, int K, intptr_t ptr_A, int lda,
                    intptr_t ptr_B, int ldb, intptr_t ptr_C, int ldc, intptr_t ptr_D, int ldd,
                    intptr_t ptr_workspace, size_t workspace_bytes, int a_dt, int b_dt, int c_dt, int d_dt,
                    int compute_dt, float alpha, float beta, int trans_a, int trans_b);

/* ---- Pinned host memory and the streamed optimizer chunk -------------------- */

/* Pinned (page-locked, device-visible) host memory of exactly `bytes` bytes.  Stands in
 * for the allocate-then-cudaHostRegister sequence of
 * flextrain/engine/host_memory.py:76-100, :178-212 and
 * flextrain/ops/_kernels/_mem_register.py:4-9 on systems where registering memory that
 * already exists is not permitted.  *out receives the pointer (NULL for 0 bytes). */
int fx_host_alloc(size_t bytes, void** out);
int fx_host_free(void* ptr);

/* send_home / fetch_home of one activation slot (flextrain/core/activation_schema.py:483-519; the
 * engine's call sites are flextrain/engine/active_model.py:1184-1199 and :2036-2098): all n
 * fields in one call.  Field i: rows[i] rows of row_bytes[i] bytes, rows dst_pitch[i] /
 * src_pitch[i] bytes apart.  direction 0 = device to host, 1 = host to device, 2 = device to
 * device.  Enqueued on `stream`, not waited for. */
int fx_copy_fields(int n, void* const* dst, const void* const* src, const int64_t* rows,
                   const int64_t* row_bytes, const int64_t* dst_pitch, const int64_t* src_pitch,
                   int direction, hipStream_t stream);

/* Device staging bytes fx_adamw_stream_chunk needs for n_slots slots of sub_elems
 * elements (p, g, m, v and, when stage_bf16_copy, the bf16 copy of p): the role of the reference's
 * optimizer ring slots (flextrain/engine/buffers.py:1088-1291), sized by the caller there. */
size_t fx_adamw_stream_ws_bytes(int64_t sub_elems, int n_slots, int p_dt, int g_dt, int state_dt,
                                int stage_bf16_copy);

/* The optimizer step of one host-offloaded chunk: the fetch / step / offload pipeline of
 * ActiveModel.step (flextrain/engine/active_model.py:486-655) with
 * BufferManager.fetch_layer_{params,grads,opt} / offload_layer_{params,opt}
 * (flextrain/engine/buffers.py:1088-1291) for one flat chunk of n elements.
 * p_host, g_host, m_host, v_host: pinned host memory (p, m, v are updated in place).
 * p_bf16_out: optional bf16 copy of the updated parameters, in pinned host memory
 * (p_bf16_out_on_device = 0) or in device memory (1).  The chunk moves through n_slots
 * (1..16) device slots of sub_elems (multiple of 8) elements inside ws; copies in run on
 * `inbound`, kernels on `compute`, copies out on `outbound` (three distinct non-null
 * streams give full overlap).  Enqueues only: the host buffers hold the result once
 * `outbound` (and, for a device-side bf16 copy, `compute`) has drained.  The caller
 * orders the three streams after whatever produced the host buffers.
 * `ring` (fx_stream_ring_create, same n_slots) carries the slots' "free again" events from one
 * call to the next on the same workspace, so back-to-back calls need no synchronisation between
 * them and keep overlapping (the layer-after-layer pattern of ActiveModel.step).  With ring =
 * NULL the first copies-in wait for all work enqueued so far on `compute` and `outbound`. */
typedef struct FxStreamRing FxStreamRing;
int fx_stream_ring_create(int n_slots, FxStreamRing** out);
int fx_stream_ring_destroy(FxStreamRing* ring);
int fx_adamw_stream_chunk(void* p_host, const void* g_host, void* m_host, void* v_host, void* p_bf16_out,
                          int p_bf16_out_on_device, int64_t n, int p_dt, int g_dt, int state_dt, float lr,
                          float beta1, float beta2, float eps, float weight_decay, float bias_correction1,
                          float bias_correction2, void* ws, size_t ws_bytes, int64_t sub_elems, int n_slots,
                          hipStream_t inbound, hipStream_t compute, hipStream_t outbound, FxStreamRing* ring);

/* ---- Hardware probe --------------------------------------------------------- */

/* No counterpart in the reference: a benchmark aid.  Launches one workgroup per CU that issues
 * nothing but bf16 MFMAs (operands in registers; constant data, or random data when random_data
 * != 0) for `iters` rounds of 16 instructions per wave, on `stream`.  *flop_out receives the
 * floating-point operations of the launch (the caller times it); the first 16 bytes of ws
 * (fx_probe_ws_bytes() bytes of device memory) receive two uint64: shader clock cycles and
 * 100 MHz wall-clock ticks spent in the loop, from which the clock under load follows. */
size_t fx_probe_ws_bytes(void);
int fx_probe_mfma_rate(int random_data, int iters, void* ws, size_t ws_bytes, double* flop_out, hipStream_t stream);

/* ---- Save-level transmission scheduler (verbatim ABI of the reference helper) -- */

/* helpers/transmission_scheduler/transmission_scheduler/transmission_scheduler.h:23-36
 * (implementation transmission_scheduler.c:25-457).  Host code, no GPU work.
 * T tasks, N buffers, k options per task; compute (T), durations and sizes (T*k,
 * row-major) in milliseconds / arbitrary value units; time_scale ticks per
 * millisecond; buf_size from compute_buf_size.  Writes the chosen option of every
 * task to out_choices (T ints) and returns the maximal total value, or 0.0 when
 * no schedule meets the deadlines (out_choices is then left untouched). */
double solve_scheduler(int T, int N, int k, const double* compute, const double* durations,
                       const double* sizes, double deadline, int time_scale, int buf_size,
                       int* out_choices);

/* transmission_scheduler.h:38-40 (transmission_scheduler.c:463-533): window width
 * for solve_scheduler, a power of two >= 2048. */
int compute_buf_size(int T, int N, int k, const double* compute, const double* durations, double deadline,
                     int time_scale);

#ifdef __cplusplus
}
#endif

#endif /* FLEXHIP_H */
