/*
 * pegainfer_kernels_blocks.h - building blocks of libpegainfer_kernels_hip.so that are not tied to one model family
 * and exist in a bf16 and a true-fp32 instance: Dynamic-Tanh norms over an fp32 residual stream, squared-ReLU and
 * SwiGLU activations, a strided / batched / grouped GEMM, attention over a paged LATENT cache (one compressed key/value
 * vector plus one shared rotated key part per token), and sigmoid-scored grouped top-k expert routing.
 *
 * Conventions: device pointers; `dtype` 0 = bf16 bit patterns, 1 = float (storage of activations AND weights of that
 * call); all arithmetic is fp32; stream last; every function only enqueues work and returns hipGetLastError() as int.
 * Token-major activations ([rows, d], d contiguous).
 */
#ifndef PEGAINFER_KERNELS_BLOCKS_H
#define PEGAINFER_KERNELS_BLOCKS_H

#include <stdint.h>

#include "pegainfer_kernels.h"

#ifdef __cplusplus
extern "C" {
#endif

/* ---- residual stream in fp32 ---- */
/* out[t, :] = embed[token_ids[t], :] widened to fp32 */
pegainfer_status_t pegainfer_embed_f32(const void* embed, const uint32_t* token_ids, float* out, int32_t width,
                                       int32_t n_tokens, int32_t dtype, pegainfer_stream_t stream);
/* Dynamic Tanh: out = tanh(alpha * x) * w + b.  x fp32 [rows, d]; alpha a one-element tensor, w / b [d]; out [rows, d] */
pegainfer_status_t pegainfer_dyt_norm(const float* x, const void* alpha, const void* w, const void* b, void* out,
                                      int32_t d, int32_t rows, int32_t dtype, pegainfer_stream_t stream);
/* x += dyt(y; post);  then, when next_w != NULL, out = dyt(x; next) - the post-norm of one sublayer, the residual sum and
 * the pre-norm of the following sublayer in one pass over the row.  y, out [rows, d]; x fp32 [rows, d] in place */
pegainfer_status_t pegainfer_dyt_add_norm(float* x, const void* y, const void* post_alpha, const void* post_w,
                                          const void* post_b, const void* next_alpha, const void* next_w,
                                          const void* next_b, void* out, int32_t d, int32_t rows, int32_t dtype,
                                          pegainfer_stream_t stream);
/* rows of an fp32 matrix gathered by index: out[i, :] = x[rows_index[i], :] (the positions whose logits are wanted) */
pegainfer_status_t pegainfer_gather_rows_f32(const float* x, const int32_t* rows_index, float* out, int32_t d,
                                             int32_t n_rows, pegainfer_stream_t stream);

/* ---- activations ---- */
/* out = max(x, 0)^2, elementwise (in place allowed) */
pegainfer_status_t pegainfer_relu_sq(const void* x, void* out, int64_t n, int32_t dtype, pegainfer_stream_t stream);
/* out[row, i] = silu(gu[row, i]) * gu[row, I + i]   (gate | up stacked along the row) */
pegainfer_status_t pegainfer_silu_mul_rows(const void* gate_up, void* out, int32_t I, int32_t rows, int32_t dtype,
                                           pegainfer_stream_t stream);

/* ---- strided / batched / grouped GEMM:  y[row, g, m] = sum_k x[row, g, k] * w[g, m, k]  (+ epilogue) ----
 * Dense form (tile_group == NULL): `rows` rows in each of `groups` groups.
 * Grouped form: a device-side table of row tiles, each of <= 64 (or 128: tile_rows_cap) consecutive POSITIONS of a sorted list that belong to
 * one group (expert); positions map to x / y rows through x_row_index / y_row_index (NULL = identity).  Tiles beyond
 * *n_tiles exit; the grid is max_tiles wide.
 * Three kernels behind one entry: an fp32-FMA tile kernel (any sizes and strides, both storage types), a matrix-core tile
 * kernel (bf16 weights with contiguous k in 16-byte chunks; an fp32 x is rounded to bf16 as it is staged) and a few-rows
 * form that streams the weights once (<= 8 rows per tile: decode).  In each the k order of an output is fixed, so a row's
 * result does not depend on what else is in the launch; which kernel runs depends on the launch's shape. */
enum { PEGAINFER_EPI_NONE = 0, PEGAINFER_EPI_RELU_SQ = 1, PEGAINFER_EPI_SIGMOID_GATE = 2 };
typedef struct {
  const void* x;
  const void* w;
  void* y;
  int32_t x_dtype, w_dtype, y_dtype;
  int32_t m, k, rows, groups;
  int64_t x_row_stride, x_group_stride;
  int64_t w_m_stride, w_k_stride, w_group_stride;
  int64_t y_row_stride, y_group_stride;
  const int32_t* tile_group;
  const int32_t* tile_row0;
  const int32_t* tile_rows;
  const int32_t* n_tiles;
  int32_t max_tiles;
  const int32_t* x_row_index;
  const int32_t* y_row_index;
  int32_t epilogue;          /* SIGMOID_GATE: y *= sigmoid(gate[row * gate_row_stride + g]) */
  const void* gate;
  int32_t gate_dtype;
  int64_t gate_row_stride;
  int32_t max_tile_rows;     /* grouped form: an upper bound of tile_rows the caller knows (0 = tile_rows_cap) */
  int32_t tile_rows_cap;     /* grouped form: the rows_per_tile the table was cut with (0 = 64) */
  int32_t plain;             /* != 0: always the fp32-FMA tile kernel (exact products of the stored values) */
} pegainfer_gemm_desc;
pegainfer_status_t pegainfer_gemm_strided(const pegainfer_gemm_desc* d, pegainfer_stream_t stream);

/* ---- attention over a paged latent cache ----
 * Cache: page-first; one layer's entry of one token = [c: rank values | kr: rot values], at
 *   cache + page * page_stride + layer_off + slot * (rank + rot)        (elements of `dtype`).
 * A step's token rows carry their request (token_req), their position in that request (positions) and the request's
 * page list (page_ids[page_indptr[req] ...]).
 *
 * pegainfer_latent_prep: per token row, from one projection row  [ q: heads * (nope + rot) | ... | dkv: rank + rot ]:
 *   c  = dkv[:rank] / sqrt(mean(dkv[:rank]^2) + eps) * c_norm_w            -> cache entry [0, rank)
 *   kr = rotate_half(dkv[rank:], position)                                   -> cache entry [rank, rank + rot)
 *   qc[t, h, rank:] = rotate_half(q[t, h, nope:], position)   (fp32; qc[t, h, :rank] is filled by the absorb GEMM)
 * rotate_half acts on the first rot_dims of the rot values: pair (i, i + rot_dims / 2), angle position * inv_freq[i],
 * both in fp32; the remaining values pass through. */
pegainfer_status_t pegainfer_latent_prep(const void* proj, int64_t proj_row_stride, int64_t dkv_offset,
                                         const void* c_norm_w, float eps, const float* inv_freq, int32_t rot_dims,
                                         const int32_t* positions, const int32_t* token_req, const int32_t* page_indptr,
                                         const int32_t* page_ids, void* cache, int64_t page_stride, int64_t layer_off,
                                         int32_t page_size, float* qc, int32_t heads, int32_t nope, int32_t rot,
                                         int32_t rank, int32_t n_tokens, int32_t dtype, pegainfer_stream_t stream);
/* Causal softmax attention of every (token, head) row over its request's cache entries 0 .. position:
 *   score_j = (qc[t, h, :] . entry_j) * scale;  o_lat[t, h, :] = sum_j softmax(score)_j * entry_j[:rank]
 * qc fp32 [T, heads, rank + rot], o_lat fp32 [T, heads, rank]; scores, running maxima / sums and accumulators in fp32.
 * A row's keys are cut into splits of split_keys (<= 0: 1024) that run in parallel and are merged in split order;
 * workspace: fp32 scratch of pegainfer_latent_attention_workspace(...) floats (NULL allowed when that is 0).
 * Two forms.  tile_row0 == NULL: the plain form, any sizes, bf16 or fp32 cache, fp32 arithmetic throughout.
 * tile_row0 != NULL: the matrix-core form for a bf16 cache (pegainfer_latent_attention_tiled_ok says whether the sizes fit):
 * the flattened rows t * heads + h are cut by the caller into n_tiles runs of <= 64 rows that stay inside one request
 * (tile_row0[i], tile_rows[i]); q and the softmax weights are rounded to bf16 where they enter the matrix cores. */
int64_t pegainfer_latent_attention_workspace(int32_t n_tokens, int32_t heads, int32_t rank, int32_t max_kv_len,
                                             int32_t split_keys);
int32_t pegainfer_latent_attention_tiled_ok(int32_t rank, int32_t rot, int64_t page_stride, int64_t layer_off, int32_t dtype);
pegainfer_status_t pegainfer_latent_attention(const float* qc, float* o_lat, const void* cache, int64_t page_stride,
                                              int64_t layer_off, int32_t page_size, const int32_t* positions,
                                              const int32_t* token_req, const int32_t* page_indptr,
                                              const int32_t* page_ids, int32_t heads, int32_t rank, int32_t rot,
                                              float scale, int32_t n_tokens, int32_t max_kv_len, int32_t split_keys,
                                              float* workspace, const int32_t* tile_row0, const int32_t* tile_rows,
                                              int32_t n_tiles, int32_t dtype, pegainfer_stream_t stream);

/* ---- routed experts ----
 * Router: z = W_r h (fp32 accumulation of the stored values), s = sigmoid(z), choice = s + correction (NULL = none).
 * The experts form n_groups equal groups of neighbours; a group's score is the sum of its two largest choices (of its
 * one choice when a group is a single expert); only the keep_groups best groups stay eligible; the `top` largest
 * eligible choices are taken (ties: the lower index).  out_expert / out_weight [rows, top]; the weight is s of the
 * chosen expert, not renormalised. */
pegainfer_status_t pegainfer_route_sigmoid_grouped(const void* h, const void* w_router, const void* correction,
                                                   int32_t* out_expert, float* out_weight, int32_t d, int32_t experts,
                                                   int32_t n_groups, int32_t keep_groups, int32_t top, int32_t rows,
                                                   int32_t dtype, pegainfer_stream_t stream);
/* Sort the rows * top (row, choice) pairs by expert into a position list and cut it into row tiles of <= rows_per_tile
 * (64 or 128) positions:
 *   pos_pair[p] = pair index (row * top + choice) at position p;  pos_row[p] = its row
 *   tile_group / tile_row0 / tile_rows [max_tiles], *n_tiles;  max_tiles >= ceil(pairs / rows_per_tile) + experts
 * One workgroup, counters in LDS (experts <= 8192).  The order inside an expert is arbitrary; results do not depend on it. */
pegainfer_status_t pegainfer_route_sort(const int32_t* expert, int32_t n_pairs, int32_t top, int32_t experts,
                                        int32_t* pos_pair, int32_t* pos_row, int32_t* tile_group, int32_t* tile_row0,
                                        int32_t* tile_rows, int32_t* n_tiles, int32_t max_tiles, int32_t rows_per_tile,
                                        pegainfer_stream_t stream);
/* out[row, :] = sum_c weight[row, c] * y_pairs[row * top + c, :]   (c ascending; y_pairs fp32) */
pegainfer_status_t pegainfer_route_combine(const float* y_pairs, const float* weight, void* out, int32_t d, int32_t top,
                                           int32_t rows, int32_t dtype, pegainfer_stream_t stream);

/* ---- sequences with state: ragged batches ----
 * A step's token rows are the concatenation of its entries; entry e owns rows entry_row0[e] .. entry_row0[e + 1] - 1 and
 * the state slot entry_slot[e].  Per-slot state lives in fp32 at  state + slot * slot_stride  (floats). */

/* Causal per-channel convolution over time with carried inputs:
 *   out[t, c] = (mode & 1 ? in[t, c] : 0) + sum_j w[c, j] * in[t - taps + 1 + j, c]      (mode & 2: silu of the whole)
 * inputs before the entry's first row come from the slot's state (its last taps - 1 inputs, oldest first, [taps - 1][C]);
 * before the sequence's start that state is zero.  in: fp32 or bf16 by in_dtype; w [C][taps] by w_dtype; out by out_dtype.
 * pegainfer_time_conv only reads the state; pegainfer_time_conv_commit, enqueued after it, moves the state on by the
 * entry's rows. */
pegainfer_status_t pegainfer_time_conv(const void* in, int32_t in_dtype, int64_t in_row_stride, const void* w, int32_t w_dtype,
                                       const float* state, int64_t slot_stride, void* out, int32_t out_dtype,
                                       int64_t out_row_stride, int32_t channels, int32_t taps, int32_t mode,
                                       const int32_t* row_entry, const int32_t* entry_row0, const int32_t* entry_slot,
                                       int32_t n_rows, pegainfer_stream_t stream);
/* both in one launch for a step in which every entry brings exactly one row (row e belongs to entry e): decoding */
pegainfer_status_t pegainfer_time_conv_step(const void* in, int32_t in_dtype, int64_t in_row_stride, const void* w, int32_t w_dtype,
                                            float* state, int64_t slot_stride, void* out, int32_t out_dtype, int64_t out_row_stride,
                                            int32_t channels, int32_t taps, int32_t mode, const int32_t* entry_slot,
                                            int32_t n_entries, pegainfer_stream_t stream);
pegainfer_status_t pegainfer_time_conv_commit(const void* in, int32_t in_dtype, int64_t in_row_stride, float* state,
                                              int64_t slot_stride, int32_t channels, int32_t taps, const int32_t* entry_row0,
                                              const int32_t* entry_slot, int32_t n_entries, pegainfer_stream_t stream);

/* The three with biases (of w_dtype / bias_dtype, [channels], NULL = none): in_bias is part of every real input - it is added to the
 * rows read from `in` and so also sits in the carried inputs, but not in the zeros before a sequence's start (a projection's bias
 * ahead of the convolution); out_bias is added to the sum before the activation (the convolution's own bias). */
pegainfer_status_t pegainfer_time_conv_biased(const void* in, int32_t in_dtype, int64_t in_row_stride, const void* w, int32_t w_dtype,
                                              const void* in_bias, const void* out_bias, const float* state, int64_t slot_stride,
                                              void* out, int32_t out_dtype, int64_t out_row_stride, int32_t channels, int32_t taps,
                                              int32_t mode, const int32_t* row_entry, const int32_t* entry_row0,
                                              const int32_t* entry_slot, int32_t n_rows, pegainfer_stream_t stream);
pegainfer_status_t pegainfer_time_conv_step_biased(const void* in, int32_t in_dtype, int64_t in_row_stride, const void* w,
                                                   int32_t w_dtype, const void* in_bias, const void* out_bias, float* state,
                                                   int64_t slot_stride, void* out, int32_t out_dtype, int64_t out_row_stride,
                                                   int32_t channels, int32_t taps, int32_t mode, const int32_t* entry_slot,
                                                   int32_t n_entries, pegainfer_stream_t stream);
pegainfer_status_t pegainfer_time_conv_commit_biased(const void* in, int32_t in_dtype, int64_t in_row_stride, const void* in_bias,
                                                     int32_t bias_dtype, float* state, int64_t slot_stride, int32_t channels,
                                                     int32_t taps, const int32_t* entry_row0, const int32_t* entry_slot,
                                                     int32_t n_entries, pegainfer_stream_t stream);

/* RMS norm in groups on a sublayer's OUTPUT, the residual sum, and optionally a weighted sum over earlier streams:
 *   n      = y cut into `groups` equal consecutive parts, each / sqrt(mean(part^2) + eps), whole row * w
 *   r      = (x_in ? x_in : 0) + n                           -> x_out (fp32, optional), xb_out (dtype, optional)
 *   mix    = sum_{j < n_mix - 1} coef[j] * stack[j * stack_stride + row * d + :] + coef[n_mix - 1] * r     -> mix_out (fp32)
 * y by y_dtype, w and coef by dtype; everything is computed in fp32.  x_out may alias x_in; mix_out may alias x_in. */
pegainfer_status_t pegainfer_group_rms_add(const float* x_in, const void* y, int32_t y_dtype, const void* w, int32_t groups,
                                           float eps, float* x_out, void* xb_out, int32_t d, int32_t rows, int32_t dtype,
                                           const float* stack, int64_t stack_stride, const void* coef, int32_t n_mix,
                                           float* mix_out, void* mixb_out, pegainfer_stream_t stream);

/* out[row, i] = g * sigmoid(alpha * g) * (u + 1),  g = min(gu[row, i], limit),  u = clamp(gu[row, I + i], -limit, limit) */
pegainfer_status_t pegainfer_clamp_glu_rows(const void* gate_up, void* out, int32_t I, int32_t rows, float limit, float alpha,
                                            int32_t dtype, pegainfer_stream_t stream);

/* Router with a choice of score: score_kind 0 = sigmoid per expert (pegainfer_route_sigmoid_grouped), 1 = softmax over all
 * experts.  Groups, correction, selection and weights as there. */
enum { PEGAINFER_SCORE_SIGMOID = 0, PEGAINFER_SCORE_SOFTMAX = 1 };
pegainfer_status_t pegainfer_route_topk(const void* h, const void* w_router, const void* correction, int32_t* out_expert,
                                        float* out_weight, int32_t d, int32_t experts, int32_t n_groups, int32_t keep_groups,
                                        int32_t top, int32_t rows, int32_t score_kind, int32_t dtype, pegainfer_stream_t stream);
/* the selection alone, from router logits a GEMM has left in fp32 ([rows, experts]; correction of dtype or NULL): the few-rows
 * GEMM streams the router once with the whole chip where one workgroup per row would read it alone (decoding) */
pegainfer_status_t pegainfer_route_from_logits(const float* logits, const void* correction, int32_t* out_expert, float* out_weight,
                                               int32_t experts, int32_t n_groups, int32_t keep_groups, int32_t top, int32_t rows,
                                               int32_t score_kind, int32_t dtype, pegainfer_stream_t stream);
/* the same with the logits at a row stride of their own (a GEMM may leave other columns beside them), a choice of the group
 * score (the sum of a group's two largest choices, or its largest) and, with renorm != 0, weights divided by their sum + 1e-20 */
enum { PEGAINFER_GROUP_TOP2_SUM = 0, PEGAINFER_GROUP_MAX = 1 };
pegainfer_status_t pegainfer_route_from_logits_ex(const float* logits, int64_t logits_stride, const void* correction,
                                                  int32_t* out_expert, float* out_weight, int32_t experts, int32_t n_groups,
                                                  int32_t keep_groups, int32_t top, int32_t rows, int32_t score_kind,
                                                  int32_t group_kind, int32_t renorm, int32_t dtype, pegainfer_stream_t stream);
/* pegainfer_route_combine plus a row every token gets (a shared expert's output, [rows, d] of dtype; NULL = none) */
pegainfer_status_t pegainfer_route_combine_add(const float* y_pairs, const float* weight, const void* add, void* out, int32_t d,
                                               int32_t top, int32_t rows, int32_t dtype, pegainfer_stream_t stream);

/* pegainfer_route_combine_add whose added row is first multiplied by sigmoid(add_gate[row * add_gate_stride]) (fp32 logits, one
 * per row; NULL = no gate) */
pegainfer_status_t pegainfer_route_combine_gated(const float* y_pairs, const float* weight, const void* add,
                                                 const float* add_gate, int64_t add_gate_stride, void* out, int32_t d,
                                                 int32_t top, int32_t rows, int32_t dtype, pegainfer_stream_t stream);

/* Residual sum with a constant factor, then an RMS norm whose gain is ONE number (gain: a one-element tensor of dtype):
 *   r = x_in + mult * (y + bias) + add_rows + add_vec          -> x_out (fp32; may alias x_in)
 *   n = r / sqrt(mean(r^2) + eps) * gain[0]                    -> n_out (fp32)
 * y [rows, d] of y_dtype or NULL (then bias and mult are unused); bias, add_vec [d] of dtype or NULL; add_rows fp32 [rows, d] or
 * NULL; x_out or n_out may be NULL. */
pegainfer_status_t pegainfer_scalar_rms_add(const float* x_in, const void* y, int32_t y_dtype, const void* bias, float mult,
                                            const float* add_rows, const void* add_vec, float* x_out, const void* gain,
                                            float eps, float* n_out, int32_t d, int32_t rows, int32_t dtype,
                                            pegainfer_stream_t stream);

/* Up to three sublayer outputs join the stream in one launch, then the RMS norm (a weight per channel) of what reads the stream
 * next.  A term with norm_w is RMS-normed over the row first:
 *   term_t = (norm_w ? (y + bias) / sqrt(mean((y + bias)^2) + eps) * norm_w : y + bias) * factor
 *   r = x_in + sum_t term_t                         -> x_out (fp32; may alias x_in; optional)
 *   n = r / sqrt(mean(r^2) + eps) * gain            -> n_out (n_dtype: 1 = float, else the storage type; optional)
 * y rows of dtype at y_row_stride; bias, norm_w, gain [d] of dtype.  x_in may be NULL when there are terms; n_terms = 0 is the
 * plain norm of x_in. */
typedef struct {
  const void* y;
  int64_t y_row_stride;
  const void* bias;
  const void* norm_w;
  float factor;
} pegainfer_sum_term;
pegainfer_status_t pegainfer_terms_rms_add(const float* x_in, const pegainfer_sum_term* terms, int32_t n_terms, float* x_out,
                                           const void* gain, float eps, void* n_out, int32_t n_dtype, int32_t d, int32_t rows,
                                           int32_t dtype, pegainfer_stream_t stream);
/* out[row, i] = act(gate[row, i]) * up[row, i], i < I; gate and up are column ranges of rows with stride in_row_stride (elements of
 * dtype).  act 0 = silu, 1 = relu, 2 = gelu (tanh form) */
enum { PEGAINFER_ACT_SILU = 0, PEGAINFER_ACT_RELU = 1, PEGAINFER_ACT_GELU_TANH = 2 };
pegainfer_status_t pegainfer_glu_rows(const void* gate, const void* up, int64_t in_row_stride, void* out, int64_t out_row_stride,
                                      int32_t I, int32_t rows, int32_t act, int32_t dtype, pegainfer_stream_t stream);
/* out[i] = cap * tanh(in[i] / cap) over n fp32 values (in place allowed) */
pegainfer_status_t pegainfer_softcap_rows(const float* in, float* out, int64_t n, float cap, pegainfer_stream_t stream);

/* ---- recurrent matrix memories (state per (slot, head): S [dim][vdim] fp32, row-major) ----
 * Gated delta rule.  Per row, from qkv (fp32 [rows][qkv_stride]: q heads at 0, k heads at kv_heads * dim, v heads at
 * 2 * kv_heads * dim) and the projection row `proj` (dtype; beta logits at b_off, decay inputs at a_off, one per head):
 *   q, k -> x / sqrt(sum(x^2) + 1e-6) per head (q also * dim^-1/2), IN PLACE in qkv;
 *   beta = sigmoid(b);  g = exp(-exp(A_log) * softplus(a + dt_bias))           -> gates (fp32 scratch [rows][2 * heads])
 *   S <- g S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q          head h reads q / k head h / (heads / kv_heads)
 * o: fp32 [rows][heads * vdim].  dim <= 256.  Two launches: a prep over all rows, then the recurrence per (entry, head). */
pegainfer_status_t pegainfer_delta_rule(float* qkv, int64_t qkv_stride, const void* proj, int64_t proj_stride, int64_t b_off,
                                        int64_t a_off, const void* A_log, const void* dt_bias, float* gates, float* state,
                                        int64_t slot_stride, float* o, int32_t heads, int32_t kv_heads, int32_t dim,
                                        int32_t vdim, int32_t n_rows, const int32_t* entry_row0, const int32_t* entry_slot,
                                        int32_t n_entries, int32_t dtype, pegainfer_stream_t stream);
/* The gated delta rule with one decay per (head, key channel), acting on the rows of S:  g = exp(-exp(A_log[h]) *
 * softplus(a[row, h * dim + d] + dt_bias[h * dim + d])), a: fp32 [rows][heads * dim] at stride a_stride (the output of the decay
 * projection), dt_bias [heads * dim], A_log [heads]; gates: fp32 scratch [rows][heads * dim + heads].  Everything else as
 * pegainfer_delta_rule. */
pegainfer_status_t pegainfer_delta_rule_channel(float* qkv, int64_t qkv_stride, const void* proj, int64_t proj_stride,
                                                int64_t b_off, const float* a, int64_t a_stride, const void* A_log,
                                                const void* dt_bias, float* gates, float* state, int64_t slot_stride, float* o,
                                                int32_t heads, int32_t kv_heads, int32_t dim, int32_t vdim, int32_t n_rows,
                                                const int32_t* entry_row0, const int32_t* entry_slot, int32_t n_entries,
                                                int32_t dtype, pegainfer_stream_t stream);
/* Exponentially gated matrix memory with a running maximum (state per (slot, head): S [dim][vdim], n [dim], m; the slot's
 * region is [S of all heads | n of all heads | m of all heads]).  Per row from `proj` (dtype): q at q_off, k at k_off
 * (heads x dim), v at v_off (heads x vdim), gate inputs at i_off / f_off (one per head), biases i_bias / f_bias:
 *   i = cap tanh((zi + bi) / cap);  f = logsigmoid(cap tanh((zf + bf) / cap));  m' = max(f + m, i)
 *   S <- exp(f + m - m') S + exp(i - m') k v^T;  n likewise with k;  o = S^T (q dim^-1/2) / (max(|n . q dim^-1/2|, exp(-m')) + 1e-6)
 * m starts at 0.  o: fp32 [rows][heads * vdim].  dim <= 256. */
pegainfer_status_t pegainfer_gated_matrix_memory(const void* proj, int64_t proj_stride, int64_t q_off, int64_t k_off,
                                                 int64_t v_off, int64_t i_off, int64_t f_off, const void* i_bias,
                                                 const void* f_bias, float cap, float* state, int64_t slot_stride, float* o,
                                                 int32_t heads, int32_t dim, int32_t vdim, const int32_t* entry_row0,
                                                 const int32_t* entry_slot, int32_t n_entries, int32_t dtype,
                                                 pegainfer_stream_t stream);
/* Selective state-space scan with ONE decay per head and token (state per (slot, head): S [n_state][vdim] fp32, row-major; the
 * slot's region holds the heads back to back).  Per row from xbc (fp32 [rows][xbc_stride]: x heads * vdim at 0, B groups * n_state
 * after it, C groups * n_state after that; head h reads group h / (heads / groups)) and the raw step size proj[row, dt_off + h]
 * (dtype):
 *   dt = softplus(raw + dt_bias[h]);  S <- exp(-exp(A_log[h]) dt) S + dt B x^T;  y = S^T C + D[h] x
 * y: fp32 [rows][heads * vdim].  n_state <= 256.  Everything in fp32, the token order is fixed. */
pegainfer_status_t pegainfer_ssd_scan(const float* xbc, int64_t xbc_stride, const void* proj, int64_t proj_stride, int64_t dt_off,
                                      const void* A_log, const void* dt_bias, const void* D, float* state, int64_t slot_stride,
                                      float* o, int32_t heads, int32_t groups, int32_t n_state, int32_t vdim,
                                      const int32_t* entry_row0, const int32_t* entry_slot, int32_t n_entries, int32_t dtype,
                                      pegainfer_stream_t stream);
/* Per-head RMS norm of a memory's read-out, a weight, a gate and a constant factor:
 *   out[row, h, :] = o[row, h, :] / sqrt(mean(o[row, h, :]^2) + eps) * w * act(gate[row, h, :]) * factor
 * w: [vdim] shared by the heads (w_per_head == 0) or [heads * vdim]; gate_kind 0 = silu, 1 = sigmoid; gate rows of dtype
 * with stride gate_stride; out rows of dtype with stride out_stride. */
pegainfer_status_t pegainfer_head_rms_gate(const float* o, const void* w, int32_t w_per_head, const void* gate,
                                           int64_t gate_stride, int32_t gate_kind, float factor, float eps, void* out,
                                           int64_t out_stride, int32_t heads, int32_t vdim, int32_t rows, int32_t dtype,
                                           pegainfer_stream_t stream);

/* pegainfer_head_rms_gate with a choice of order: gate_first != 0 norms the GATED values,
 *   out[row, h, :] = g / sqrt(mean(g^2) + eps) * w * factor,  g = o[row, h, :] * act(gate[row, h, :]) */
pegainfer_status_t pegainfer_head_gate_rms(const float* o, const void* w, int32_t w_per_head, const void* gate, int64_t gate_stride,
                                           int32_t gate_kind, int32_t gate_first, float factor, float eps, void* out,
                                           int64_t out_stride, int32_t heads, int32_t vdim, int32_t rows, int32_t dtype,
                                           pegainfer_stream_t stream);

/* ---- softmax attention over a paged key/value cache, any head sizes, grouped key/value heads ----
 * Cache: page-first; one layer's part of a page = [slot][kv_heads][dim] keys at k_off, [slot][kv_heads][vdim] values at
 * v_off (elements of dtype from the page's start).
 * pegainfer_qk_norm_rope_paged: per row from `proj` (dtype): q heads at q_off, k heads at k_off, v heads at v_off.
 *   q, k -> RMS norm over dim (eps) * q_norm / k_norm ([dim], plain weight), then neighbours (2i, 2i + 1) of the first
 *   rot_dims values rotated by position * inv_freq[i] (fp32 angles); k and v go to the cache entry of (request, position),
 *   q to q_out (fp32 [rows][heads][dim]) or, when q_out_stored is given, to that buffer in dtype instead (the form the
 *   matrix-core attention kernels of pegainfer_kernels.h read). */
pegainfer_status_t pegainfer_qk_norm_rope_paged(const void* proj, int64_t proj_stride, int64_t q_off, int64_t k_off,
                                                int64_t v_off, int32_t heads, int32_t kv_heads, int32_t dim, int32_t vdim,
                                                const void* q_norm, const void* k_norm, float eps, const float* inv_freq,
                                                int32_t rot_dims, const int32_t* positions, const int32_t* row_entry,
                                                const int32_t* page_indptr, const int32_t* page_ids, void* cache,
                                                int64_t page_stride, int64_t k_cache_off, int64_t v_cache_off,
                                                int32_t page_size, float* q_out, void* q_out_stored, int32_t n_rows,
                                                int32_t dtype, pegainfer_stream_t stream);
/* The same with more options: q_norm / k_norm may both be NULL (no norm); q_bias [heads * dim], k_bias [kv_heads * dim],
 * v_bias [kv_heads * vdim] of dtype or NULL are added to the projection's values first; qt_every > 0 multiplies the query by
 * 1 + qt_coef * ln(floor((position + 1) / qt_every) + 1) (query temperature); rot_dims may be 0. */
pegainfer_status_t pegainfer_qk_prep_paged(const void* proj, int64_t proj_stride, int64_t q_off, int64_t k_off, int64_t v_off,
                                          int32_t heads, int32_t kv_heads, int32_t dim, int32_t vdim, const void* q_norm,
                                          const void* k_norm, float eps, const void* q_bias, const void* k_bias,
                                          const void* v_bias, float qt_coef, int32_t qt_every, const float* inv_freq,
                                          int32_t rot_dims, const int32_t* positions, const int32_t* row_entry,
                                          const int32_t* page_indptr, const int32_t* page_ids, void* cache, int64_t page_stride,
                                          int64_t k_cache_off, int64_t v_cache_off, int32_t page_size, float* q_out,
                                          void* q_out_stored, int32_t n_rows, int32_t dtype, pegainfer_stream_t stream);
/* The same with a choice of where the rows come from, of the norm and of the rotation's layout.  proj_dtype: type of the rows
 * read (the storage type, or 1 = float for rows that an fp32 stage such as a time convolution left; offsets and stride in its
 * elements).  norm_kind HEAD_WEIGHT: per head before the rotation, times q_norm / k_norm [dim] (no norm when they are NULL);
 * HEAD_UNIT_AFTER: per head AFTER the rotation, no weight (q_norm / k_norm unused); ALL_WEIGHT: ONE root mean square over all
 * heads of q (of k) before the rotation, times q_norm [heads * dim] / k_norm [kv_heads * dim].  rot_layout PAIRS: neighbours
 * (2i, 2i + 1) turn together; HALVES: value i with value i + rot_dims / 2, both by position * inv_freq[i].  dim <= 256. */
enum { PEGAINFER_QKNORM_HEAD_WEIGHT = 0, PEGAINFER_QKNORM_HEAD_UNIT_AFTER = 1, PEGAINFER_QKNORM_ALL_WEIGHT = 2 };
enum { PEGAINFER_ROT_PAIRS = 0, PEGAINFER_ROT_HALVES = 1 };
pegainfer_status_t pegainfer_qk_prep_paged_form(const void* proj, int32_t proj_dtype, int64_t proj_stride, int64_t q_off,
                                               int64_t k_off, int64_t v_off, int32_t heads, int32_t kv_heads, int32_t dim,
                                               int32_t vdim, const void* q_norm, const void* k_norm, int32_t norm_kind, float eps,
                                               const void* q_bias, const void* k_bias, const void* v_bias, float qt_coef,
                                               int32_t qt_every, const float* inv_freq, int32_t rot_dims, int32_t rot_layout,
                                               const int32_t* positions, const int32_t* row_entry, const int32_t* page_indptr,
                                               const int32_t* page_ids, void* cache, int64_t page_stride, int64_t k_cache_off,
                                               int64_t v_cache_off, int32_t page_size, float* q_out, void* q_out_stored,
                                               int32_t n_rows, int32_t dtype, pegainfer_stream_t stream);
/* Causal softmax attention, scores and weights in fp32:  out[row, h, :] = factor * sum_{j <= position} softmax_j(q . k_j * scale) v_j.
 * The rows are cut by the caller into tiles that stay inside one entry: tile i covers rows tile_row0[i] .. + tile_ntok[i] - 1
 * and, of each key/value group's query heads, tile_qh0[i] .. + tile_nqh[i] - 1, with ntok * nqh <= 16.  dim, vdim <= 256.
 * out rows of dtype with stride out_stride. */
pegainfer_status_t pegainfer_paged_attention(const float* q, const void* cache, int64_t page_stride, int64_t k_cache_off,
                                             int64_t v_cache_off, int32_t page_size, const int32_t* positions,
                                             const int32_t* row_entry, const int32_t* page_indptr, const int32_t* page_ids,
                                             int32_t heads, int32_t kv_heads, int32_t dim, int32_t vdim, float scale,
                                             float factor, const int32_t* tile_row0, const int32_t* tile_ntok,
                                             const int32_t* tile_qh0, const int32_t* tile_nqh, int32_t n_tiles, void* out,
                                             int64_t out_stride, int32_t dtype, pegainfer_stream_t stream);
/* The same kernel with its options.  maps = 2: a query head and a key head hold [map 1 : dim | map 2 : dim] (q rows and cache
 * keys are 2 * dim wide), each map is a softmax of its own over the same values, out = map 1 - lambda * map 2 (maps * dim <= 256).
 * block > 0: a key j is visible to position i only if j <= i and floor(j / block) == floor(i / block), blocks counted from
 * position 0 of the sequence.  sink: [heads] logits of dtype (or NULL) that join every softmax denominator as exp(sink), without
 * scale, key or value.  head_norm != 0: out / sqrt(mean(out^2) + norm_eps) over the head's vdim values.  `factor` comes last.
 * n_split > 1: every tile's keys are dealt in tiles of 64 to n_split workgroups (split z takes key tiles z, z + n_split, ...:
 * the grid does not depend on the contexts' lengths) whose softmax states a second launch folds in split order - for steps of
 * few rows over long contexts (decoding); `workspace` then holds pegainfer_paged_attention_workspace(...) floats.
 * Two kernels behind the entry: a bf16 cache runs on the matrix cores (q and the softmax weights rounded to bf16 where they enter
 * them; scores, maxima, sums and outputs fp32) unless plain != 0; an fp32 cache, or plain, runs the fp32-FMA kernel.
 * pegainfer_paged_attention is the plain kernel's plain form. */
pegainfer_status_t pegainfer_paged_attention_ex(const float* q, const void* cache, int64_t page_stride, int64_t k_cache_off,
                                                int64_t v_cache_off, int32_t page_size, const int32_t* positions,
                                                const int32_t* row_entry, const int32_t* page_indptr, const int32_t* page_ids,
                                                int32_t heads, int32_t kv_heads, int32_t dim, int32_t vdim, float scale,
                                                float factor, const int32_t* tile_row0, const int32_t* tile_ntok,
                                                const int32_t* tile_qh0, const int32_t* tile_nqh, int32_t n_tiles, void* out,
                                                int64_t out_stride, int32_t maps, float lambda, int32_t block, const void* sink,
                                                int32_t head_norm, float norm_eps, int32_t n_split, float* workspace,
                                                int32_t plain, int32_t dtype, pegainfer_stream_t stream);
/* The same with more ways to shape the scores.  softcap > 0: score <- softcap * tanh(score / softcap), after the scale.
 * window > 0: a key j is visible to position i only if j <= i and (i - j < window or j < keep_first): a sliding window whose
 * first keep_first tokens of the sequence stay visible, at their true positions; key tiles that no row of a workgroup sees are
 * not visited.  dist_bias: fp32 [n_dist][heads] (or NULL), added to the scaled, capped score of query head h by distance,
 * dist_bias[min(i - j, n_dist - 1)][h]: a learned bias over distance buckets, expanded by the caller to one row per distance up to
 * the distance from which the bucket no longer changes.  gate_kind != 0: an output gate, logits of dtype in rows at gate_stride; the
 * finished head (after norm and factor) is multiplied by sigmoid(gate[row, h * vdim + c]) (PER_VALUE) or sigmoid(gate[row, h])
 * (PER_HEAD). */
enum { PEGAINFER_GATE_NONE = 0, PEGAINFER_GATE_PER_VALUE = 1, PEGAINFER_GATE_PER_HEAD = 2 };
pegainfer_status_t pegainfer_paged_attention_masked(const float* q, const void* cache, int64_t page_stride, int64_t k_cache_off,
                                                    int64_t v_cache_off, int32_t page_size, const int32_t* positions,
                                                    const int32_t* row_entry, const int32_t* page_indptr, const int32_t* page_ids,
                                                    int32_t heads, int32_t kv_heads, int32_t dim, int32_t vdim, float scale,
                                                    float factor, const int32_t* tile_row0, const int32_t* tile_ntok,
                                                    const int32_t* tile_qh0, const int32_t* tile_nqh, int32_t n_tiles, void* out,
                                                    int64_t out_stride, int32_t maps, float lambda, int32_t block, const void* sink,
                                                    int32_t head_norm, float norm_eps, float softcap, int32_t window,
                                                    int32_t keep_first, const float* dist_bias, int32_t n_dist, const void* gate,
                                                    int64_t gate_stride, int32_t gate_kind, int32_t n_split, float* workspace,
                                                    int32_t plain, int32_t dtype, pegainfer_stream_t stream);
/* fp32 values of scratch a launch with n_split > 1 needs (0 for n_split <= 1) */
int64_t pegainfer_paged_attention_workspace(int32_t n_tiles, int32_t kv_heads, int32_t vdim, int32_t maps, int32_t n_split);
/* out[row, :cols] = in[row, :cols] * factor; rows of in / out at their own strides (elements of dtype) */
pegainfer_status_t pegainfer_scale_rows(const void* in, int64_t in_stride, void* out, int64_t out_stride, int32_t cols,
                                        int32_t rows, float factor, int32_t dtype, pegainfer_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* PEGAINFER_KERNELS_BLOCKS_H */
