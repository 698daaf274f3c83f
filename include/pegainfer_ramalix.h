/*
 * pegainfer_ramalix.h - C ABI of the Ramalix host runtime in libpegainfer_qwen3.so.
 *
 * Ramalix: a decoder whose layers are listed one by one in config.json ("layers": type, mixer sizes, feed-forward), of which
 * a span ("loop": start, stop, times) is walked several times on the same weights - every walk (pass) with a cache and state
 * of its own, the embedding rows added again before every pass but the first, and a learned row per pass.  Residual stream in
 * fp32; pre-norm sublayers x <- x + residual_mult * f(h) whose RMS norms have ONE number as gain and whose input h first gets
 * a short causal convolution over time added to it (mixer and feed-forward alike).  Mixers: "attention" (two softmax maps per
 * head over the same values, combined as map 1 - lambda * map 2 and normed per head; biases; a query factor that grows with the
 * logarithm of the position), "attention_2" (partial pair rotation, keys visible only inside the query's own block of
 * positions, a per-head sink logit in the softmax denominator) and "channel_delta" (gated delta rule with a decay per head
 * and key channel, decays and output gate through low-rank projection pairs, short convolutions on q / k / v).  Feed-forward:
 * SwiGLU experts routed by a softmax router restricted to the best groups, weights renormalised, plus a shared expert scaled
 * by a per-token sigmoid gate.  Logits over an output table of their own, times a constant.
 *
 * Same shape as the other runtimes of this library: one model = one device + one in-order HIP stream; a request is a slot
 * that holds a KvState over the shared PagePool (kv_pool.h) for the attention runs AND a region of the state arena
 * (seq_state.h: convolution tails, matrix memories, fp32) for every run; a step's metadata travels as ONE pinned block; every
 * op goes through the kernel library's C ABI.  ONE step function serves prompts, portions of prompts and single decoded
 * tokens of several requests in the same batch.  Served in bf16 (matrix products in bf16 with fp32 accumulation; norms,
 * routers, attention scores / weights, recurrences and the residual sum in fp32) or entirely in fp32.
 * All functions return 0 on success or a negative error (see pegainfer_ramalix_last_error).
 */
#ifndef PEGAINFER_RAMALIX_H
#define PEGAINFER_RAMALIX_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void* pegainfer_ramalix_t;

/* dtype: 0 = bf16, 1 = fp32 (PEGAINFER_DTYPE_* of pegainfer_duguzen.h).  max_tokens: capacity of the key/value cache in
 * tokens (whole pages of pegainfer_ramalix_page_size() tokens; a live request occupies its length rounded up to pages).
 * max_requests: request slots = state regions = the largest batch of one step. */
pegainfer_ramalix_t pegainfer_ramalix_create(const char* config_json, int32_t device_ordinal, int32_t dtype,
                                             int32_t max_tokens, int32_t max_requests);
pegainfer_ramalix_t pegainfer_ramalix_from_pretrained(const char* model_dir, int32_t device_ordinal, int32_t dtype,
                                                      int32_t max_tokens, int32_t max_requests);
void pegainfer_ramalix_destroy(pegainfer_ramalix_t m);
const char* pegainfer_ramalix_last_error(pegainfer_ramalix_t m);

/* one tensor by its checkpoint name, host bf16 bit patterns (widened exactly when the model is served in fp32) */
int32_t pegainfer_ramalix_load_tensor(pegainfer_ramalix_t m, const char* name, const void* host_bf16, int64_t numel);
/* seeded weights for every tensor the configuration names (benchmarks and tests without a checkpoint); the ranks of the
 * two-step projections, which a checkpoint gives by its tensor shapes, are read from the mixer's optional "a_rank" / "g_rank"
 * entries (32 when absent) */
int32_t pegainfer_ramalix_fill_synthetic(pegainfer_ramalix_t m, uint64_t seed, float std);
int32_t pegainfer_ramalix_finalize(pegainfer_ramalix_t m);

/* a new request takes a free slot and starts from zero state; a dropped slot, its pages and its state region are handed
 * out again */
int32_t pegainfer_ramalix_new_request(pegainfer_ramalix_t m);
int32_t pegainfer_ramalix_drop_request(pegainfer_ramalix_t m, int32_t request_id);
int32_t pegainfer_ramalix_request_seq_len(pegainfer_ramalix_t m, int32_t request_id);
int32_t pegainfer_ramalix_available_pages(pegainfer_ramalix_t m);
int32_t pegainfer_ramalix_capacity_pages(pegainfer_ramalix_t m);
int32_t pegainfer_ramalix_page_size(pegainfer_ramalix_t m);
int32_t pegainfer_ramalix_max_batch_size(pegainfer_ramalix_t m);
int32_t pegainfer_ramalix_vocab_size(pegainfer_ramalix_t m);
int32_t pegainfer_ramalix_width(pegainfer_ramalix_t m);
int32_t pegainfer_ramalix_num_layer_runs(pegainfer_ramalix_t m);
int32_t pegainfer_ramalix_dtype(pegainfer_ramalix_t m);
/* floats of recurrent state one request holds (convolution tails + matrix memories of all layer runs) */
int64_t pegainfer_ramalix_state_floats(pegainfer_ramalix_t m);

/* THE step: entry i appends lens[i] tokens (tokens_concat, entries back to back) to request request_ids[i], continuing
 * from the cache and state earlier steps left; all entries run as one batch.  want_rows: indices into the concatenated
 * token rows whose logits are computed (n_want = -1: the last row of every entry).  out_logits_host (optional) receives
 * [n_want, vocab] floats; out_tokens (optional) the greedy token of every wanted row.  Nothing is changed when the step
 * is rejected (unknown request, not enough free pages, a request listed twice). */
int32_t pegainfer_ramalix_step(pegainfer_ramalix_t m, int32_t n_entries, const int32_t* request_ids, const int32_t* lens,
                               const uint32_t* tokens_concat, int32_t n_want, const int32_t* want_rows,
                               float* out_logits_host, int32_t* out_tokens);
int32_t pegainfer_ramalix_sample(pegainfer_ramalix_t m, int32_t row, float temperature, int32_t top_k, float top_p,
                                 float random_val, int32_t* out_token);
int32_t pegainfer_ramalix_logprobs(pegainfer_ramalix_t m, int32_t row, uint32_t token, int32_t top_k, float* out_logprob,
                                   uint32_t* out_top_ids, float* out_top_logprobs);

/* the residual stream after every layer run (before what a following pass adds), all token rows of the last step: while
 * enabled each step keeps [layer runs, rows, width] floats on the device; debug_hidden copies one run's rows and returns the
 * row count */
int32_t pegainfer_ramalix_debug_hidden_enable(pegainfer_ramalix_t m, int32_t enable);
int32_t pegainfer_ramalix_debug_hidden(pegainfer_ramalix_t m, int32_t layer_run, float* out_host, int32_t max_rows);

float pegainfer_ramalix_last_step_ms(pegainfer_ramalix_t m);
int64_t pegainfer_ramalix_weight_bytes(pegainfer_ramalix_t m);
/* 1: a bf16 model's dense projections run on the plain fp32-arithmetic GEMM instead of the tuned bf16 routes */
int32_t pegainfer_ramalix_set_plain_kernels(pegainfer_ramalix_t m, int32_t on);

#ifdef __cplusplus
}
#endif
#endif /* PEGAINFER_RAMALIX_H */
