/*
 * pegainfer_kukulorn.h - C ABI of the Kukulorn host runtime in libpegainfer_qwen3.so.
 *
 * Kukulorn: a decoder whose layers are listed one by one in config.json ("layers": type, mixer sizes, feed-forward or none), of
 * which a span ("loop": start, stop, times) is walked several times on the same weights - every walk (pass) with a cache and
 * state of its own, and before every pass the stream is mixed with the embedding rows again, x <- W_in [x ; x0].  Residual
 * stream in fp32.  A layer has ONE RMS norm (a weight per channel) whose output both sublayers read: x <- x + mixer(h) + ff(h).
 * Mixers: "attention" (grouped key/value heads; biases; a short causal convolution over time on q, k and v right after the
 * projection; rotation of the halves of the first rot.dims values with long-context frequency scaling; q and k brought to unit
 * root mean square per head after the rotation; scores soft-capped by tanh; a sigmoid output gate per value) and "parallel"
 * (left: attention without rotation, q and k RMS-normed over the whole projection, a learned bias by logarithmic distance
 * buckets, a sliding window that keeps the first tokens, a sigmoid gate per head; right: a selective state-space layer with a
 * scalar decay per head, its gated output normed in groups; the two outputs RMS-normed over the width and averaged).
 * Feed-forward: act(W_gate h) * (W_up h) with act = relu.  Logits over the embedding table, soft-capped.
 *
 * Same shape as the other runtimes of this library: one model = one device + one in-order HIP stream; a request is a slot
 * that holds a KvState over the shared PagePool (kv_pool.h) for the attention of every layer run AND a region of the state
 * arena (seq_state.h: convolution tails, state-space memories, fp32); a step's metadata travels as ONE pinned block; every
 * op goes through the kernel library's C ABI.  ONE step function serves prompts, portions of prompts and single decoded
 * tokens of several requests in the same batch.  Served in bf16 (matrix products in bf16 with fp32 accumulation; norms,
 * attention scores / weights, angles, the recurrence and the residual sum in fp32) or entirely in fp32.
 * All functions return 0 on success or a negative error (see pegainfer_kukulorn_last_error).
 */
#ifndef PEGAINFER_KUKULORN_H
#define PEGAINFER_KUKULORN_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void* pegainfer_kukulorn_t;

/* dtype: 0 = bf16, 1 = fp32 (PEGAINFER_DTYPE_* of pegainfer_duguzen.h).  max_tokens: capacity of the key/value cache in
 * tokens (whole pages of pegainfer_kukulorn_page_size() tokens; a live request occupies its length rounded up to pages).
 * max_requests: request slots = state regions = the largest batch of one step. */
pegainfer_kukulorn_t pegainfer_kukulorn_create(const char* config_json, int32_t device_ordinal, int32_t dtype,
                                             int32_t max_tokens, int32_t max_requests);
pegainfer_kukulorn_t pegainfer_kukulorn_from_pretrained(const char* model_dir, int32_t device_ordinal, int32_t dtype,
                                                      int32_t max_tokens, int32_t max_requests);
void pegainfer_kukulorn_destroy(pegainfer_kukulorn_t m);
const char* pegainfer_kukulorn_last_error(pegainfer_kukulorn_t m);

/* one tensor by its checkpoint name, host bf16 bit patterns (widened exactly when the model is served in fp32) */
int32_t pegainfer_kukulorn_load_tensor(pegainfer_kukulorn_t m, const char* name, const void* host_bf16, int64_t numel);
/* seeded weights for every tensor the configuration names (benchmarks and tests without a checkpoint); the number of distance
 * buckets of a bias table, which a checkpoint gives by the tensor's shape, is read from the mixer's optional "rel_rows" entry
 * (32 when absent) */
int32_t pegainfer_kukulorn_fill_synthetic(pegainfer_kukulorn_t m, uint64_t seed, float std);
int32_t pegainfer_kukulorn_finalize(pegainfer_kukulorn_t m);

/* a new request takes a free slot and starts from zero state; a dropped slot, its pages and its state region are handed
 * out again */
int32_t pegainfer_kukulorn_new_request(pegainfer_kukulorn_t m);
int32_t pegainfer_kukulorn_drop_request(pegainfer_kukulorn_t m, int32_t request_id);
int32_t pegainfer_kukulorn_request_seq_len(pegainfer_kukulorn_t m, int32_t request_id);
int32_t pegainfer_kukulorn_available_pages(pegainfer_kukulorn_t m);
int32_t pegainfer_kukulorn_capacity_pages(pegainfer_kukulorn_t m);
int32_t pegainfer_kukulorn_page_size(pegainfer_kukulorn_t m);
int32_t pegainfer_kukulorn_max_batch_size(pegainfer_kukulorn_t m);
int32_t pegainfer_kukulorn_vocab_size(pegainfer_kukulorn_t m);
int32_t pegainfer_kukulorn_width(pegainfer_kukulorn_t m);
int32_t pegainfer_kukulorn_num_layer_runs(pegainfer_kukulorn_t m);
int32_t pegainfer_kukulorn_dtype(pegainfer_kukulorn_t m);
/* floats of recurrent state one request holds (convolution tails + state-space memories of all layer runs) */
int64_t pegainfer_kukulorn_state_floats(pegainfer_kukulorn_t m);

/* THE step: entry i appends lens[i] tokens (tokens_concat, entries back to back) to request request_ids[i], continuing
 * from the cache and state earlier steps left; all entries run as one batch.  want_rows: indices into the concatenated
 * token rows whose logits are computed (n_want = -1: the last row of every entry).  out_logits_host (optional) receives
 * [n_want, vocab] floats; out_tokens (optional) the greedy token of every wanted row.  Nothing is changed when the step
 * is rejected (unknown request, not enough free pages, a request listed twice). */
int32_t pegainfer_kukulorn_step(pegainfer_kukulorn_t m, int32_t n_entries, const int32_t* request_ids, const int32_t* lens,
                               const uint32_t* tokens_concat, int32_t n_want, const int32_t* want_rows,
                               float* out_logits_host, int32_t* out_tokens);
int32_t pegainfer_kukulorn_sample(pegainfer_kukulorn_t m, int32_t row, float temperature, int32_t top_k, float top_p,
                                 float random_val, int32_t* out_token);
int32_t pegainfer_kukulorn_logprobs(pegainfer_kukulorn_t m, int32_t row, uint32_t token, int32_t top_k, float* out_logprob,
                                   uint32_t* out_top_ids, float* out_top_logprobs);

/* the residual stream after every layer run (before the input projection of a following pass), all token rows of the last step: while
 * enabled each step keeps [layer runs, rows, width] floats on the device; debug_hidden copies one run's rows and returns the
 * row count */
int32_t pegainfer_kukulorn_debug_hidden_enable(pegainfer_kukulorn_t m, int32_t enable);
int32_t pegainfer_kukulorn_debug_hidden(pegainfer_kukulorn_t m, int32_t layer_run, float* out_host, int32_t max_rows);

float pegainfer_kukulorn_last_step_ms(pegainfer_kukulorn_t m);
int64_t pegainfer_kukulorn_weight_bytes(pegainfer_kukulorn_t m);
/* 1: a bf16 model's dense projections run on the plain fp32-arithmetic GEMM instead of the tuned bf16 routes */
int32_t pegainfer_kukulorn_set_plain_kernels(pegainfer_kukulorn_t m, int32_t on);

#ifdef __cplusplus
}
#endif
#endif /* PEGAINFER_KUKULORN_H */
