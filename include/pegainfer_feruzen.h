/*
 * pegainfer_feruzen.h - C ABI of the Feruzen host runtime in libpegainfer_qwen3.so.
 *
 * Feruzen: a decoder whose layers are listed one by one in config.json ("layers": type, mixer sizes, feed-forward).
 * Residual stream in fp32; a sublayer reads the stream itself and its OUTPUT passes an RMS norm in groups before the
 * residual sum; the mixer's input first gets a short causal convolution over time added to it; what a layer hands on is a
 * learned weighted sum over the streams of all layers so far.  Mixers: "delta" (gated delta rule over a matrix state, short
 * convolutions on q / k / v) and "parallel" (softmax attention with grouped key/value heads over a paged cache, side by
 * side with an exponentially gated matrix memory; their outputs are added with fixed factors).  Feed-forward: clamped
 * gated-linear units, dense or routed (softmax scores, top-k, a shared expert).
 *
 * Same shape as the other runtimes of this library: one model = one device + one in-order HIP stream; a request is a slot
 * that holds a KvState over the shared PagePool (kv_pool.h) for the attention layers AND a region of the state arena
 * (seq_state.h: convolution tails, matrix memories, fp32) for the recurrent ones; a step's metadata travels as ONE pinned
 * block; every op goes through the kernel library's C ABI.  ONE step function serves prompts, portions of prompts and
 * single decoded tokens of several requests in the same batch.  Served in bf16 (matrix products in bf16 with fp32
 * accumulation; norms, routers, attention scores / weights, recurrences and the residual sum in fp32) or entirely in fp32.
 * All functions return 0 on success or a negative error (see pegainfer_feruzen_last_error).
 */
#ifndef PEGAINFER_FERUZEN_H
#define PEGAINFER_FERUZEN_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void* pegainfer_feruzen_t;

/* dtype: 0 = bf16, 1 = fp32 (PEGAINFER_DTYPE_* of pegainfer_duguzen.h).  max_tokens: capacity of the key/value cache in
 * tokens (whole pages of pegainfer_feruzen_page_size() tokens; a live request occupies its length rounded up to pages).
 * max_requests: request slots = state regions = the largest batch of one step. */
pegainfer_feruzen_t pegainfer_feruzen_create(const char* config_json, int32_t device_ordinal, int32_t dtype,
                                             int32_t max_tokens, int32_t max_requests);
pegainfer_feruzen_t pegainfer_feruzen_from_pretrained(const char* model_dir, int32_t device_ordinal, int32_t dtype,
                                                      int32_t max_tokens, int32_t max_requests);
void pegainfer_feruzen_destroy(pegainfer_feruzen_t m);
const char* pegainfer_feruzen_last_error(pegainfer_feruzen_t m);

/* one tensor by its checkpoint name, host bf16 bit patterns (widened exactly when the model is served in fp32) */
int32_t pegainfer_feruzen_load_tensor(pegainfer_feruzen_t m, const char* name, const void* host_bf16, int64_t numel);
/* seeded weights for every tensor the configuration names (benchmarks and tests without a checkpoint) */
int32_t pegainfer_feruzen_fill_synthetic(pegainfer_feruzen_t m, uint64_t seed, float std);
int32_t pegainfer_feruzen_finalize(pegainfer_feruzen_t m);

/* a new request takes a free slot and starts from zero state; a dropped slot, its pages and its state region are handed
 * out again */
int32_t pegainfer_feruzen_new_request(pegainfer_feruzen_t m);
int32_t pegainfer_feruzen_drop_request(pegainfer_feruzen_t m, int32_t request_id);
int32_t pegainfer_feruzen_request_seq_len(pegainfer_feruzen_t m, int32_t request_id);
int32_t pegainfer_feruzen_available_pages(pegainfer_feruzen_t m);
int32_t pegainfer_feruzen_capacity_pages(pegainfer_feruzen_t m);
int32_t pegainfer_feruzen_page_size(pegainfer_feruzen_t m);
int32_t pegainfer_feruzen_max_batch_size(pegainfer_feruzen_t m);
int32_t pegainfer_feruzen_vocab_size(pegainfer_feruzen_t m);
int32_t pegainfer_feruzen_width(pegainfer_feruzen_t m);
int32_t pegainfer_feruzen_num_layer_runs(pegainfer_feruzen_t m);
int32_t pegainfer_feruzen_dtype(pegainfer_feruzen_t m);
/* floats of recurrent state one request holds (convolution tails + matrix memories of all layers) */
int64_t pegainfer_feruzen_state_floats(pegainfer_feruzen_t m);

/* THE step: entry i appends lens[i] tokens (tokens_concat, entries back to back) to request request_ids[i], continuing
 * from the cache and state earlier steps left; all entries run as one batch.  want_rows: indices into the concatenated
 * token rows whose logits are computed (n_want = -1: the last row of every entry).  out_logits_host (optional) receives
 * [n_want, vocab] floats; out_tokens (optional) the greedy token of every wanted row.  Nothing is changed when the step
 * is rejected (unknown request, not enough free pages, a request listed twice). */
int32_t pegainfer_feruzen_step(pegainfer_feruzen_t m, int32_t n_entries, const int32_t* request_ids, const int32_t* lens,
                               const uint32_t* tokens_concat, int32_t n_want, const int32_t* want_rows,
                               float* out_logits_host, int32_t* out_tokens);
int32_t pegainfer_feruzen_sample(pegainfer_feruzen_t m, int32_t row, float temperature, int32_t top_k, float top_p,
                                 float random_val, int32_t* out_token);
int32_t pegainfer_feruzen_logprobs(pegainfer_feruzen_t m, int32_t row, uint32_t token, int32_t top_k, float* out_logprob,
                                   uint32_t* out_top_ids, float* out_top_logprobs);

/* the stream every layer hands on, all token rows of the last step: while enabled each step keeps [layers, rows, width]
 * floats on the device; debug_hidden copies one layer's rows and returns the row count */
int32_t pegainfer_feruzen_debug_hidden_enable(pegainfer_feruzen_t m, int32_t enable);
int32_t pegainfer_feruzen_debug_hidden(pegainfer_feruzen_t m, int32_t layer_run, float* out_host, int32_t max_rows);

float pegainfer_feruzen_last_step_ms(pegainfer_feruzen_t m);
int64_t pegainfer_feruzen_weight_bytes(pegainfer_feruzen_t m);
/* 1: a bf16 model's dense projections run on the plain fp32-arithmetic GEMM instead of the tuned bf16 routes */
int32_t pegainfer_feruzen_set_plain_kernels(pegainfer_feruzen_t m, int32_t on);

#ifdef __cplusplus
}
#endif
#endif /* PEGAINFER_FERUZEN_H */
