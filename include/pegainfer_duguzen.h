/*
 * pegainfer_duguzen.h - C ABI of the Duguzen host runtime in libpegainfer_qwen3.so.
 *
 * Duguzen: a decoder whose layers are listed one by one in config.json ("layers": type, mixer sizes, feed-forward, and
 * optionally "weights_of": j = compute with layer j's tensors but keep a cache of its own).  Residual stream in fp32 with
 * Dynamic-Tanh norms before and after every sublayer; mixer "latent_attention" (compressed key/value latent + one shared
 * rotated key part per token - the only things cached -, per-head sigmoid output gate); feed-forward either dense
 * (squared ReLU) or routed (sigmoid scores, correction for the choice only, neighbour groups, top-k, SwiGLU experts).
 *
 * Same shape as the other runtimes of this library: one model = one device + one in-order HIP stream, requests are slots
 * holding a KvState over the shared PagePool (csrc/host/kv_pool.h), a step's metadata travels as ONE pinned block, every
 * op goes through the kernel library's C ABI.  What differs: ONE step function serves prompts, portions of prompts and
 * single decoded tokens of several requests in the same batch (a portion may start and end anywhere), and the model can
 * be served in bf16 (matrix products in bf16 with fp32 accumulation; norms, routers, attention scores / weights and the
 * residual sum in fp32) or entirely in fp32.
 * All functions return 0 on success or a negative error (see pegainfer_duguzen_last_error).
 */
#ifndef PEGAINFER_DUGUZEN_H
#define PEGAINFER_DUGUZEN_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void* pegainfer_duguzen_t;

enum { PEGAINFER_DTYPE_BF16 = 0, PEGAINFER_DTYPE_F32 = 1 };

/* config_json: the text of a config.json.  max_tokens: capacity of the latent cache in tokens (rounded up to whole pages
 * of pegainfer_duguzen_page_size() tokens; every live request occupies its length rounded up to whole pages).
 * max_requests: request slots (= the largest batch of one step).  Weights come afterwards: load_tensor per tensor or
 * fill_synthetic, then finalize. */
pegainfer_duguzen_t pegainfer_duguzen_create(const char* config_json, int32_t device_ordinal, int32_t dtype,
                                             int32_t max_tokens, int32_t max_requests);
/* config.json + model.safetensors (or index + shards) of a folder, read natively (mmap); finalised */
pegainfer_duguzen_t pegainfer_duguzen_from_pretrained(const char* model_dir, int32_t device_ordinal, int32_t dtype,
                                                      int32_t max_tokens, int32_t max_requests);
void pegainfer_duguzen_destroy(pegainfer_duguzen_t m);
const char* pegainfer_duguzen_last_error(pegainfer_duguzen_t m);

/* one tensor by its checkpoint name, host bf16 bit patterns (widened exactly when the model is served in fp32) */
int32_t pegainfer_duguzen_load_tensor(pegainfer_duguzen_t m, const char* name, const void* host_bf16, int64_t numel);
/* seeded N(0, std) weights for every tensor the configuration names, generated on the host in bf16 (norm weights 1 + N,
 * alphas 0.5 + N, corrections N(0, 0.1)); for benchmarks and tests without a checkpoint */
int32_t pegainfer_duguzen_fill_synthetic(pegainfer_duguzen_t m, uint64_t seed, float std);
int32_t pegainfer_duguzen_finalize(pegainfer_duguzen_t m);

/* requests = slots with a page list (kv_pool.h KvState); a dropped slot and its pages are handed out again */
int32_t pegainfer_duguzen_new_request(pegainfer_duguzen_t m);
int32_t pegainfer_duguzen_drop_request(pegainfer_duguzen_t m, int32_t request_id);
int32_t pegainfer_duguzen_request_seq_len(pegainfer_duguzen_t m, int32_t request_id);
int32_t pegainfer_duguzen_available_pages(pegainfer_duguzen_t m);
int32_t pegainfer_duguzen_capacity_pages(pegainfer_duguzen_t m);
int32_t pegainfer_duguzen_page_size(pegainfer_duguzen_t m);
int32_t pegainfer_duguzen_max_batch_size(pegainfer_duguzen_t m);
int32_t pegainfer_duguzen_vocab_size(pegainfer_duguzen_t m);
int32_t pegainfer_duguzen_width(pegainfer_duguzen_t m);
int32_t pegainfer_duguzen_num_layer_runs(pegainfer_duguzen_t m);
int32_t pegainfer_duguzen_dtype(pegainfer_duguzen_t m);

/* THE step: entry i appends lens[i] tokens (tokens_concat, entries back to back) to request request_ids[i], continuing
 * from what earlier steps left in its cache; all entries run as one batch.  want_rows: indices into the concatenated
 * token rows whose logits are computed (n_want = -1: the last row of every entry).  out_logits_host (optional) receives
 * [n_want, vocab] floats; out_tokens (optional) the greedy token of every wanted row.  Nothing is changed when the step
 * is rejected (unknown request, not enough free pages, a request listed twice). */
int32_t pegainfer_duguzen_step(pegainfer_duguzen_t m, int32_t n_entries, const int32_t* request_ids, const int32_t* lens,
                               const uint32_t* tokens_concat, int32_t n_want, const int32_t* want_rows,
                               float* out_logits_host, int32_t* out_tokens);
/* gpu_sample rule of the other runtimes over wanted row `row` of the LAST step (greedy when temperature <= 0 or
 * top_k == 1, with top_p >= 1), and its TokenLogprob (pegainfer_logprobs_from_logits over the row's fp32 logits) */
int32_t pegainfer_duguzen_sample(pegainfer_duguzen_t m, int32_t row, float temperature, int32_t top_k, float top_p,
                                 float random_val, int32_t* out_token);
int32_t pegainfer_duguzen_logprobs(pegainfer_duguzen_t m, int32_t row, uint32_t token, int32_t top_k, float* out_logprob,
                                   uint32_t* out_top_ids, float* out_top_logprobs);

/* residual stream after every layer run, all token rows of the last step: while enabled each step keeps
 * [layer runs, rows, width] floats on the device; debug_hidden copies one layer run's rows and returns the row count */
int32_t pegainfer_duguzen_debug_hidden_enable(pegainfer_duguzen_t m, int32_t enable);
int32_t pegainfer_duguzen_debug_hidden(pegainfer_duguzen_t m, int32_t layer_run, float* out_host, int32_t max_rows);

/* device time of the last step (hipEvent pair on the model stream), ms; bytes of weights on the device */
float pegainfer_duguzen_last_step_ms(pegainfer_duguzen_t m);
int64_t pegainfer_duguzen_weight_bytes(pegainfer_duguzen_t m);
/* 0 (default): a bf16 model runs its dense projections on the library's tuned GEMM routes (gemm_cuda) and its attention
 * on the matrix-core form; 1: everything on the plain fp32-arithmetic kernels (the forms the fp32 model always uses) - the
 * two agree to bf16 rounding */
int32_t pegainfer_duguzen_set_plain_kernels(pegainfer_duguzen_t m, int32_t on);

#ifdef __cplusplus
}
#endif
#endif /* PEGAINFER_DUGUZEN_H */
