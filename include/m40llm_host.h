/*
 * C view of the C++ host layer that sits above the m40llm C ABI (libm40llm_host.so).
 *
 * The reference's host side is Rust (src/decode.rs, src/decode_batch.rs, src/kv_compression.rs,
 * src/kv_selection.rs, src/sampling.rs and the decode part of src/infer/forward.rs); no Rust
 * toolchain exists in this build environment, so the same modules are written in C++
 * (the headers under m40-llm_amd/host) and exposed here so that tests and bindings in any language can drive
 * them.  Every function that can fail returns a negative value and leaves a message for
 * m40host_last_error().
 */
#ifndef M40LLM_HOST_H
#define M40LLM_HOST_H

#include <stddef.h>
#include <stdint.h>

#include "m40llm.h"

#ifdef __cplusplus
extern "C" {
#endif

const char* m40host_last_error(void);

/* ---- sampling (src/sampling.rs) ---------------------------------------------------------- */
/* top_k < 0 = none, top_p <= 0 = none */
void* m40host_sampler_create(float temperature, int64_t top_k, float top_p, uint64_t seed);
void* m40host_greedy_sampler(uint64_t seed);                                  /* src/decode.rs:111-117 */
int64_t m40host_sampler_sample(void* sampler, const float* logits, size_t n);
int64_t m40host_sampler_sample_greedy(void* sampler, const float* logits, size_t n);
void m40host_sampler_destroy(void* sampler);

/* ---- stopping criteria and decode loop (src/decode.rs) ----------------------------------------- */
/* max_tokens < 0 = none, eos_id < 0 = none.  with_stop_ids != 0 builds the criteria from stop_ids
 * (first id doubles as eos), else from eos_id alone. */
int m40host_should_stop(int64_t max_tokens, int64_t eos_id, const uint32_t* stop_ids, size_t n_stop,
                        int with_stop_ids, const uint32_t* generated, size_t n_generated);
/* logits callback: fill logits_out[vocab] for the ids so far; return 0, or nonzero to abort */
typedef int (*m40host_logits_fn)(void* user, const uint32_t* ids, size_t n_ids, float* logits_out, size_t vocab);
/* returns the total number of ids written to ids_out (prompt + generated), or a negative value */
int64_t m40host_decode_loop(const uint32_t* prompt, size_t n_prompt, void* sampler, int64_t max_tokens,
                            int64_t eos_id, const uint32_t* stop_ids, size_t n_stop, int with_stop_ids,
                            size_t vocab, m40host_logits_fn logits_fn, void* user, uint32_t* ids_out,
                            size_t ids_capacity);

/* ---- sequence-slot pool (src/decode_batch.rs:14-85) ------------------------------------------------ */
void* m40host_pool_create(uint32_t capacity);
void m40host_pool_destroy(void* pool);
uint32_t m40host_pool_capacity(void* pool);
size_t m40host_pool_available(void* pool);
void* m40host_pool_try_lease(void* pool);             /* NULL when no slot is free */
uint32_t m40host_lease_sequence_id(void* lease);
void m40host_lease_release(void* lease);              /* returns the slot to the back of the free list */

/* ---- batch metadata and decode batch plan (src/infer/batch.rs:276-355, src/decode_batch.rs:142-355) */
/* status: 0 active, 1 completed, 2 cancelled.  NULL on error. */
void* m40host_batch_plan_from_requests(const uint64_t* request_ids, const uint32_t* sequence_ids,
                                       const uint32_t* kv_lens, const uint32_t* status, size_t n);
void m40host_batch_plan_destroy(void* plan);
uint32_t m40host_batch_plan_size(void* plan);
void m40host_batch_plan_sequence_ids(void* plan, uint32_t* out);
void m40host_batch_plan_sequence_lens(void* plan, uint32_t* out);
uint32_t m40host_batch_plan_total_q_tokens(void* plan);
uint32_t m40host_batch_plan_total_kv_tokens(void* plan);
uint64_t m40host_batch_plan_total_attention_cells(void* plan);
uint32_t m40host_batch_plan_query_len(void* plan, size_t index);
int64_t m40host_batch_plan_index_for_request(void* plan, uint64_t request_id);   /* -1 = none */
int64_t m40host_batch_plan_output_offset_f32(void* plan, uint64_t request_id, uint32_t q_heads, uint32_t head_dim);
/* uploads ids/lens and calls the batched attention entry point; Q/Out packed in plan order */
int m40host_batch_plan_dispatch_attention(void* plan, M40llmCudaContext* ctx, const M40llmKVCache* kv,
                                          const void* d_q_f32, uint32_t q_heads, void* d_out_f32, int async);
/* validation only: 0 ok, -1 rejected (message in m40host_last_error) */
int m40host_batch_metadata_check(const uint32_t* seq_lens, const uint32_t* kv_lens, const uint32_t* query_lens,
                                 size_t n, uint32_t* total_q, uint32_t* total_kv, uint64_t* attention_cells);

/* ---- KV-compression configuration (src/kv_compression.rs) ------------------------------------------ */
typedef struct M40HostKvConfig {
    uint32_t mode;                   /* 0 off, 1 dense-recent-only, 2 block-select-exact, 3 recent-only,
                                        4 block-summary, 5 block-select-lossy */
    uint32_t recent_window, block_size, top_blocks, representatives;
    uint32_t representative_policy;  /* 0 last, 1 stride */
    uint32_t exact_old_backing;      /* 0 dense, 1 q8, 2 fp16-k-q4-v */
    uint32_t exact_old_attention;    /* 0 staged, 1 q8-direct, 2 fp16-k-q4-v-direct */
} M40HostKvConfig;
void m40host_kvcfg_default(M40HostKvConfig* out);
void m40host_kvcfg_dense_reference(M40HostKvConfig* out);
void m40host_kvcfg_for_mode(uint32_t mode, M40HostKvConfig* out);
int m40host_kvcfg_validate(const M40HostKvConfig* cfg, char* err, size_t err_len);
int m40host_kvcfg_validate_runtime_support(const M40HostKvConfig* cfg, uint32_t max_seq_len, uint32_t head_dim,
                                           char* err, size_t err_len);
uint32_t m40host_kvcfg_effective_backing(const M40HostKvConfig* cfg);
uint32_t m40host_kvcfg_effective_attention(const M40HostKvConfig* cfg);
void m40host_kvcfg_set_runtime(const M40HostKvConfig* cfg);
void m40host_kvcfg_get_runtime(M40HostKvConfig* out);
void* m40host_kvcfg_scoped_push(const M40HostKvConfig* cfg);   /* shadows the runtime config on this thread */
void m40host_kvcfg_scoped_pop(void* guard);

/* ---- selection telemetry (src/kv_selection.rs) ------------------------------------------------------ */
int m40host_kvsel_enabled(void);
void m40host_kvsel_reset(void);
void m40host_kvsel_set_attention_context(int64_t layer, int64_t token);   /* < 0 = none */
void m40host_kvsel_record(const uint32_t* blocks, size_t n, uint32_t total_old_blocks, uint32_t top_blocks);
void m40host_kvsel_record_scored_timed(const uint32_t* blocks, const float* scores, const uint32_t* starts,
                                       const uint32_t* ends, size_t n, uint32_t total_old_blocks,
                                       uint32_t top_blocks, float elapsed_ms /* < 0 = none */);
/* returns 0 when nothing was recorded, else 1 and fills the summary */
int m40host_kvsel_snapshot(uint32_t* selected_out, size_t capacity, size_t* n_selected, uint32_t* total_old_blocks,
                           uint32_t* top_blocks, size_t* n_records);
int m40host_kvsel_snapshot_record(size_t index, int64_t* layer, int64_t* token, uint32_t* ranks, uint32_t* blocks,
                                  float* scores, uint32_t* starts, uint32_t* ends, size_t capacity, size_t* n,
                                  uint32_t* total_old_blocks, uint32_t* top_blocks, float* elapsed_ms);
int m40host_kvsel_should_capture_attention(void);
void m40host_kvsel_record_attention(float recent_mass, float selected_old_mass);
size_t m40host_kvsel_attention_count(void);

/* ---- model step (decode part of src/infer/forward.rs, src/infer/logits.rs, src/decode_session.rs) --- */
typedef struct M40HostModel M40HostModel;
typedef struct M40HostModelConfig {
    uint32_t n_layers, d_model, q_heads, kv_heads, head_dim, ffn, vocab;
    float rms_eps, rope_base, rope_scale;
    uint32_t rope_layout, has_qkv_bias, norm_weight_dtype;
    uint32_t max_seq_len, max_sequences;
} M40HostModelConfig;
typedef struct M40HostLayerWeights {
    const void *wq, *wk, *wv, *wo, *wgate, *wup, *wdown;   /* device, f16 GGUF layout */
    const void *bq, *bk, *bv;                              /* device f32 or NULL */
    const void *attn_norm, *ffn_norm;                      /* device, dtype = norm_weight_dtype */
} M40HostLayerWeights;
/* kv_cfg NULL = dense cache (mode off) */
M40HostModel* m40host_model_create(M40llmCudaContext* ctx, const M40HostModelConfig* cfg,
                                   const M40HostLayerWeights* layers, const void* out_norm, const void* lm_head,
                                   const void* tok_emb, const M40HostKvConfig* kv_cfg);
void m40host_model_destroy(M40HostModel* model);
M40llmKVCache* m40host_model_kv(M40HostModel* model);
uint32_t m40host_model_kv_slot(M40HostModel* model, uint32_t sequence_id, uint32_t layer);
/* mode 0 = the reference's call sequence, 1 = fused single-stream path, 2 = fused + graph replay */
int m40host_model_set_mode(M40HostModel* model, uint32_t mode);
/* one token through all layers; either output may be NULL */
int m40host_model_forward_token(M40HostModel* model, uint32_t sequence_id, uint32_t position, uint32_t token_id,
                                float* hidden_host, float* logits_host);
int m40host_model_decode_greedy(M40HostModel* model, uint32_t sequence_id, const uint32_t* prompt, uint32_t n_prompt,
                                uint32_t n_gen, uint32_t start_pos, uint32_t* ids_out, float* gaps_out);
/* prompt (untimed) + `warmup` untimed greedy steps + `steps` greedy steps timed on the host clock between two
 * stream synchronisations; ids_out holds n_prompt + warmup + steps ids; elapsed_ms covers the timed steps only */
int m40host_model_decode_timed(M40HostModel* model, uint32_t sequence_id, const uint32_t* prompt, uint32_t n_prompt,
                               uint32_t warmup, uint32_t steps, uint32_t* ids_out, double* elapsed_ms);
/* same for a batch of sequences whose caches are pre-filled to kv_lens; ids_out [rows][warmup+steps] */
int m40host_model_decode_batch_timed(M40HostModel* model, const uint32_t* sequence_ids, const uint32_t* kv_lens,
                                     const uint32_t* first_tokens, uint32_t rows, uint32_t warmup, uint32_t steps,
                                     uint32_t* ids_out, double* elapsed_ms);
/* 1 when the last decode_timed / decode_batch_timed call measured the host-sampled path: a device-side greedy pick
 * had a top-1 / top-2 logit gap under the tie guard, so warm-up and timed steps were redone through the host sampler
 * (as m40host_model_decode_greedy / decode_batch_greedy do); 0 when the device path was measured */
int m40host_model_last_timed_host_fallback(M40HostModel* model);
/* top-1 / top-2 logit gap under which a device-side greedy pick is not trusted (default 1e-6) */
int m40host_model_set_tie_guard(M40HostModel* model, float guard);
/* one batched step: hidden_host [rows][d_model] and logits_host [rows][vocab] may be NULL */
int m40host_model_forward_batched(M40HostModel* model, const uint32_t* sequence_ids, const uint32_t* kv_lens,
                                  const uint32_t* token_ids, uint32_t rows, float* hidden_host, float* logits_host);
int m40host_model_decode_batch_greedy(M40HostModel* model, const uint32_t* sequence_ids, const uint32_t* kv_lens,
                                      const uint32_t* first_tokens, uint32_t rows, uint32_t steps, uint32_t* ids_out,
                                      float* gaps_out);
/* Packed prefill of `batch` prompts (forward_prefill_all_layers_varlen_for_sequences, src/infer/forward.rs:2153-2600):
 * tokens holds the prompts one after the other (lens[i] ids each); every sequence starts at position 0 of its cache
 * slots, which afterwards hold lens[i] tokens.  Dense cache, head_dim 64 or 128, at most 64 prompts and 65535 tokens
 * per call.  hidden_last_host [batch][d_model] and logits_last_host [batch][vocab] receive the last token of each
 * prompt; either may be NULL. */
int m40host_model_forward_prefill(M40HostModel* model, const uint32_t* sequence_ids, const uint32_t* lens,
                                  const uint32_t* tokens, uint32_t batch, float* hidden_last_host, float* logits_last_host);

/* ---- continuous-batching decode scheduler (src/server.rs:203-770 without HTTP, tokenizer and channels) ---------- */
typedef struct M40HostScheduler M40HostScheduler;
typedef struct M40HostTickReport {
    uint32_t prefill_rows, prefill_tokens, decode_rows, completed, cancelled, failed;
} M40HostTickReport;
/* Engine callbacks for a scheduler that is not tied to a model (tests, other back ends): fill one row of `vocab`
 * logits per item; return 0, or nonzero to fail every request of the call. */
typedef int (*m40host_sched_prefill_fn)(void* user, const uint32_t* sequence_ids, const uint32_t* lens, const uint32_t* tokens,
                                        uint32_t batch, float* logits_out);
typedef int (*m40host_sched_decode_fn)(void* user, const uint32_t* sequence_ids, const uint32_t* kv_lens, const uint32_t* tokens,
                                       uint32_t rows, float* logits_out);
/* sequence_slots 0 (or above the model's max_sequences) = the model's max_sequences.  Prompts are prefilled with the
 * packed prefill forward when the model can (dense cache, head_dim 64 / 128), token by token otherwise; decode ticks
 * run one batched step with the fused kernels in the model's host mode 1 / 2; requests with top_k = 1 and no top_p get
 * their token from the device-side argmax unless the top two logits are a near tie (then from the host sampler). */
M40HostScheduler* m40host_scheduler_create_for_model(M40HostModel* model, uint32_t sequence_slots);
M40HostScheduler* m40host_scheduler_create_with_engine(uint32_t vocab, uint32_t max_seq_len, uint32_t sequence_slots,
                                                       m40host_sched_prefill_fn prefill_fn, m40host_sched_decode_fn decode_fn,
                                                       void* user);
void m40host_scheduler_destroy(M40HostScheduler* scheduler);
/* enqueue_scheduler_request: leases a sequence slot (FIFO pool) or fails with "decode batching requires a sequence
 * lease"; max_tokens < 0 = the context length; top_k < 0 / top_p <= 0 = none (top_k 1 = greedy).  Returns the request
 * id (1, 2, ...) or -1. */
int64_t m40host_scheduler_submit(M40HostScheduler* scheduler, const uint32_t* prompt, size_t n_prompt, int64_t max_tokens,
                                 const uint32_t* stop_ids, size_t n_stop, float temperature, int64_t top_k, float top_p,
                                 uint64_t seed);
int m40host_scheduler_cancel(M40HostScheduler* scheduler, uint64_t request_id);   /* 1 if the request was active */
/* one scheduler tick: cancelled requests leave, finished ones are reported, pending prompts are prefilled together and
 * sample their first token, every other request takes one batched decode step */
int m40host_scheduler_tick(M40HostScheduler* scheduler, M40HostTickReport* report);
/* 0 unknown, 1 pending prefill, 2 decoding, 3 complete, 4 cancelled, 5 failed */
uint32_t m40host_scheduler_state(M40HostScheduler* scheduler, uint64_t request_id);
uint32_t m40host_scheduler_sequence_of(M40HostScheduler* scheduler, uint64_t request_id);   /* 0xffffffff when not active */
size_t m40host_scheduler_active(M40HostScheduler* scheduler);
size_t m40host_scheduler_available_slots(M40HostScheduler* scheduler);
/* generated ids so far (any state): returns their number, writes at most `capacity` */
int64_t m40host_scheduler_generated(M40HostScheduler* scheduler, uint64_t request_id, uint32_t* ids_out, size_t capacity);
size_t m40host_scheduler_error(M40HostScheduler* scheduler, uint64_t request_id, char* buf, size_t capacity);

/* ---- GGUF ingestion (src/gguf.rs:172-329, src/infer/load.rs:10-92, src/infer/tensor_views.rs:29-117,
 *      src/infer/types.rs:114-242, src/infer/mapping.rs:95-540, src/infer/embeddings.rs:14-143) -------------- */
typedef struct M40HostGguf M40HostGguf;                 /* a parsed file header: no device, no tensor data */
typedef struct M40HostGgufWeights M40HostGgufWeights;   /* a file whose data section is resident on the device */
/* Parse magic, version, metadata and tensor descriptors (load_gguf).  NULL + m40host_last_error() when the file is
 * not GGUF, is truncated, or holds an unknown value type.  _parse does the same for a header held in memory. */
M40HostGguf* m40host_gguf_open(const char* path);
M40HostGguf* m40host_gguf_parse(const void* bytes, size_t n);
void m40host_gguf_close(M40HostGguf* gguf);
/* Everything the host layer derives from the header, as one JSON object: version, data_offset, file_len, metadata
 * (arrays cut to their first 32 elements, with "len"), tensors, then "config" (ModelConfig::from_metadata), "views"
 * (byte_offset, nbytes, strides per tensor), "layers" (per layer, the tensor chosen for each role of map_standard_layer,
 * or {"error": message}), "lm_head" (map_lm_head: name, d_model, vocab, tied) and "output_norm"; a stage that the reference
 * would reject appears as "<stage>_error" with the reference's message instead.  Returns the size needed including
 * the terminating zero; writes at most `capacity` bytes. */
size_t m40host_gguf_describe_json(const M40HostGguf* gguf, char* buf, size_t capacity);
/* Where one token's embedding starts in the data section, its length and the table's ggml dtype code
 * (embeddings.rs:33-60).  -1 + last_error for a token outside the vocabulary or an unsupported dtype. */
int m40host_gguf_embedding_row(const M40HostGguf* gguf, uint64_t token_id, uint64_t* byte_offset, uint64_t* row_bytes,
                               uint32_t* dtype_raw);
/* LoadedModel::from_gguf: parse, validate every tensor against the data section, then stream the data section into
 * one device allocation (m40llm_ext_upload_file_range).  Nothing is allocated when validation fails. */
M40HostGgufWeights* m40host_gguf_load(M40llmCudaContext* ctx, const char* path);
void m40host_gguf_weights_free(M40HostGgufWeights* weights);     /* after every model made from it is destroyed */
uint64_t m40host_gguf_weights_len(const M40HostGgufWeights* weights);
const void* m40host_gguf_weights_base(const M40HostGgufWeights* weights);
/* device address of a tensor = base + its offset in the data section; NULL + last_error for an unknown name */
const void* m40host_gguf_tensor_ptr(const M40HostGgufWeights* weights, const char* name);
/* load_token_embedding_to_f32: F16 rows widened, Q8_0 rows dequantised (d * q), both on the device */
int m40host_gguf_load_token_embedding_f32(const M40HostGgufWeights* weights, uint64_t token_id, void* d_out_f32);
/* A decoder that reads the file's tensors in place (validate_full_layer_decode, then the model of
 * m40host_model_create).  max_seq_len 0 = the file's context_length; kv_cfg NULL = dense cache. */
M40HostModel* m40host_model_from_gguf(M40HostGgufWeights* weights, uint32_t max_seq_len, uint32_t max_sequences,
                                      const M40HostKvConfig* kv_cfg);

#ifdef __cplusplus
}
#endif
#endif
