/*
 * m40llm C ABI, MI355X (gfx950) implementation.
 *
 * The drop-in boundary of the decode-step hot path: the `m40llm_*` symbols the
 * reference's Rust FFI block declares (src/cuda.rs:87-682) and its native side
 * defines (cuda/kernels.cu, C view in cuda/stub.c), with the same names, argument
 * meaning, stream behaviour and negative error codes.  Plain pointers and sizes
 * only.  Each declaration cites the reference definition it replaces.
 *
 * Conventions (all from the reference):
 *   - every function returns int (0 = ok, distinct negative code per failure
 *     site) or a handle (NULL = failure);
 *   - buffers are device pointers unless the name says host;
 *   - stream_kind: 0 = prefill stream, 1 = decode stream, anything else is an error
 *     (cuda/kernels.cu:287-292);
 *   - rope_layout: 0 = adjacent pairs (2i,2i+1), 1 = NeoX split half (i,i+hd/2);
 *   - weight_dtype: 0 = f16, 1 = f32;  exact_old_backing: 0 dense, 1 q8, 2 fp16-K/q4-V,
 *     3 (extension, M40LLM_EXT_OLD_BACKING_FP16_K_Q4G32_V) fp16-K with V 4-bit in groups of 32;
 *   - `_async` = enqueue on the decode stream and return; the GEMMs and
 *     f16_to_f32 / q80_to_f32 run on the prefill stream and block until done.
 *   - calls on one context are serialised by the caller (the reference holds a
 *     mutex around every FFI call, src/cuda.rs:1121-1137).
 *
 * Symbols of the reference that lie outside the decode hot path (staged / q8 /
 * lossy-summary attention modes, cuBLAS-only GEMM, persistent
 * decode prototype, telemetry readers) are exported and return their
 * "unavailable" code exactly as cuda/stub.c does (-1), so a binding that declares
 * all of them still links.  They are listed at the end of this header.
 *
 * Entry points that have no counterpart in the reference are prefixed
 * `m40llm_ext_` and say so.
 */
#ifndef M40LLM_H
#define M40LLM_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct M40llmCudaContext M40llmCudaContext;     /* src/cuda.rs:30-33   */
typedef struct M40llmKVCache M40llmKVCache;             /* src/cuda.rs:35-38   */
typedef struct M40llmCudaGraphExec M40llmCudaGraphExec; /* src/cuda.rs:40-42   */
typedef struct M40llmCudaEvent M40llmCudaEvent;         /* src/cuda.rs:43-45   */
typedef struct M40llmAttentionTelemetry M40llmAttentionTelemetry;

#define M40LLM_STREAM_PREFILL 0u
#define M40LLM_STREAM_DECODE 1u
#define M40LLM_ROPE_LAYOUT_ADJACENT 0u
#define M40LLM_ROPE_LAYOUT_NEOX 1u

/* ---- context, memory, streams (cuda/kernels.cu:276-514, 1245-1292, 7960ff) ---- */
M40llmCudaContext* m40llm_create_context(int device_id);                         /* kernels.cu:366-474 */
void m40llm_destroy_context(M40llmCudaContext* ctx);
int m40llm_current_device_props(char* name_buf, size_t buf_len, int* major, int* minor,
                                int* device_id);                                  /* kernels.cu:1245-1263 */
int m40llm_device_malloc(M40llmCudaContext* ctx, size_t bytes, void** out_ptr);   /* kernels.cu:302-310 */
int m40llm_device_free(M40llmCudaContext* ctx, void* ptr);                        /* kernels.cu:312-319 */
int m40llm_memcpy_h2d(M40llmCudaContext* ctx, void* dst_device, const void* src_host, size_t bytes);
int m40llm_memcpy_d2h(M40llmCudaContext* ctx, void* dst_host, const void* src_device, size_t bytes);
int m40llm_memcpy_d2d_async(M40llmCudaContext* ctx, void* dst_device, const void* src_device,
                            size_t bytes, uint32_t stream_kind);                  /* kernels.cu:337-355 */
int m40llm_validate_device_ptr(const void* ptr);                                  /* kernels.cu:357-364 */
int m40llm_upload_weights(M40llmCudaContext* ctx, const void* host_ptr, size_t num_bytes,
                          void** out_device_ptr);                                 /* kernels.cu:1268-1292 */
int m40llm_stream_synchronize(M40llmCudaContext* ctx, uint32_t stream_kind);      /* kernels.cu:476-484 */
int m40llm_stream_wait_for_stream(M40llmCudaContext* ctx, uint32_t waiting_stream_kind,
                                  uint32_t signal_stream_kind);                   /* kernels.cu:486-514 */

/* events and graphs (cuda/kernels.cu:516-680) */
int m40llm_cuda_event_create(M40llmCudaContext* ctx, M40llmCudaEvent** out_event);
int m40llm_cuda_event_record(M40llmCudaContext* ctx, M40llmCudaEvent* event, uint32_t stream_kind);
int m40llm_cuda_event_elapsed_sync(M40llmCudaContext* ctx, M40llmCudaEvent* start,
                                   M40llmCudaEvent* stop, float* elapsed_ms);
void m40llm_cuda_event_destroy(M40llmCudaEvent* event);
int m40llm_cuda_graph_begin_capture(M40llmCudaContext* ctx, uint32_t stream_kind);
int m40llm_cuda_graph_end_capture(M40llmCudaContext* ctx, uint32_t stream_kind,
                                  M40llmCudaGraphExec** out_graph);
int m40llm_cuda_graph_cancel_capture(M40llmCudaContext* ctx, uint32_t stream_kind);
int m40llm_cuda_graph_launch(M40llmCudaContext* ctx, M40llmCudaGraphExec* graph, uint32_t stream_kind);
int m40llm_cuda_graph_launch_timed_sync(M40llmCudaContext* ctx, M40llmCudaGraphExec* graph,
                                        uint32_t stream_kind, float* elapsed_ms);
void m40llm_cuda_graph_destroy(M40llmCudaGraphExec* graph);

/* ---- GEMV / GEMM: C[M,N] f32 row-major (cuda/kernels.cu:4981-5302) ------------- */
/* A f32 [M,K] x B f16 GGUF layout B[n*K + k]: the decode projection (kernels.cu:5158-5195) */
int m40llm_gemm_f32xf16_gguf_f32(M40llmCudaContext* ctx, const void* d_A_f32, const void* d_B_f16,
                                 void* d_C_f32, int M, int N, int K);
/* A f32 x B f16 row-major B[k*N + n] (kernels.cu:5106-5155) */
int m40llm_gemm_f32xf16_f32(M40llmCudaContext* ctx, const void* d_A_f32, const void* d_B_f16,
                            void* d_C_f32, int M, int N, int K);
/* A f16 x B f16 row-major -> f32 (kernels.cu:5267-5302) */
int m40llm_gemm_f16xf16_f32(M40llmCudaContext* ctx, const void* d_A_f16, const void* d_B_f16,
                            void* d_C_f32, int M, int N, int K);
/* A f16 x B f16 row-major -> f16, f32 accumulate (kernels.cu:5068-5103) */
int m40llm_gemm_f16_storage_f32_compute(M40llmCudaContext* ctx, const void* d_A, const void* d_B,
                                        void* d_C, int M, int N, int K);
/* GGUF f16 [N][K] -> f32 [K][N], then C[M,N] = A[M,K] x that operand (cuda/kernels.cu:5054-5066, 5197-5265; the
 * reference multiplies with cublasSgemm, here a plain f32 kernel).  Prefill stream; the non-async forms block. */
int m40llm_materialize_gguf_f16_to_f32_colmajor_nt(M40llmCudaContext* ctx, const void* d_B_f16,
                                                   void* d_B_f32_colmajor_nt, int N, int K);
int m40llm_gemm_f32xf32_f32(M40llmCudaContext* ctx, const void* d_A_f32, const void* d_B_f32_colmajor_nt,
                            void* d_C_f32, int M, int N, int K);
int m40llm_gemm_f32xf32_f32_async(M40llmCudaContext* ctx, const void* d_A_f32, const void* d_B_f32_colmajor_nt,
                                  void* d_C_f32, int M, int N, int K);
int m40llm_f16_to_f32(M40llmCudaContext* ctx, const void* d_in_f16, void* d_out_f32, size_t n);   /* :1129-1158 */
int m40llm_q80_to_f32(M40llmCudaContext* ctx, const void* d_in_q80, void* d_out_f32, size_t n);   /* :1160-1173 */

/* ---- elementwise, decode stream (cuda/kernels.cu:1036-1241, 7370-7546) ---------- */
int m40llm_rms_norm_f32(M40llmCudaContext* ctx, const void* d_in, void* d_out, uint32_t rows,
                        uint32_t dim, float eps);
int m40llm_rms_norm_f32_async(M40llmCudaContext* ctx, const void* d_in, void* d_out, uint32_t rows,
                              uint32_t dim, float eps);
int m40llm_rms_norm_f32_weighted(M40llmCudaContext* ctx, const void* d_in, const void* d_weight,
                                 void* d_out, uint32_t rows, uint32_t dim, float eps,
                                 uint32_t weight_dtype);
int m40llm_rms_norm_f32_weighted_async(M40llmCudaContext* ctx, const void* d_in, const void* d_weight,
                                       void* d_out, uint32_t rows, uint32_t dim, float eps,
                                       uint32_t weight_dtype);
int m40llm_rope_f32(M40llmCudaContext* ctx, void* d_q, void* d_k, uint32_t rows, uint32_t num_heads,
                    uint32_t head_dim, uint32_t past_len, float freq_base, float freq_scale);
int m40llm_rope_f32_async(M40llmCudaContext* ctx, void* d_q, void* d_k, uint32_t rows,
                          uint32_t num_heads, uint32_t head_dim, uint32_t past_len, float freq_base,
                          float freq_scale);
int m40llm_rope_f32_layout_async(M40llmCudaContext* ctx, void* d_q, void* d_k, uint32_t rows,
                                 uint32_t num_heads, uint32_t head_dim, uint32_t past_len,
                                 float freq_base, float freq_scale, uint32_t rope_layout);
int m40llm_rope_f32_inplace(M40llmCudaContext* ctx, void* d_x, uint32_t rows, uint32_t num_heads,
                            uint32_t head_dim, uint32_t past_len, float freq_base, float freq_scale);
int m40llm_rope_f32_inplace_async(M40llmCudaContext* ctx, void* d_x, uint32_t rows,
                                  uint32_t num_heads, uint32_t head_dim, uint32_t past_len,
                                  float freq_base, float freq_scale);
int m40llm_rope_f32_inplace_layout_async(M40llmCudaContext* ctx, void* d_x, uint32_t rows,
                                         uint32_t num_heads, uint32_t head_dim, uint32_t past_len,
                                         float freq_base, float freq_scale, uint32_t rope_layout);
int m40llm_rope_f32_inplace_position_dev_async(M40llmCudaContext* ctx, void* d_x, uint32_t rows,
                                               uint32_t num_heads, uint32_t head_dim,
                                               const uint32_t* past_len_dev, float freq_base,
                                               float freq_scale);
int m40llm_rope_f32_inplace_position_dev_layout_async(M40llmCudaContext* ctx, void* d_x, uint32_t rows,
                                                      uint32_t num_heads, uint32_t head_dim,
                                                      const uint32_t* past_len_dev, float freq_base,
                                                      float freq_scale, uint32_t rope_layout);
int m40llm_residual_add_f32(M40llmCudaContext* ctx, const void* d_a, const void* d_b, void* d_out, size_t n);
int m40llm_residual_add_f32_async(M40llmCudaContext* ctx, const void* d_a, const void* d_b, void* d_out, size_t n);
int m40llm_swiglu_f32(M40llmCudaContext* ctx, const void* d_gate, const void* d_up, void* d_out, size_t n);
int m40llm_swiglu_f32_async(M40llmCudaContext* ctx, const void* d_gate, const void* d_up, void* d_out, size_t n);

/* ---- KV cache (cuda/kernels.cu:5304-5543, 5793-6379) ---------------------------- */
M40llmKVCache* m40llm_kvcache_create(M40llmCudaContext* ctx, uint32_t max_seq_len,
                                     uint32_t max_batch_size, uint32_t num_heads, uint32_t head_dim);
/* Only exact_old_backing 0 (ring only), 2 (fp16-K/q4-V) and 3 allocate usable
 * storage here; backing 1 (q8) returns NULL.
 * Backing 3 has no counterpart in the reference: it is backing 2 with the old V rows held 4-bit in groups of 32
 * dimensions under an f16 scale and an f16 minimum (the V format the compressed-attention benchmark configuration
 * names; 80 bytes per token and head at head_dim 128 against 68).  Per group: d = f16((max - min) / 15),
 * m = f16(min), q = d > 0 ? clamp(lrintf((v - m) / d), 0, 15) : 0, value = fmaf(q, d, m).  Appends, evictions, the
 * block-select attention entry points and the debug read-backs take such a cache like a backing-2 cache;
 * m40llm_ext_kvcache_debug_read_raw(which = 2) returns head_dim / 32 words (bits of d | bits of m << 16) per token
 * and head instead of one f32 scale. */
#define M40LLM_EXT_OLD_BACKING_FP16_K_Q4G32_V 3u
M40llmKVCache* m40llm_kvcache_create_compressed(M40llmCudaContext* ctx, uint32_t max_seq_len,
                                                uint32_t max_batch_size, uint32_t num_heads,
                                                uint32_t head_dim, uint32_t recent_window,
                                                uint32_t block_size, uint32_t top_blocks,
                                                uint32_t representatives,
                                                uint32_t representative_policy,
                                                uint32_t exact_old_backing);
void m40llm_kvcache_destroy(M40llmKVCache* kv);
int m40llm_kvcache_reset(M40llmCudaContext* ctx, M40llmKVCache* kv);               /* :6308-6358 */
int m40llm_kvcache_append_token(M40llmCudaContext* ctx, M40llmKVCache* kv, uint32_t seq_id,
                                const void* k_dev_f16, const void* v_dev_f16);     /* :5793-5823 */
int m40llm_kvcache_append_token_f32(M40llmCudaContext* ctx, M40llmKVCache* kv, uint32_t seq_id,
                                    const void* k_dev_f32, const void* v_dev_f32);
int m40llm_kvcache_append_token_f32_async(M40llmCudaContext* ctx, M40llmKVCache* kv, uint32_t seq_id,
                                          const void* k_dev_f32, const void* v_dev_f32); /* :5837-5907 */
int m40llm_kvcache_append_token_f32_rope_k(M40llmCudaContext* ctx, M40llmKVCache* kv, uint32_t seq_id,
                                           const void* k_dev_f32, const void* v_dev_f32,
                                           uint32_t past_len, float freq_base, float freq_scale);
int m40llm_kvcache_append_token_f32_rope_k_async(M40llmCudaContext* ctx, M40llmKVCache* kv,
                                                 uint32_t seq_id, const void* k_dev_f32,
                                                 const void* v_dev_f32, uint32_t past_len,
                                                 float freq_base, float freq_scale);
int m40llm_kvcache_append_token_f32_rope_k_layout_async(M40llmCudaContext* ctx, M40llmKVCache* kv,
                                                        uint32_t seq_id, const void* k_dev_f32,
                                                        const void* v_dev_f32, uint32_t past_len,
                                                        float freq_base, float freq_scale,
                                                        uint32_t rope_layout);     /* :5976-6029 */
int m40llm_kvcache_append_token_f32_rope_k_at_async(M40llmCudaContext* ctx, M40llmKVCache* kv,
                                                    uint32_t seq_id, const void* k_dev_f32,
                                                    const void* v_dev_f32, uint32_t position,
                                                    uint32_t past_len, float freq_base,
                                                    float freq_scale);
/* dispatches to the compressed append/evict path when the cache is compressed (:6045-6093) */
int m40llm_kvcache_append_token_f32_rope_k_at_layout_async(M40llmCudaContext* ctx, M40llmKVCache* kv,
                                                           uint32_t seq_id, const void* k_dev_f32,
                                                           const void* v_dev_f32, uint32_t position,
                                                           uint32_t past_len, float freq_base,
                                                           float freq_scale, uint32_t rope_layout);
int m40llm_kvcache_append_token_f32_rope_k_compressed_at_async(M40llmCudaContext* ctx, M40llmKVCache* kv,
                                                               uint32_t seq_id, const void* k_dev_f32,
                                                               const void* v_dev_f32, uint32_t position,
                                                               float freq_base, float freq_scale);
int m40llm_kvcache_append_token_f32_rope_k_compressed_at_layout_async(
    M40llmCudaContext* ctx, M40llmKVCache* kv, uint32_t seq_id, const void* k_dev_f32,
    const void* v_dev_f32, uint32_t position, float freq_base, float freq_scale,
    uint32_t rope_layout);                                                         /* :6108-6250 */
int m40llm_kvcache_append_token_f32_rope_k_position_dev_async(M40llmCudaContext* ctx, M40llmKVCache* kv,
                                                              uint32_t seq_id, const void* k_dev_f32,
                                                              const void* v_dev_f32,
                                                              const uint32_t* position_dev,
                                                              float freq_base, float freq_scale);
int m40llm_kvcache_append_token_f32_rope_k_position_dev_layout_async(
    M40llmCudaContext* ctx, M40llmKVCache* kv, uint32_t seq_id, const void* k_dev_f32,
    const void* v_dev_f32, const uint32_t* position_dev, float freq_base, float freq_scale,
    uint32_t rope_layout);                                                         /* :6265-6306 */
/* one token as [kv_heads*head_dim] f16 K then V, host buffers (:6360-6379) */
int m40llm_kvcache_debug_read_token(M40llmCudaContext* ctx, M40llmKVCache* kv, uint32_t seq_id,
                                    uint32_t token, void* out_k_host, void* out_v_host);
/* telemetry twin of the block ranking: q-head 0 / kv-head 0 only (:6449-6677) */
int m40llm_kvcache_debug_select_old_blocks(M40llmCudaContext* ctx, const M40llmKVCache* kv,
                                           uint32_t seq_id, const void* q_dev_f32, uint32_t q_heads,
                                           uint32_t seq_len, uint32_t recent_window,
                                           uint32_t block_size, uint32_t top_blocks,
                                           uint32_t* out_blocks_host, float* out_scores_host,
                                           uint32_t* out_start_host, uint32_t* out_end_host,
                                           uint32_t* out_count, uint32_t max_out,
                                           uint32_t* out_total_old_blocks);

/* ---- attention, decode stream (cuda/kernels.cu:3837-4070, 4504-4577, 4694-4832) -- */
int m40llm_attention_last_token_f32(M40llmCudaContext* ctx, const M40llmKVCache* kv, uint32_t seq_id,
                                    const void* q_dev_f32, uint32_t seq_len, void* out_dev_f32);
int m40llm_attention_last_token_f32_gqa(M40llmCudaContext* ctx, const M40llmKVCache* kv,
                                        uint32_t seq_id, const void* q_dev_f32, uint32_t q_heads,
                                        uint32_t seq_len, void* out_dev_f32);
int m40llm_attention_last_token_f32_gqa_async(M40llmCudaContext* ctx, const M40llmKVCache* kv,
                                              uint32_t seq_id, const void* q_dev_f32, uint32_t q_heads,
                                              uint32_t seq_len, void* out_dev_f32);
int m40llm_attention_last_token_f32_gqa_seq_len_dev_async(M40llmCudaContext* ctx, const M40llmKVCache* kv,
                                                          uint32_t seq_id, const void* q_dev_f32,
                                                          uint32_t q_heads, const uint32_t* seq_len_dev,
                                                          void* out_dev_f32);
int m40llm_attention_last_token_f32_gqa_dense_recent_async(M40llmCudaContext* ctx, const M40llmKVCache* kv,
                                                           uint32_t seq_id, const void* q_dev_f32,
                                                           uint32_t q_heads, uint32_t seq_len,
                                                           uint32_t recent_window, void* out_dev_f32);
/* Variable-length batch: Q and Out packed [batch][q_heads][head_dim]; seq_ids / seq_lens are
 * device u32 arrays.  The reference accepts head_dim 64 and lengths <= 8192 only
 * (kernels.cu:4707, :4743); this implementation also takes head_dim 128 and any
 * length <= max_seq_len. */
int m40llm_attention_last_token_f32_gqa_batched(M40llmCudaContext* ctx, const M40llmKVCache* kv,
                                                const uint32_t* seq_ids_dev, const uint32_t* seq_lens_dev,
                                                uint32_t batch_size, const void* q_dev_f32,
                                                uint32_t q_heads, void* out_dev_f32);
int m40llm_attention_last_token_f32_gqa_batched_async(M40llmCudaContext* ctx, const M40llmKVCache* kv,
                                                      const uint32_t* seq_ids_dev,
                                                      const uint32_t* seq_lens_dev, uint32_t batch_size,
                                                      const void* q_dev_f32, uint32_t q_heads,
                                                      void* out_dev_f32);
/* block-select over a dense cache (reference: head_dim 64 only; 128 accepted here) */
int m40llm_attention_last_token_f32_gqa_block_select_exact_async(
    M40llmCudaContext* ctx, const M40llmKVCache* kv, uint32_t seq_id, const void* q_dev_f32,
    uint32_t q_heads, uint32_t seq_len, uint32_t recent_window, uint32_t block_size,
    uint32_t top_blocks, void* out_dev_f32);
/* block-select over the fp16-K / q4-V compressed cache, head_dim 64 or 128 */
int m40llm_attention_last_token_f32_gqa_block_select_exact_fp16_k_q4_v_old_direct_async(
    M40llmCudaContext* ctx, const M40llmKVCache* kv, uint32_t seq_id, const void* q_dev_f32,
    uint32_t q_heads, uint32_t seq_len, uint32_t recent_window, uint32_t block_size,
    uint32_t top_blocks, void* out_dev_f32);

/* ---- additions with no counterpart in the reference -------------------------------- */
/* q8_0 weights (34-byte blocks along K, GGUF order) -> C[M,N] f32.  The reference only
 * dequantises q8_0 elementwise (kernels.cu:856-867); this is that dequant followed by
 * the semantics of m40llm_gemm_f32xf16_gguf_f32.  Blocking, prefill stream. */
int m40llm_ext_gemm_f32xq80_gguf_f32(M40llmCudaContext* ctx, const void* d_A_f32, const void* d_B_q80,
                                     void* d_C_f32, int M, int N, int K);
/* The same product, asynchronous on the stream stream_kind names (0 prefill, 1 decode). */
int m40llm_ext_gemm_f32xq80_gguf_f32_async(M40llmCudaContext* ctx, const void* d_A_f32, const void* d_B_q80,
                                           void* d_C_f32, int M, int N, int K, uint32_t stream_kind);
/* out[M,d_model] = down(swiglu(gate(x), up(x))) with q8_0 matrices; d_scratch_f32 holds
 * 2*M*ffn floats.  Decode stream, asynchronous. */
int m40llm_ext_ffn_swiglu_q80_f32_async(M40llmCudaContext* ctx, const void* d_x_f32,
                                        const void* d_w_gate_q80, const void* d_w_up_q80,
                                        const void* d_w_down_q80, void* d_scratch_f32,
                                        void* d_out_f32, int M, int d_model, int ffn);
/* same contraction as m40llm_gemm_f32xf16_gguf_f32, enqueued on `stream_kind` without blocking */
int m40llm_ext_gemm_f32xf16_gguf_f32_async(M40llmCudaContext* ctx, const void* d_A_f32,
                                           const void* d_B_f16, void* d_C_f32, int M, int N, int K,
                                           uint32_t stream_kind);
/* One to three f16 weight matrices (GGUF order) applied to the same f32 activations A [M][K]: C_i [M][N_i] = A x B_i,
 * each exactly what m40llm_gemm_f32xf16_gguf_f32 computes.  The reference issues these as separate GEMMs
 * (qkv_project_f32xf16_gguf_f32_async and the gate/up pair, src/infer/forward.rs:2326-2338, 2471-2490); with many rows
 * they share one pass that splits A into f16 planes and one launch.  Unused matrix slots are NULL / 0.  Asynchronous on
 * `stream_kind`. */
int m40llm_ext_gemm_f32xf16_gguf_f32_multi_async(M40llmCudaContext* ctx, const void* d_A_f32, int M, int K, int n_mats,
                                                 const void* d_B0_f16, int N0, void* d_C0_f32, const void* d_B1_f16, int N1,
                                                 void* d_C1_f32, const void* d_B2_f16, int N2, void* d_C2_f32,
                                                 uint32_t stream_kind);
/* Per-q-head selection of the block-select path, computed by the same kernels that the
 * attention entry points run (the reference's debug selector covers q-head 0 only).
 * out_blocks_host: [q_heads][64] (0xffffffff beyond the count), out_counts_host: [q_heads],
 * out_scores_host (may be NULL): [q_heads][64]. Works on dense and compressed caches. */
int m40llm_ext_block_select_read_selection(M40llmCudaContext* ctx, const M40llmKVCache* kv,
                                           uint32_t seq_id, const void* q_dev_f32, uint32_t q_heads,
                                           uint32_t seq_len, uint32_t recent_window,
                                           uint32_t block_size, uint32_t top_blocks,
                                           uint32_t* out_blocks_host, uint32_t* out_counts_host,
                                           float* out_scores_host);
/* The fp16-K / q4-V block-select attention of up to 8 different sequences (slots) in one set of launches, so that
 * independent slots overlap on the device.  seq_ids_host / seq_lens_host are host arrays of n_slots entries;
 * q_dev_f32 and out_dev_f32 hold n_slots rows of q_heads * head_dim floats.  Same results and error codes as
 * n_slots calls of m40llm_attention_last_token_f32_gqa_block_select_exact_fp16_k_q4_v_old_direct_async. */
int m40llm_ext_attention_block_select_fp16_k_q4_v_multi_async(
    M40llmCudaContext* ctx, const M40llmKVCache* kv, uint32_t n_slots, const uint32_t* seq_ids_host,
    const uint32_t* seq_lens_host, const void* q_dev_f32, uint32_t q_heads, uint32_t recent_window, uint32_t block_size,
    uint32_t top_blocks, void* out_dev_f32);
/* Fill positions [0, seq_len) of one sequence from f16 K/V rows [seq_len][kv_heads][head_dim]
 * on the device, leaving the cache exactly as seq_len ordered appends of those (already
 * rotated) rows would: dense caches get the rows, compressed caches get old-K copies,
 * q4 V + scales for positions < seq_len - recent_window and ring rows for the rest. */
int m40llm_ext_kvcache_bulk_fill_f16(M40llmCudaContext* ctx, M40llmKVCache* kv, uint32_t seq_id,
                                     const void* k_dev_f16, const void* v_dev_f16, uint32_t seq_len);
/* Packed variable-length causal prefill attention, all f32 (cuda/kernels.cu:3749-3835, entry points :4834-4977;
 * declared src/cuda.rs:619-648; CPU restatement tests/attention_prefill_varlen.rs:27-76).
 * Q and Out: [total_q][q_heads][head_dim]; K and V: [total_kv][kv_heads][head_dim]; sequence b owns q_lens[b] query
 * tokens from q_offsets[b] and kv_lens[b] keys from kv_offsets[b] (token units, device arrays); query q_idx attends
 * keys 0 .. kv_len - q_len + q_idx.  Prefill stream.  The lengths are read back and validated on the host before the
 * launch in both forms, as in the reference; only the first form waits for the kernel.
 * -1 null argument, -2 batch 0, -3 head counts, -9 head_dim not 64 / 128, -7 read-back failed,
 * -8 a length is 0, q_len > kv_len or kv_len > 8192, or the key ranges of the sequences are not laid out one after the
 * other in batch order (kv_offsets[b + 1] >= kv_offsets[b] + kv_lens[b]: how packed batches are built; this
 * implementation packs K and V by sequence), -4 launch, allocation or 16-byte misaligned Q/K/V, -5 synchronise. */
int m40llm_attention_prefill_f32_gqa_varlen(M40llmCudaContext* ctx, const void* q_dev_f32, const void* k_dev_f32,
                                            const void* v_dev_f32, const uint32_t* q_offsets_dev,
                                            const uint32_t* kv_offsets_dev, const uint32_t* q_lens_dev,
                                            const uint32_t* kv_lens_dev, uint32_t batch_size, uint32_t q_heads,
                                            uint32_t kv_heads, uint32_t head_dim, void* out_dev_f32);
int m40llm_attention_prefill_f32_gqa_varlen_async(M40llmCudaContext* ctx, const void* q_dev_f32, const void* k_dev_f32,
                                                  const void* v_dev_f32, const uint32_t* q_offsets_dev,
                                                  const uint32_t* kv_offsets_dev, const uint32_t* q_lens_dev,
                                                  const uint32_t* kv_lens_dev, uint32_t batch_size, uint32_t q_heads,
                                                  uint32_t kv_heads, uint32_t head_dim, void* out_dev_f32);

/* m40llm_attention_prefill_f32_gqa_varlen_async for a caller that also holds the key offsets and the lengths on the host
 * (the same values as the device arrays, which the kernels read): validated from the host copies, so the call does not
 * read the device arrays back -- each read-back waits for everything enqueued so far, once per layer of a prefill.  No
 * counterpart in the reference (its launcher reads the lengths back).  Same codes; -1 also for a NULL host table. */
int m40llm_ext_attention_prefill_f32_gqa_varlen_host_tables_async(M40llmCudaContext* ctx, const void* q_dev_f32,
                                                                  const void* k_dev_f32, const void* v_dev_f32,
                                                                  const uint32_t* q_offsets_dev, const uint32_t* kv_offsets_dev,
                                                                  const uint32_t* q_lens_dev, const uint32_t* kv_lens_dev,
                                                                  const uint32_t* kv_offsets_host, const uint32_t* q_lens_host,
                                                                  const uint32_t* kv_lens_host, uint32_t batch_size,
                                                                  uint32_t q_heads, uint32_t kv_heads, uint32_t head_dim,
                                                                  void* out_dev_f32);

/* raw views of the compressed cache for tests: which = 0 old_k, 1 q4_v, 2 q4_scale, 3 recent_k,
 * 4 recent_v, 5 seq_map; copies `bytes` from byte offset `offset` to the host */
int m40llm_ext_kvcache_debug_read_raw(M40llmCudaContext* ctx, const M40llmKVCache* kv, uint32_t which,
                                      size_t offset, size_t bytes, void* out_host);
/* first index of the maximum of each row of logits [rows][n] -> out_idx_dev u32 [rows]; also
 * writes the top-1 minus top-2 gap to out_gap_dev (may be NULL).  Decode stream. */
int m40llm_ext_argmax_f32_async(M40llmCudaContext* ctx, const void* d_logits_f32, uint32_t rows,
                                size_t n, uint32_t* out_idx_dev, float* out_gap_dev);
/* DIAGNOSTIC, not part of the decode path.  Bandwidth yardstick (no counterpart in the reference): reads `bytes` (16-byte aligned start) of device memory
 * once, `workgroups` (<= 65536) workgroups of 256 threads each owning a contiguous range, and xors every 32-bit word
 * read into d_out_u32[0 .. 2047] (word = workgroup index modulo 2048; not cleared by the call).  One launch on the
 * decode stream; the benchmarks time it beside the kernels it bounds. */
int m40llm_ext_read_probe_async(M40llmCudaContext* ctx, const void* d_src, size_t bytes, uint32_t workgroups,
                                uint32_t* d_out_u32);
/* Prefill, steps between the Q/K/V projections and the attention for a packed batch of prompts, one launch instead
 * of three per token (src/infer/forward.rs:2349-2396: append_token_f32_rope_k_at_layout + rope_f32_inplace_layout on
 * the Q row + on the K row, per token).  Rows are packed sequence after sequence (sequence i holds q_lens_host[i]
 * rows); row j of sequence i is the token at position start_pos_host[i] + j (start_pos_host NULL = 0) of cache slot
 * seq_slots_host[i].  d_q [rows][q_heads][head_dim] and d_k [rows][kv_heads][head_dim] are rotated in place (f32);
 * the rotated K and d_v are cast to f16 into the cache, and the slot's length becomes start + len.  With the three
 * bias vectors (all or none) Q, K and V first receive their bias in place (the per-row residual adds of
 * forward.rs:149-160).  Bit-identical to the per-token calls.  Dense caches, at most 64 sequences, distinct slots.  Decode stream.
 * -1 null, -2 batch / slot / q_heads / layout, -3/-4 cache geometry, -5 past max_seq_len, -7 empty sequence,
 * -8 a slot named twice, -9 compressed cache, -6 launch. */
int m40llm_ext_prefill_rope_append_async(M40llmCudaContext* ctx, M40llmKVCache* kv, void* d_q_f32, void* d_k_f32,
                                         void* d_v_f32, uint32_t batch, const uint32_t* seq_slots_host,
                                         const uint32_t* q_lens_host, const uint32_t* start_pos_host, uint32_t q_heads,
                                         float freq_base, float freq_scale, uint32_t rope_layout, const void* d_bq_f32,
                                         const void* d_bk_f32, const void* d_bv_f32);
/* The same launch on the stream `stream_kind` names (0 prefill, 1 decode), so that a prefill can keep all of its launches on
 * one stream.  No counterpart in the reference (its per-token calls run on the decode stream). */
int m40llm_ext_prefill_rope_append_on_stream_async(M40llmCudaContext* ctx, M40llmKVCache* kv, void* d_q_f32, void* d_k_f32,
                                                   void* d_v_f32, uint32_t batch, const uint32_t* seq_slots_host,
                                                   const uint32_t* q_lens_host, const uint32_t* start_pos_host,
                                                   uint32_t q_heads, float freq_base, float freq_scale, uint32_t rope_layout,
                                                   const void* d_bq_f32, const void* d_bk_f32, const void* d_bv_f32,
                                                   uint32_t stream_kind);
/* Many-row projections of the packed prefill with the element-wise step before them and the residual add after them
 * folded in (src/infer/forward.rs:2300-2345, 2440-2530 issue these as rms_norm / swiglu, the GEMMs and residual_add, one
 * launch each).  The rows that enter the product are, by source_kind,
 *   0: d_a_f32 [M][K] as it is;
 *   1: what m40llm_rms_norm_f32_weighted writes for d_a_f32 with d_norm_weight (f16: norm_weight_dtype 0, f32: 1) and eps;
 *   2: what m40llm_swiglu_f32 writes for gate = d_a_f32 and up = d_a2_f32, both [M][K];
 * produced inside the pass that splits the rows into f16 planes, never written out as f32.  C_i [M][N_i] = rows x B_i (one
 * to three f16 GGUF matrices, as m40llm_ext_gemm_f32xf16_gguf_f32_multi_async); with one matrix and d_R0_f32 [M][N0] not NULL
 * C_0 = R_0 + product, what m40llm_residual_add_f32 gives (d_R0_f32 may be d_C0_f32).  Every result has the bits of
 * that sequence of calls (element-wise call, m40llm_ext_gemm_f32xf16_gguf_f32_multi_async over the same matrices, residual add).  Returns 0 when enqueued on `stream_kind`, 1 when the shapes are not the many-row kernel's (M <= 32, K not
 * a multiple of 32, an operand not 16-byte aligned) or its buffer cannot be provided -- nothing was enqueued and the caller
 * issues the separate calls -- and -1 / -2 / -3 for a NULL, an argument out of range, a launch failure. */
int m40llm_ext_prefill_gemm_fused_async(M40llmCudaContext* ctx, uint32_t source_kind, const void* d_a_f32, const void* d_a2_f32,
                                        const void* d_norm_weight, uint32_t norm_weight_dtype, float eps, int M, int K,
                                        int n_mats, const void* d_B0_f16, int N0, void* d_C0_f32, const void* d_R0_f32,
                                        const void* d_B1_f16, int N1, void* d_C1_f32, const void* d_B2_f16, int N2,
                                        void* d_C2_f32, uint32_t stream_kind);
/* embedding rows of `rows` (<= 65535) token ids held on the device (f16 table [vocab][d_model]) -> f32 [rows][d_model];
 * the row form of m40llm_ext_embed_token_dev_async (src/infer/forward.rs:2241-2250 loads them one blocking call per
 * token).  Decode stream. */
int m40llm_ext_embed_rows_async(M40llmCudaContext* ctx, const void* d_table_f16, const uint32_t* tokens_dev, uint32_t rows,
                                uint32_t vocab, uint32_t d_model, void* d_out_f32);
/* Weight-file ingestion: `num_bytes` of the file at `path`, from byte `file_offset`, into one new device allocation
 * (*out_device_ptr, released with m40llm_device_free).  Replaces read-the-file + m40llm_upload_weights
 * (src/infer/load.rs:27-40, kernels.cu:1264-1290): positional reads into two pinned staging buffers overlap the
 * copies to the device, and nothing the size of the file is held in host memory.  Blocks until the data is resident.
 * -1 null argument, -2 device / allocation, -3 copy, -6 the file cannot be opened or the range is not inside it. */
int m40llm_ext_upload_file_range(M40llmCudaContext* ctx, const char* path, uint64_t file_offset, uint64_t num_bytes,
                                 void** out_device_ptr);
/* Fused batch-1 decode-step entry points (decode stream, asynchronous).  They compute exactly what the
 * reference's per-op call sequence computes (src/infer/forward.rs:304-662), several steps per launch:
 *   steps 1-5: RMSNorm -> Q/K/V projections (+bias) -> RoPE(Q) -> d_q_out; RoPE(K) and V -> f16 append at the
 *              position (taken from position_dev when that is not NULL); dense caches only. */
int m40llm_ext_fused_norm_qkv_rope_append_async(
    M40llmCudaContext* ctx, M40llmKVCache* kv, uint32_t seq_id, const void* d_x_f32, const void* d_norm_w,
    uint32_t norm_weight_dtype, float eps, const void* d_wq_f16, const void* d_wk_f16, const void* d_wv_f16,
    const void* d_bq_f32, const void* d_bk_f32, const void* d_bv_f32, uint32_t d_model, uint32_t q_heads,
    uint32_t position, const uint32_t* position_dev, float freq_base, float freq_scale, uint32_t rope_layout, void* d_q_out_f32);
/*   steps 7-8 / 12-13: out = residual + W . a (residual may be NULL or alias out) */
int m40llm_ext_gemv_residual_f32xf16_async(M40llmCudaContext* ctx, const void* d_a_f32, const void* d_w_f16,
                                           const void* d_residual_f32, void* d_out_f32, int N, int K);
/*   steps 9-11: hid = silu(Wgate . xn) * (Wup . xn), xn = RMSNorm(x) * w */
int m40llm_ext_fused_norm_gate_up_swiglu_async(M40llmCudaContext* ctx, const void* d_x_f32, const void* d_norm_w,
                                               uint32_t norm_weight_dtype, float eps, const void* d_wgate_f16,
                                               const void* d_wup_f16, void* d_hid_f32, int ffn, int d_model);
/*   output norm + lm_head (src/infer/logits.rs:57-116 without the copy to the host) */
/*   With d_block_top2 (3 planes of top2_capacity 4-byte entries: largest, second largest, first index of the
 *   largest, one entry per workgroup) the kernel also leaves per-workgroup top-2 candidates for
 *   m40llm_ext_greedy_step_async; *out_n_blocks (host) receives the number of entries. */
int m40llm_ext_fused_norm_gemv_f32xf16_async(M40llmCudaContext* ctx, const void* d_x_f32, const void* d_norm_w,
                                             uint32_t norm_weight_dtype, float eps, const void* d_w_f16,
                                             void* d_out_f32, int N, int K, void* d_block_top2,
                                             uint32_t top2_capacity, uint32_t* out_n_blocks);
/* attention with the length taken from the device: seq_len = *position_dev + 1 <= max_len_hint (the launch is sized
 * for max_len_hint tokens: with a longer sequence nothing is written) */
int m40llm_ext_attention_last_token_f32_gqa_position_dev_async(M40llmCudaContext* ctx, const M40llmKVCache* kv,
                                                               uint32_t seq_id, const void* q_dev_f32,
                                                               uint32_t q_heads, const uint32_t* position_dev,
                                                               uint32_t max_len_hint, void* out_dev_f32);
/* embedding row of the token id stored at token_dev (f16 table [vocab][d_model]) -> f32 */
/* No counterpart in the reference.  m40llm_attention_last_token_f32_gqa_async for callers that cannot allocate:
 * code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  Same argument checks, kernels
 * and results as that entry point, but the chunk partials of rows longer than 512 tokens go into a fixed 2 MiB
 * device array that is part of the library's code object (one copy per GPU, resolved once per device when a context
 * is created), and the call allocates nothing.  Returns -9 when the partials of this (q_heads, head_dim, seq_len) do
 * not fit 2 MiB: q_heads * chunks * (head_dim + 2) * 4 bytes, chunks = ceil(seq_len / chunk) with the chunk length
 * the allocating entry point uses.  Every call on one GPU shares that array: calls on the decode stream of one context
 * are ordered and safe; a call from another context while the last user's launches are still outstanding returns -10
 * (busy) instead of racing.  Captured calls are not guarded (no event can be queried under capture): graph replays
 * that overlap on one GPU race. */
int m40llm_ext_attention_last_token_f32_gqa_static_scratch_async(M40llmCudaContext* ctx, const M40llmKVCache* kv,
                                                                 uint32_t seq_id, const void* q_dev_f32,
                                                                 uint32_t q_heads, uint32_t seq_len,
                                                                 void* out_dev_f32);
int m40llm_ext_embed_token_dev_async(M40llmCudaContext* ctx, const void* d_table_f16, const uint32_t* token_dev,
                                     uint32_t vocab, uint32_t d_model, void* d_out_f32);
/* device-side greedy step over logits[n] (scanned directly, or through the per-workgroup candidates in
 * d_block_top2): state_dev = {position, step, token, capacity, ids[capacity], gaps[capacity] (f32 bits)}; stores
 * the first index of the maximum and the top-1/top-2 gap at [step], sets token, increments step and position.
 * With d_table_f16 (f16 [n][d_model]) the embedding row of the picked token is written to d_x_out_f32. */
int m40llm_ext_greedy_step_async(M40llmCudaContext* ctx, const void* d_logits_f32, uint32_t n,
                                 const void* d_block_top2, uint32_t top2_capacity, uint32_t n_blocks,
                                 uint32_t* state_dev, const void* d_table_f16, uint32_t d_model, void* d_x_out_f32);
/* Fused row-batched decode step (1 <= rows <= 16, decode stream, asynchronous; dense caches, f16 weights, K a
 * multiple of 256).  They compute what the reference's row-batched sequence computes (src/infer/forward.rs:1729-2140),
 * several steps per call, on the MFMA skinny GEMM.  seq_lens_dev[row] is the number of tokens the row's cache holds
 * before the step (= the position of the new token); ids and lengths are read on the device only.
 *   RMSNorm -> Q/K/V projections (+bias) -> RoPE at each row's position -> q; K, V -> f16 cache rows */
int m40llm_ext_batched_norm_qkv_rope_append_async(
    M40llmCudaContext* ctx, M40llmKVCache* kv, const uint32_t* seq_ids_dev, const uint32_t* seq_lens_dev, uint32_t rows,
    const void* d_x_f32, const void* d_norm_w, uint32_t norm_weight_dtype, float eps, const void* d_wq_f16,
    const void* d_wk_f16, const void* d_wv_f16, const void* d_bq_f32, const void* d_bk_f32, const void* d_bv_f32,
    uint32_t d_model, uint32_t q_heads, float freq_base, float freq_scale, uint32_t rope_layout, void* d_q_out_f32);
/*   attention of every row over seq_lens_dev[row] + len_bias tokens (no host-side validation: rows with an id or
 *   length out of range are skipped); max_len_hint >= every row's length: the launch is sized for it, and a row
 *   that is longer is skipped like one out of range */
int m40llm_ext_attention_last_token_f32_gqa_batched_lens_dev_async(M40llmCudaContext* ctx, const M40llmKVCache* kv,
                                                                   const uint32_t* seq_ids_dev,
                                                                   const uint32_t* seq_lens_dev, uint32_t len_bias,
                                                                   uint32_t batch_size, uint32_t max_len_hint,
                                                                   const void* q_dev_f32, uint32_t q_heads,
                                                                   void* out_dev_f32);
/*   out[rows][N] = residual + a[rows][K] . W^T (residual may be NULL or alias out) */
int m40llm_ext_batched_gemm_residual_f32xf16_async(M40llmCudaContext* ctx, const void* d_a_f32, const void* d_w_f16,
                                                   const void* d_residual_f32, void* d_out_f32, uint32_t rows, int N, int K);
/*   hid[rows][ffn] = silu(gate(xn)) * up(xn), xn = RMSNorm(x) * w */
int m40llm_ext_batched_norm_gate_up_swiglu_async(M40llmCudaContext* ctx, const void* d_x_f32, const void* d_norm_w,
                                                 uint32_t norm_weight_dtype, float eps, const void* d_wgate_f16,
                                                 const void* d_wup_f16, void* d_hid_f32, uint32_t rows, int ffn, int d_model);
/*   the same, and clear_floats floats at d_clear_f32 are set to zero on the side (the result of a following
 *   ..._onto_zero call; d_clear_f32 NULL: nothing is cleared) */
int m40llm_ext_batched_norm_gate_up_swiglu_clear_async(M40llmCudaContext* ctx, const void* d_x_f32, const void* d_norm_w,
                                                       uint32_t norm_weight_dtype, float eps, const void* d_wgate_f16,
                                                       const void* d_wup_f16, void* d_hid_f32, uint32_t rows, int ffn,
                                                       int d_model, void* d_clear_f32, uint32_t clear_floats);
/*   out[rows][N] = residual + a[rows][K] . W^T for an out that HOLDS ZEROS stored by an earlier call on the decode
 *   stream (the ..._clear call above) and overlaps neither a nor residual: with rows <= 8, a long K and few columns (the
 *   down projection) one launch whose workgroups add the two halves of K into out -- two terms onto zero, the same
 *   bits in either order; any other shape falls to m40llm_ext_batched_gemm_residual_f32xf16_async, which overwrites */
int m40llm_ext_batched_gemm_residual_onto_zero_f32xf16_async(M40llmCudaContext* ctx, const void* d_a_f32, const void* d_w_f16,
                                                             const void* d_residual_f32, void* d_out_f32, uint32_t rows, int N,
                                                             int K);
/*   out[rows][N] = (RMSNorm(x) * w) . W^T  (output norm + lm_head) */
int m40llm_ext_batched_norm_gemm_f32xf16_async(M40llmCudaContext* ctx, const void* d_x_f32, const void* d_norm_w,
                                               uint32_t norm_weight_dtype, float eps, const void* d_w_f16, void* d_out_f32,
                                               uint32_t rows, int N, int K);
/*   per row: first index of the maximum of logits[row][n] and the top-1/top-2 gap -> ids_dev/gaps_dev[row][step of the
 *   row] (row stride = capacity); seq_lens_dev[row] += 1; embedding row of the pick -> d_x_out_f32[row].
 *   state_dev = {unused, capacity, step of row 0, step of row 1, ...} */
int m40llm_ext_batched_greedy_step_async(M40llmCudaContext* ctx, const void* d_logits_f32, uint32_t rows, uint32_t n,
                                         uint32_t* state_dev, uint32_t* seq_lens_dev, uint32_t* ids_dev, float* gaps_dev,
                                         const void* d_table_f16, uint32_t d_model, void* d_x_out_f32);
const char* m40llm_ext_build_info(void);

/* ---- present but unavailable (return -1, as cuda/stub.c does) ---------------------- */
int m40llm_kvcache_build_q8_old_from_dense(M40llmCudaContext*, M40llmKVCache*, uint32_t, uint32_t, uint32_t);
int m40llm_kvcache_build_compressed_from_dense(M40llmCudaContext*, M40llmKVCache*, const M40llmKVCache*, uint32_t);
int m40llm_kvcache_debug_read_compressed_state(M40llmCudaContext*, M40llmKVCache*, uint32_t, uint32_t*,
                                               uint32_t*, void*, void*, float*, float*, void*, void*,
                                               void*, void*, uint32_t*);
int m40llm_kvcache_debug_attention_telemetry(M40llmCudaContext*, const M40llmKVCache*, uint32_t, uint32_t,
                                             const void*, uint32_t, uint32_t, uint32_t, uint32_t, uint32_t,
                                             uint32_t, M40llmAttentionTelemetry*);
int m40llm_attention_last_token_f32_gqa_block_select_exact_staged_async(
    M40llmCudaContext*, const M40llmKVCache*, uint32_t, const void*, uint32_t, uint32_t, uint32_t,
    uint32_t, uint32_t, void*);
int m40llm_attention_last_token_f32_gqa_block_select_exact_staged_with_buffers_async(
    M40llmCudaContext*, const M40llmKVCache*, uint32_t, const void*, uint32_t, uint32_t, uint32_t,
    uint32_t, uint32_t, void*, void*, void*, void*, uint32_t, void*);
int m40llm_attention_last_token_f32_gqa_block_select_exact_staged_q8_old_with_buffers_async(
    M40llmCudaContext*, const M40llmKVCache*, uint32_t, const void*, uint32_t, uint32_t, uint32_t,
    uint32_t, uint32_t, void*, void*, void*, void*, uint32_t, void*);
int m40llm_attention_last_token_f32_gqa_block_select_exact_staged_fp16_k_q4_v_old_with_buffers_async(
    M40llmCudaContext*, const M40llmKVCache*, uint32_t, const void*, uint32_t, uint32_t, uint32_t,
    uint32_t, uint32_t, void*, void*, void*, void*, uint32_t, void*);
int m40llm_attention_last_token_f32_gqa_block_select_exact_q8_old_direct_async(
    M40llmCudaContext*, const M40llmKVCache*, uint32_t, const void*, uint32_t, uint32_t, uint32_t,
    uint32_t, uint32_t, void*);
int m40llm_attention_last_token_f32_gqa_block_summary_lossy_async(
    M40llmCudaContext*, const M40llmKVCache*, uint32_t, const void*, uint32_t, uint32_t, uint32_t,
    uint32_t, uint32_t, void*);
int m40llm_attention_last_token_f32_gqa_compressed_recent_only_async(
    M40llmCudaContext*, const M40llmKVCache*, uint32_t, const void*, uint32_t, uint32_t, void*);
int m40llm_start_persistent_decode(M40llmCudaContext*);
int m40llm_stop_persistent_decode(M40llmCudaContext*);
int m40llm_persistent_decode_submit_vec(M40llmCudaContext*, const void*, void*, uint32_t, float, float,
                                        uint32_t, uint32_t*);
int m40llm_persistent_decode_poll(M40llmCudaContext*, uint32_t*, uint32_t*);

#ifdef __cplusplus
}
#endif
#endif /* M40LLM_H */
