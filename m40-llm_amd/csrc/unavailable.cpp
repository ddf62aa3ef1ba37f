// Symbols of the reference's FFI surface that lie outside the decode hot path.  They are
// exported so that a binding which declares the whole surface links, and every one reports
// "unavailable" the way the reference's own non-CUDA build does (cuda/stub.c: return -1).
#include "../../include/m40llm.h"

#define M40_UNAVAILABLE -1

extern "C" {

int m40llm_kvcache_build_q8_old_from_dense(M40llmCudaContext*, M40llmKVCache*, uint32_t, uint32_t, uint32_t) { return M40_UNAVAILABLE; }
int m40llm_kvcache_build_compressed_from_dense(M40llmCudaContext*, M40llmKVCache*, const M40llmKVCache*, uint32_t) { return M40_UNAVAILABLE; }
int m40llm_kvcache_debug_read_compressed_state(M40llmCudaContext*, M40llmKVCache*, uint32_t, uint32_t*, uint32_t*,
                                               void*, void*, float*, float*, void*, void*, void*, void*, uint32_t*) {
    return M40_UNAVAILABLE;
}
int m40llm_kvcache_debug_attention_telemetry(M40llmCudaContext*, const M40llmKVCache*, uint32_t, uint32_t, const void*,
                                             uint32_t, uint32_t, uint32_t, uint32_t, uint32_t, uint32_t,
                                             M40llmAttentionTelemetry*) {
    return M40_UNAVAILABLE;
}
int m40llm_attention_last_token_f32_gqa_block_select_exact_staged_async(M40llmCudaContext*, const M40llmKVCache*,
                                                                        uint32_t, const void*, uint32_t, uint32_t,
                                                                        uint32_t, uint32_t, uint32_t, void*) {
    return M40_UNAVAILABLE;
}
int m40llm_attention_last_token_f32_gqa_block_select_exact_staged_with_buffers_async(
    M40llmCudaContext*, const M40llmKVCache*, uint32_t, const void*, uint32_t, uint32_t, uint32_t, uint32_t, uint32_t,
    void*, void*, void*, void*, uint32_t, void*) {
    return M40_UNAVAILABLE;
}
int m40llm_attention_last_token_f32_gqa_block_select_exact_staged_q8_old_with_buffers_async(
    M40llmCudaContext*, const M40llmKVCache*, uint32_t, const void*, uint32_t, uint32_t, uint32_t, uint32_t, uint32_t,
    void*, void*, void*, void*, uint32_t, void*) {
    return M40_UNAVAILABLE;
}
int m40llm_attention_last_token_f32_gqa_block_select_exact_staged_fp16_k_q4_v_old_with_buffers_async(
    M40llmCudaContext*, const M40llmKVCache*, uint32_t, const void*, uint32_t, uint32_t, uint32_t, uint32_t, uint32_t,
    void*, void*, void*, void*, uint32_t, void*) {
    return M40_UNAVAILABLE;
}
int m40llm_attention_last_token_f32_gqa_block_select_exact_q8_old_direct_async(M40llmCudaContext*, const M40llmKVCache*,
                                                                               uint32_t, const void*, uint32_t, uint32_t,
                                                                               uint32_t, uint32_t, uint32_t, void*) {
    return M40_UNAVAILABLE;
}
int m40llm_attention_last_token_f32_gqa_block_summary_lossy_async(M40llmCudaContext*, const M40llmKVCache*, uint32_t,
                                                                  const void*, uint32_t, uint32_t, uint32_t, uint32_t,
                                                                  uint32_t, void*) {
    return M40_UNAVAILABLE;
}
int m40llm_attention_last_token_f32_gqa_compressed_recent_only_async(M40llmCudaContext*, const M40llmKVCache*, uint32_t,
                                                                     const void*, uint32_t, uint32_t, void*) {
    return M40_UNAVAILABLE;
}
int m40llm_start_persistent_decode(M40llmCudaContext*) { return M40_UNAVAILABLE; }
int m40llm_stop_persistent_decode(M40llmCudaContext*) { return M40_UNAVAILABLE; }
int m40llm_persistent_decode_submit_vec(M40llmCudaContext*, const void*, void*, uint32_t, float, float, uint32_t,
                                        uint32_t*) {
    return M40_UNAVAILABLE;
}
int m40llm_persistent_decode_poll(M40llmCudaContext*, uint32_t*, uint32_t*) { return M40_UNAVAILABLE; }

}  // extern "C"
