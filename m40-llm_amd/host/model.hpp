// One-token decoder step orchestration above the C ABI: single-sequence and row-batched
// variable-length decode, logits, greedy decode loops.
//
// Mirrors, for the decode path only:
//   forward_one_token_minimal_with_norms          src/infer/forward.rs:246-667  (14 FFI calls / layer)
//   forward_one_token_all_layers_for_sequence     src/infer/forward.rs:1659-1716 (ping-pong buffers)
//   forward_one_token_all_layers_batched_...      src/infer/forward.rs:1729-2140
//   KV slot addressing slot = seq * layers + layer src/infer/kv.rs:77-121
//   run_attention_async mode dispatch              src/infer/kv.rs:433-765 (Off and block-select-exact
//                                                  with the fp16-K/q4-V direct backing)
//   logits_from_hidden_into                        src/infer/logits.rs:57-116
//   load_token_embedding_to_f32 (F16 rows)         src/infer/embeddings.rs:64-79
//   DecodeSession::logits_for_ids token loop       src/decode_session.rs:637-703
//
// Two execution modes share the same arithmetic contract:
//   mode 0 "reference calls": exactly the reference's sequence of m40llm_* calls, GEMMs on the
//           prefill stream, everything else on the decode stream, ordered by stream waits.
//   mode 1 "fused": single decode stream, fused entry points (m40llm_ext_*), device-side greedy.
#pragma once

#include <chrono>
#include <cmath>
#include <cstdint>
#include <cstring>
#include <optional>
#include <stdexcept>
#include <string>
#include <vector>

#include "../../include/m40llm.h"
#include "decode_batch.hpp"
#include "kv_compression.hpp"
#include "kv_selection.hpp"
#include "sampling.hpp"

namespace m40host {

struct ModelConfig {
    uint32_t n_layers, d_model, q_heads, kv_heads, head_dim, ffn, vocab;
    float rms_eps, rope_base, rope_scale;
    uint32_t rope_layout;         // 0 adjacent (Llama), 1 NeoX (Qwen): src/infer/types.rs:34-40
    uint32_t has_qkv_bias;
    uint32_t norm_weight_dtype;   // 0 f16, 1 f32
    uint32_t max_seq_len, max_sequences;
};

struct LayerWeights {   // device pointers; f16 GGUF layout [N cols][K]
    const void *wq, *wk, *wv, *wo, *wgate, *wup, *wdown;
    const void *bq, *bk, *bv;         // f32, or all null
    const void *attn_norm, *ffn_norm;
};

#define M40H_TRY(expr)                                                                    \
    do {                                                                                  \
        const int rc__ = (expr);                                                          \
        if (rc__ != 0) throw std::runtime_error(std::string(#expr) + " -> " + std::to_string(rc__)); \
    } while (0)

class DeviceBuf {
public:
    DeviceBuf() = default;
    DeviceBuf(M40llmCudaContext* ctx, size_t bytes) : ctx_(ctx), bytes_(bytes) {
        if (m40llm_device_malloc(ctx, bytes ? bytes : 4, &p_) != 0) throw std::runtime_error("device_malloc failed");
    }
    DeviceBuf(DeviceBuf&& o) noexcept : ctx_(o.ctx_), p_(o.p_), bytes_(o.bytes_) { o.p_ = nullptr; }
    DeviceBuf& operator=(DeviceBuf&& o) noexcept {
        reset();
        ctx_ = o.ctx_; p_ = o.p_; bytes_ = o.bytes_; o.p_ = nullptr;
        return *this;
    }
    DeviceBuf(const DeviceBuf&) = delete;
    DeviceBuf& operator=(const DeviceBuf&) = delete;
    ~DeviceBuf() { reset(); }
    void reset() { if (p_) m40llm_device_free(ctx_, p_); p_ = nullptr; }
    void* ptr() const { return p_; }
    float* f32(size_t off = 0) const { return static_cast<float*>(p_) + off; }
    uint32_t* u32(size_t off = 0) const { return static_cast<uint32_t*>(p_) + off; }
    size_t bytes() const { return bytes_; }

private:
    M40llmCudaContext* ctx_ = nullptr;
    void* p_ = nullptr;
    size_t bytes_ = 0;
};

// Named f32 scratch buffers sized by row count (src/infer/workspace.rs:60-126).
struct ForwardWorkspace {
    uint32_t rows = 0;
    uint32_t generation = 0;   // bumped whenever the buffers are reallocated: captured graphs hold their addresses
    DeviceBuf xn, q, k, v, ctx_out, y_attn, x1, x1n, gate, up, hid, y_mlp, scratch_a, scratch_b, norm_hidden, logits;
    DeviceBuf argmax_idx, argmax_gap, positions;
    void ensure(M40llmCudaContext* c, const ModelConfig& m, uint32_t want_rows) {
        if (want_rows <= rows) return;
        const size_t D = m.d_model, KV = (size_t)m.kv_heads * m.head_dim, F = m.ffn, R = want_rows;
        xn = DeviceBuf(c, R * D * 4); q = DeviceBuf(c, R * D * 4); k = DeviceBuf(c, R * KV * 4); v = DeviceBuf(c, R * KV * 4);
        ctx_out = DeviceBuf(c, R * D * 4); y_attn = DeviceBuf(c, R * D * 4); x1 = DeviceBuf(c, R * D * 4);
        x1n = DeviceBuf(c, R * D * 4); gate = DeviceBuf(c, R * F * 4); up = DeviceBuf(c, R * F * 4);
        hid = DeviceBuf(c, R * F * 4); y_mlp = DeviceBuf(c, R * D * 4); scratch_a = DeviceBuf(c, R * D * 4);
        scratch_b = DeviceBuf(c, R * D * 4); norm_hidden = DeviceBuf(c, R * D * 4);
        logits = DeviceBuf(c, R * (size_t)m.vocab * 4);
        argmax_idx = DeviceBuf(c, R * 4); argmax_gap = DeviceBuf(c, R * 4); positions = DeviceBuf(c, R * 4 * 2);
        rows = want_rows;
        ++generation;
    }
};

struct PrefillWorkspace {   // activations of a packed prefill: no per-row logits
    uint32_t rows = 0, batch = 0;
    DeviceBuf xn, q, k, v, att, y, x1, gate, up, hid, a, b, tokens, offsets, lens;
    void ensure(M40llmCudaContext* c, const ModelConfig& m, uint32_t want_rows, uint32_t want_batch) {
        if (want_rows > rows) {
            const size_t D = m.d_model, KV = (size_t)m.kv_heads * m.head_dim, F = m.ffn, R = want_rows;
            xn = DeviceBuf(c, R * D * 4); q = DeviceBuf(c, R * D * 4); k = DeviceBuf(c, R * KV * 4); v = DeviceBuf(c, R * KV * 4);
            att = DeviceBuf(c, R * D * 4); y = DeviceBuf(c, R * D * 4); x1 = DeviceBuf(c, R * D * 4);
            gate = DeviceBuf(c, R * F * 4); up = DeviceBuf(c, R * F * 4); hid = DeviceBuf(c, R * F * 4);
            a = DeviceBuf(c, R * D * 4); b = DeviceBuf(c, R * D * 4);
            tokens = DeviceBuf(c, R * 4);
            rows = want_rows;
        }
        if (want_batch > batch) {
            offsets = DeviceBuf(c, (size_t)want_batch * 4); lens = DeviceBuf(c, (size_t)want_batch * 4);
            batch = want_batch;
        }
    }
};

class DecodeModel {
public:
    DecodeModel(M40llmCudaContext* ctx, const ModelConfig& cfg, const LayerWeights* layers, const void* out_norm,
                const void* lm_head, const void* tok_emb, const KvCompressionConfig& kvcfg)
        : ctx_(ctx), cfg_(cfg), layers_(layers, layers + cfg.n_layers), out_norm_(out_norm), lm_head_(lm_head),
          tok_emb_(tok_emb), kvcfg_(kvcfg) {
        if (cfg.d_model != cfg.q_heads * cfg.head_dim)
            throw std::invalid_argument("d_model != query heads * head_dim");     // forward.rs:288-295
        if (cfg.q_heads == 0 || cfg.kv_heads == 0 || cfg.q_heads % cfg.kv_heads != 0)
            throw std::invalid_argument("query heads must be a multiple of kv heads");
        const std::string err = kvcfg.validate_runtime_support(cfg.max_seq_len, cfg.head_dim);
        if (!err.empty()) throw std::invalid_argument(err);
        const uint32_t slots = cfg.max_sequences * cfg.n_layers;   // one slot per (sequence, layer)
        if (kvcfg.uses_compressed_exact_old_backing()) {
            kv_ = m40llm_kvcache_create_compressed(ctx, cfg.max_seq_len, slots, cfg.kv_heads, cfg.head_dim,
                                                   kvcfg.recent_window, kvcfg.block_size, kvcfg.top_blocks,
                                                   kvcfg.representatives, (uint32_t)kvcfg.representative_policy,
                                                   (uint32_t)kvcfg.effective_exact_old_backing());
        } else {
            kv_ = m40llm_kvcache_create(ctx, cfg.max_seq_len, slots, cfg.kv_heads, cfg.head_dim);
        }
        if (!kv_) throw std::runtime_error("KV cache allocation failed");
        ws_.ensure(ctx, cfg, 1);
    }
    ~DecodeModel() {
        drop_graph();
        drop_batch_graph();
        if (kv_) m40llm_kvcache_destroy(kv_);
    }
    DecodeModel(const DecodeModel&) = delete;
    DecodeModel& operator=(const DecodeModel&) = delete;

    const ModelConfig& config() const { return cfg_; }
    M40llmKVCache* kv() const { return kv_; }
    M40llmCudaContext* ctx() const { return ctx_; }
    uint32_t mode() const { return mode_; }
    void set_mode(uint32_t m) { mode_ = m; }
    uint32_t kv_slot(uint32_t seq, uint32_t layer) const {
        if (seq >= cfg_.max_sequences) throw std::out_of_range("sequence id out of range");   // kv.rs:92-107
        return seq * cfg_.n_layers + layer;
    }

    // Grows the activation buffers.  A captured graph has the old buffers' addresses baked in, so both graphs are
    // dropped (after the streams have drained: the old buffers may still be in use) before anything is reallocated.
    void ensure_workspace(uint32_t rows) {
        if (rows <= ws_.rows) return;
        if (ws_.rows != 0) sync_all();
        drop_graph();
        drop_batch_graph();
        ws_.ensure(ctx_, cfg_, rows);
    }

    // ---- single sequence ---------------------------------------------------------------------
    // token embedding row (f16) -> f32 activation (embeddings.rs:64-79)
    void embed(uint32_t token_id, float* d_x) {
        if (token_id >= cfg_.vocab) throw std::out_of_range("token id out of range");
        const char* row = static_cast<const char*>(tok_emb_) + (size_t)token_id * cfg_.d_model * 2;
        M40H_TRY(m40llm_f16_to_f32(ctx_, row, d_x, cfg_.d_model));
    }

    // One decoder layer for the token at position seq_len-1, reference call order.
    void layer_reference(uint32_t layer, uint32_t seq, uint32_t seq_len, const float* d_x, float* d_out) {
        const LayerWeights& w = layers_[layer];
        const uint32_t D = cfg_.d_model, KV = cfg_.kv_heads * cfg_.head_dim, F = cfg_.ffn;
        const uint32_t slot = kv_slot(seq, layer), pos = seq_len - 1;
        const uint32_t PRE = M40LLM_STREAM_PREFILL, DEC = M40LLM_STREAM_DECODE;
        // 1. attention norm (decode stream)
        M40H_TRY(m40llm_rms_norm_f32_weighted_async(ctx_, d_x, w.attn_norm, ws_.xn.ptr(), 1, D, cfg_.rms_eps, cfg_.norm_weight_dtype));
        // 2. QKV projections (prefill stream, blocking)
        M40H_TRY(m40llm_stream_wait_for_stream(ctx_, PRE, DEC));
        M40H_TRY(m40llm_gemm_f32xf16_gguf_f32(ctx_, ws_.xn.ptr(), w.wq, ws_.q.ptr(), 1, (int)D, (int)D));
        M40H_TRY(m40llm_gemm_f32xf16_gguf_f32(ctx_, ws_.xn.ptr(), w.wk, ws_.k.ptr(), 1, (int)KV, (int)D));
        M40H_TRY(m40llm_gemm_f32xf16_gguf_f32(ctx_, ws_.xn.ptr(), w.wv, ws_.v.ptr(), 1, (int)KV, (int)D));
        // 3. optional biases: residual_add per row (forward.rs:124-163)
        if (cfg_.has_qkv_bias) {
            M40H_TRY(m40llm_stream_wait_for_stream(ctx_, DEC, PRE));
            M40H_TRY(m40llm_residual_add_f32_async(ctx_, ws_.q.ptr(), w.bq, ws_.q.ptr(), D));
            M40H_TRY(m40llm_residual_add_f32_async(ctx_, ws_.k.ptr(), w.bk, ws_.k.ptr(), KV));
            M40H_TRY(m40llm_residual_add_f32_async(ctx_, ws_.v.ptr(), w.bv, ws_.v.ptr(), KV));
        }
        // 4. RoPE on Q, 5. fused RoPE-K + f16 append at `pos`
        M40H_TRY(m40llm_stream_wait_for_stream(ctx_, DEC, PRE));
        M40H_TRY(m40llm_rope_f32_inplace_layout_async(ctx_, ws_.q.ptr(), 1, cfg_.q_heads, cfg_.head_dim, pos, cfg_.rope_base,
                                                      cfg_.rope_scale, cfg_.rope_layout));
        M40H_TRY(m40llm_kvcache_append_token_f32_rope_k_at_layout_async(ctx_, kv_, slot, ws_.k.ptr(), ws_.v.ptr(), pos, pos,
                                                                        cfg_.rope_base, cfg_.rope_scale, cfg_.rope_layout));
        // 6. attention, dispatched on the KV-compression mode
        run_attention(layer, slot, seq_len, ws_.q.f32(), ws_.ctx_out.f32());
        // 7. output projection, 8. residual
        M40H_TRY(m40llm_stream_wait_for_stream(ctx_, PRE, DEC));
        M40H_TRY(m40llm_gemm_f32xf16_gguf_f32(ctx_, ws_.ctx_out.ptr(), w.wo, ws_.y_attn.ptr(), 1, (int)D, (int)D));
        M40H_TRY(m40llm_stream_wait_for_stream(ctx_, DEC, PRE));
        M40H_TRY(m40llm_residual_add_f32_async(ctx_, d_x, ws_.y_attn.ptr(), ws_.x1.ptr(), D));
        // 9. FFN norm, 10. gate/up, 11. SwiGLU, 12. down, 13. residual
        M40H_TRY(m40llm_rms_norm_f32_weighted_async(ctx_, ws_.x1.ptr(), w.ffn_norm, ws_.x1n.ptr(), 1, D, cfg_.rms_eps, cfg_.norm_weight_dtype));
        M40H_TRY(m40llm_stream_wait_for_stream(ctx_, PRE, DEC));
        M40H_TRY(m40llm_gemm_f32xf16_gguf_f32(ctx_, ws_.x1n.ptr(), w.wgate, ws_.gate.ptr(), 1, (int)F, (int)D));
        M40H_TRY(m40llm_gemm_f32xf16_gguf_f32(ctx_, ws_.x1n.ptr(), w.wup, ws_.up.ptr(), 1, (int)F, (int)D));
        M40H_TRY(m40llm_stream_wait_for_stream(ctx_, DEC, PRE));
        M40H_TRY(m40llm_swiglu_f32_async(ctx_, ws_.gate.ptr(), ws_.up.ptr(), ws_.hid.ptr(), F));
        M40H_TRY(m40llm_stream_wait_for_stream(ctx_, PRE, DEC));
        M40H_TRY(m40llm_gemm_f32xf16_gguf_f32(ctx_, ws_.hid.ptr(), w.wdown, ws_.y_mlp.ptr(), 1, (int)D, (int)F));
        M40H_TRY(m40llm_stream_wait_for_stream(ctx_, DEC, PRE));
        M40H_TRY(m40llm_residual_add_f32_async(ctx_, ws_.x1.ptr(), ws_.y_mlp.ptr(), d_out, D));
    }

    // One decoder layer, fused entry points, decode stream only.  The position comes from the host
    // (position_dev == nullptr) or from device memory (graph replay).
    void layer_fused(uint32_t layer, uint32_t seq, uint32_t pos, const uint32_t* position_dev, uint32_t max_len_hint,
                     const float* d_x, float* d_out) {
        const LayerWeights& w = layers_[layer];
        const uint32_t D = cfg_.d_model, F = cfg_.ffn;
        const uint32_t slot = kv_slot(seq, layer);
        M40H_TRY(m40llm_ext_fused_norm_qkv_rope_append_async(ctx_, kv_, slot, d_x, w.attn_norm, cfg_.norm_weight_dtype,
                                                             cfg_.rms_eps, w.wq, w.wk, w.wv, w.bq, w.bk, w.bv, cfg_.d_model,
                                                             cfg_.q_heads, pos, position_dev, cfg_.rope_base, cfg_.rope_scale,
                                                             cfg_.rope_layout, ws_.q.ptr()));
        if (position_dev) {
            M40H_TRY(m40llm_ext_attention_last_token_f32_gqa_position_dev_async(ctx_, kv_, slot, ws_.q.ptr(), cfg_.q_heads,
                                                                                position_dev, max_len_hint, ws_.ctx_out.ptr()));
        } else {
            M40H_TRY(m40llm_attention_last_token_f32_gqa_async(ctx_, kv_, slot, ws_.q.ptr(), cfg_.q_heads, pos + 1,
                                                               ws_.ctx_out.ptr()));
        }
        M40H_TRY(m40llm_ext_gemv_residual_f32xf16_async(ctx_, ws_.ctx_out.ptr(), w.wo, d_x, ws_.x1.ptr(), (int)D, (int)D));
        M40H_TRY(m40llm_ext_fused_norm_gate_up_swiglu_async(ctx_, ws_.x1.ptr(), w.ffn_norm, cfg_.norm_weight_dtype, cfg_.rms_eps,
                                                            w.wgate, w.wup, ws_.hid.ptr(), (int)F, (int)D));
        M40H_TRY(m40llm_ext_gemv_residual_f32xf16_async(ctx_, ws_.hid.ptr(), w.wdown, ws_.x1.ptr(), d_out, (int)D, (int)F));
    }

    bool fused_available() const { return !kvcfg_.is_enabled(); }

    // All layers for one token; returns the device pointer that holds the final hidden state.
    const float* forward_token(uint32_t seq, uint32_t pos, uint32_t token_id) {
        if (pos >= cfg_.max_seq_len) throw std::out_of_range("position beyond max_seq_len");
        ensure_workspace(1);
        float* a = ws_.scratch_a.f32();
        float* b = ws_.scratch_b.f32();
        const bool fused = mode_ >= 1 && fused_available();
        // the embedding is written on the prefill stream: decode-stream work of the previous token that still
        // reads or writes the ping-pong buffers must be ordered before it
        M40H_TRY(m40llm_stream_wait_for_stream(ctx_, M40LLM_STREAM_PREFILL, M40LLM_STREAM_DECODE));
        embed(token_id, a);
        for (uint32_t l = 0; l < cfg_.n_layers; ++l) {
            kv_selection::set_attention_context(l, pos);
            if (fused) layer_fused(l, seq, pos, nullptr, 0, a, b);
            else layer_reference(l, seq, pos + 1, a, b);
            std::swap(a, b);
        }
        return a;
    }

    // ---- device-driven greedy loop (modes 1 and 2) ---------------------------------------------
    // state = {position of the last processed token, step, token, capacity, ids[cap], gaps[cap]}
    static constexpr float kGreedyTieGuard = 1e-6f;
    // the guard in force; tests raise it to drive the host-sampled fallback on purpose
    void set_tie_guard(float g) { tie_guard_ = g; }
    float tie_guard() const { return tie_guard_; }
    void ensure_state(uint32_t capacity) {
        if (capacity <= state_cap_) return;
        state_ = DeviceBuf(ctx_, (size_t)(4 + 2 * capacity) * 4);
        state_cap_ = capacity;
        drop_graph();
    }
    void drop_graph() {
        if (graph_) m40llm_cuda_graph_destroy(graph_);
        graph_ = nullptr;
    }
    uint32_t* state_dev() const { return static_cast<uint32_t*>(state_.ptr()); }

    // lm_head on `hidden` -> device greedy pick -> embedding of the picked token -> all layers at
    // the device-side position; leaves the new hidden state in `hidden` (ping-pong safe).
    void enqueue_generation_step(uint32_t seq, float* hidden, float* other, uint32_t max_len_hint) {
        if (!top2_.ptr()) top2_ = DeviceBuf(ctx_, (size_t)3 * kTop2Capacity * 4);
        uint32_t n_blocks = 0;
        M40H_TRY(m40llm_ext_fused_norm_gemv_f32xf16_async(ctx_, hidden, out_norm_, cfg_.norm_weight_dtype, cfg_.rms_eps, lm_head_,
                                                          ws_.logits.ptr(), (int)cfg_.vocab, (int)cfg_.d_model, top2_.ptr(),
                                                          kTop2Capacity, &n_blocks));
        // greedy pick from the per-workgroup candidates + embedding row of the picked token into `hidden`
        M40H_TRY(m40llm_ext_greedy_step_async(ctx_, ws_.logits.ptr(), cfg_.vocab, top2_.ptr(), kTop2Capacity, n_blocks,
                                              state_dev(), tok_emb_, cfg_.d_model, hidden));
        float* a = hidden;
        float* b = other;
        for (uint32_t l = 0; l < cfg_.n_layers; ++l) {
            layer_fused(l, seq, 0, state_dev(), max_len_hint, a, b);
            std::swap(a, b);
        }
        if (a != hidden)   // odd layer count: bring the result back so every step starts from `hidden`
            M40H_TRY(m40llm_memcpy_d2d_async(ctx_, hidden, a, (size_t)cfg_.d_model * 4, M40LLM_STREAM_DECODE));
    }

    uint32_t len_hint_for(uint32_t last_pos_inclusive) const {
        uint32_t h = ((last_pos_inclusive + 1 + 511u) / 512u) * 512u;
        return h > cfg_.max_seq_len ? cfg_.max_seq_len : h;
    }

    // Runs `steps` generation steps starting after `n_done` steps already taken; positions advance on the device.
    void run_generation_steps(uint32_t seq, float* hidden, float* other, uint32_t first_new_pos, uint32_t steps) {
        uint32_t done = 0;
        while (done < steps) {
            const uint32_t pos = first_new_pos + done;
            const uint32_t hint = len_hint_for(pos);
            // steps that share this attention grid size
            uint32_t n = steps - done;
            if (hint < cfg_.max_seq_len && pos + n > hint) n = hint - pos;
            if (mode_ >= 2) {
                if (!graph_ || graph_seq_ != seq || graph_hint_ != hint || graph_hidden_ != hidden ||
                    graph_ws_generation_ != ws_.generation) {
                    drop_graph();
                    M40H_TRY(m40llm_stream_synchronize(ctx_, M40LLM_STREAM_DECODE));
                    M40H_TRY(m40llm_cuda_graph_begin_capture(ctx_, M40LLM_STREAM_DECODE));
                    try {
                        enqueue_generation_step(seq, hidden, other, hint);
                    } catch (...) {
                        m40llm_cuda_graph_cancel_capture(ctx_, M40LLM_STREAM_DECODE);
                        throw;
                    }
                    M40H_TRY(m40llm_cuda_graph_end_capture(ctx_, M40LLM_STREAM_DECODE, &graph_));
                    graph_seq_ = seq; graph_hint_ = hint; graph_hidden_ = hidden; graph_ws_generation_ = ws_.generation;
                }
                for (uint32_t i = 0; i < n; ++i) M40H_TRY(m40llm_cuda_graph_launch(ctx_, graph_, M40LLM_STREAM_DECODE));
            } else {
                for (uint32_t i = 0; i < n; ++i) enqueue_generation_step(seq, hidden, other, hint);
            }
            done += n;
        }
    }

    // Greedy decode on the device path.  Returns false when a top-1/top-2 logit gap fell under the tie guard
    // (the host sampler's tie rule could then differ from a plain argmax): the caller redoes the decode on the
    // host-sampled path.
    bool decode_greedy_device(uint32_t seq, const uint32_t* prompt, uint32_t n_prompt, uint32_t warmup, uint32_t steps,
                              uint32_t start_pos, uint32_t* ids_out, float* gaps_out, double* elapsed_ms) {
        if (n_prompt == 0) throw std::invalid_argument("decode needs at least one prompt token");
        const uint32_t total = warmup + steps;
        if (start_pos + n_prompt + total > cfg_.max_seq_len) throw std::out_of_range("decode would exceed max_seq_len");
        ensure_workspace(1);
        ensure_state(total);
        uint32_t pos = start_pos;
        const float* h = nullptr;
        for (uint32_t i = 0; i < n_prompt; ++i) {
            ids_out[i] = prompt[i];
            h = forward_token(seq, pos++, prompt[i]);
        }
        float* hidden = const_cast<float*>(h);
        float* other = hidden == ws_.scratch_a.f32() ? ws_.scratch_b.f32() : ws_.scratch_a.f32();
        std::vector<uint32_t> st(4 + 2 * (size_t)state_cap_, 0);
        st[0] = pos - 1; st[1] = 0; st[2] = prompt[n_prompt - 1]; st[3] = state_cap_;
        M40H_TRY(m40llm_stream_synchronize(ctx_, M40LLM_STREAM_DECODE));
        M40H_TRY(m40llm_memcpy_h2d(ctx_, state_.ptr(), st.data(), st.size() * 4));
        if (warmup) run_generation_steps(seq, hidden, other, pos, warmup);
        sync_all();
        const auto t0 = std::chrono::steady_clock::now();
        run_generation_steps(seq, hidden, other, pos + warmup, steps);
        sync_all();
        const auto t1 = std::chrono::steady_clock::now();
        if (elapsed_ms) *elapsed_ms = std::chrono::duration<double, std::milli>(t1 - t0).count();
        M40H_TRY(m40llm_memcpy_d2h(ctx_, st.data(), state_.ptr(), st.size() * 4));
        bool ok = true;
        for (uint32_t g = 0; g < total; ++g) {
            ids_out[n_prompt + g] = st[4 + g];
            float gap;
            std::memcpy(&gap, &st[4 + state_cap_ + g], 4);
            if (gaps_out) gaps_out[g] = gap;
            if (!(gap >= tie_guard_)) ok = false;
        }
        return ok;
    }

    // output norm -> lm_head GEMV -> sync -> D2H (logits.rs:57-116)
    void logits_from_hidden(const float* d_hidden, float* host_logits) {
        M40H_TRY(m40llm_stream_wait_for_stream(ctx_, M40LLM_STREAM_PREFILL, M40LLM_STREAM_DECODE));
        M40H_TRY(m40llm_rms_norm_f32_weighted_async(ctx_, d_hidden, out_norm_, ws_.norm_hidden.ptr(), 1, cfg_.d_model,
                                                    cfg_.rms_eps, cfg_.norm_weight_dtype));
        M40H_TRY(m40llm_stream_wait_for_stream(ctx_, M40LLM_STREAM_PREFILL, M40LLM_STREAM_DECODE));
        M40H_TRY(m40llm_gemm_f32xf16_gguf_f32(ctx_, ws_.norm_hidden.ptr(), lm_head_, ws_.logits.ptr(), 1, (int)cfg_.vocab,
                                              (int)cfg_.d_model));
        M40H_TRY(m40llm_stream_synchronize(ctx_, M40LLM_STREAM_PREFILL));
        M40H_TRY(m40llm_memcpy_d2h(ctx_, host_logits, ws_.logits.ptr(), (size_t)cfg_.vocab * 4));
    }

    // ---- packed prefill of several prompts ---------------------------------------------------------
    // All tokens of all prompts as rows of one batch (forward.rs:2153-2600): per layer the projections are GEMMs over
    // every row, RoPE + bias + the f16 KV append run as one launch, and the attention is the packed causal prefill
    // kernel.  Each sequence starts at position 0 of its (cleared) cache slots.  Returns the hidden rows
    // [total rows][d_model] on the device; row offsets are the running sum of `lens`.
    bool packed_prefill_available() const { return !kvcfg_.is_enabled() && (cfg_.head_dim == 64 || cfg_.head_dim == 128); }
    const float* forward_prefill(const uint32_t* seq_ids, const uint32_t* lens, const uint32_t* tokens, uint32_t batch) {
        if (batch == 0) throw std::invalid_argument("batched prefill requires at least one item");
        if (kvcfg_.is_enabled()) throw std::invalid_argument("batched prefill requires the dense KV cache");
        if (cfg_.head_dim != 64 && cfg_.head_dim != 128)
            throw std::invalid_argument("batched prefill attention currently requires head_dim=64 or 128, got " +
                                        std::to_string(cfg_.head_dim));   // forward.rs:2177-2182
        uint64_t total = 0;
        std::vector<uint32_t> offsets(batch);
        for (uint32_t i = 0; i < batch; ++i) {
            if (lens[i] == 0) throw std::invalid_argument("batched prefill item has empty prompt");
            if (lens[i] > cfg_.max_seq_len) throw std::out_of_range("prompt longer than max_seq_len");
            (void)kv_slot(seq_ids[i], cfg_.n_layers - 1);
            offsets[i] = (uint32_t)total;
            total += lens[i];
        }
        if (total > 65535u) throw std::invalid_argument("batched prefill is limited to 65535 rows per call");
        const uint32_t rows = (uint32_t)total;
        for (uint32_t r = 0; r < rows; ++r)
            if (tokens[r] >= cfg_.vocab) throw std::out_of_range("token id out of range");
        pws_.ensure(ctx_, cfg_, rows, batch);
        const uint32_t D = cfg_.d_model, KV = cfg_.kv_heads * cfg_.head_dim, F = cfg_.ffn;
        const uint32_t PRE = M40LLM_STREAM_PREFILL, DEC = M40LLM_STREAM_DECODE;
        M40H_TRY(m40llm_stream_synchronize(ctx_, DEC));   // the tables below are rewritten: nothing may still read them
        M40H_TRY(m40llm_stream_synchronize(ctx_, PRE));
        M40H_TRY(m40llm_memcpy_h2d(ctx_, pws_.tokens.ptr(), tokens, (size_t)rows * 4));
        M40H_TRY(m40llm_memcpy_h2d(ctx_, pws_.offsets.ptr(), offsets.data(), (size_t)batch * 4));
        M40H_TRY(m40llm_memcpy_h2d(ctx_, pws_.lens.ptr(), lens, (size_t)batch * 4));
        float* a = pws_.a.f32();
        float* b = pws_.b.f32();
        M40H_TRY(m40llm_ext_embed_rows_async(ctx_, tok_emb_, pws_.tokens.u32(), rows, cfg_.vocab, D, a));
        M40H_TRY(m40llm_stream_wait_for_stream(ctx_, PRE, DEC));
        std::vector<uint32_t> slots(batch);
        const uint32_t* d_off = pws_.offsets.u32();
        const uint32_t* d_len = pws_.lens.u32();
        // Every launch of a layer goes to the prefill stream: RMSNorm and SwiGLU are produced inside the GEMMs' packing
        // pass and the residual adds inside their last step (m40llm_ext_prefill_gemm_fused_async), so a layer is four
        // projections, the RoPE + append launch and the attention, with no hop between streams.
        for (uint32_t l = 0; l < cfg_.n_layers; ++l) {
            const LayerWeights& w = layers_[l];
            for (uint32_t i = 0; i < batch; ++i) slots[i] = kv_slot(seq_ids[i], l);
            prefill_project(1, a, nullptr, w.attn_norm, pws_.xn.f32(), rows, D, 3, w.wq, D, pws_.q.f32(), w.wk, KV, pws_.k.f32(), w.wv, KV,
                            pws_.v.f32(), nullptr);
            M40H_TRY(m40llm_ext_prefill_rope_append_on_stream_async(ctx_, kv_, pws_.q.ptr(), pws_.k.ptr(), pws_.v.ptr(), batch, slots.data(),
                                                                    lens, nullptr, cfg_.q_heads, cfg_.rope_base, cfg_.rope_scale,
                                                                    cfg_.rope_layout, cfg_.has_qkv_bias ? w.bq : nullptr,
                                                                    cfg_.has_qkv_bias ? w.bk : nullptr, cfg_.has_qkv_bias ? w.bv : nullptr,
                                                                    PRE));
            M40H_TRY(m40llm_ext_attention_prefill_f32_gqa_varlen_host_tables_async(ctx_, pws_.q.ptr(), pws_.k.ptr(), pws_.v.ptr(), d_off, d_off,
                                                                                   d_len, d_len, offsets.data(), lens, lens, batch,
                                                                                   cfg_.q_heads, cfg_.kv_heads, cfg_.head_dim,
                                                                                   pws_.att.ptr()));
            prefill_project(0, pws_.att.f32(), nullptr, nullptr, nullptr, rows, D, 1, w.wo, D, pws_.x1.f32(), nullptr, 0, nullptr, nullptr, 0,
                            nullptr, a);
            prefill_project(1, pws_.x1.f32(), nullptr, w.ffn_norm, pws_.xn.f32(), rows, D, 2, w.wgate, F, pws_.gate.f32(), w.wup, F,
                            pws_.up.f32(), nullptr, 0, nullptr, nullptr);
            prefill_project(2, pws_.gate.f32(), pws_.up.f32(), nullptr, pws_.hid.f32(), rows, F, 1, w.wdown, D, b, nullptr, 0, nullptr, nullptr,
                            0, nullptr, pws_.x1.f32());
            std::swap(a, b);
        }
        M40H_TRY(m40llm_stream_synchronize(ctx_, PRE));
        M40H_TRY(m40llm_stream_synchronize(ctx_, DEC));
        return a;
    }

    // One projection step of the packed prefill on the prefill stream: rows x B_i (up to three matrices), the rows being
    // `x` (kind 0), RMSNorm(x) with norm_w (kind 1) or SwiGLU(x, x2) (kind 2), and C_0 = residual + product when a
    // residual is given (one matrix).  One fused call; where that declines (few rows, odd shapes) the separate launches of
    // forward.rs:2300-2530 with `tmp` holding the normalised / activated rows.
    void prefill_project(uint32_t kind, const float* x, const float* x2, const void* norm_w, float* tmp, uint32_t rows, uint32_t K,
                         int n_mats, const void* B0, uint32_t N0, float* C0, const void* B1, uint32_t N1, float* C1, const void* B2,
                         uint32_t N2, float* C2, const float* residual) {
        const uint32_t PRE = M40LLM_STREAM_PREFILL, DEC = M40LLM_STREAM_DECODE;
        const int rc = m40llm_ext_prefill_gemm_fused_async(ctx_, kind, x, x2, norm_w, cfg_.norm_weight_dtype, cfg_.rms_eps, (int)rows, (int)K,
                                                           n_mats, B0, (int)N0, C0, residual, B1, (int)N1, C1, B2, (int)N2, C2, PRE);
        if (rc == 0) return;
        if (rc != 1) M40H_TRY(rc);
        const float* in = x;
        if (kind != 0) {
            M40H_TRY(m40llm_stream_wait_for_stream(ctx_, DEC, PRE));
            if (kind == 1)
                M40H_TRY(m40llm_rms_norm_f32_weighted_async(ctx_, x, norm_w, tmp, rows, K, cfg_.rms_eps, cfg_.norm_weight_dtype));
            else
                M40H_TRY(m40llm_swiglu_f32_async(ctx_, x, x2, tmp, (size_t)rows * K));
            M40H_TRY(m40llm_stream_wait_for_stream(ctx_, PRE, DEC));
            in = tmp;
        }
        float* out0 = residual ? pws_.y.f32() : C0;
        M40H_TRY(m40llm_ext_gemm_f32xf16_gguf_f32_multi_async(ctx_, in, (int)rows, (int)K, n_mats, B0, (int)N0, out0, B1, (int)N1, C1, B2,
                                                              (int)N2, C2, PRE));
        if (residual) {
            M40H_TRY(m40llm_stream_wait_for_stream(ctx_, DEC, PRE));
            M40H_TRY(m40llm_residual_add_f32_async(ctx_, residual, out0, C0, (size_t)rows * N0));
            M40H_TRY(m40llm_stream_wait_for_stream(ctx_, PRE, DEC));
        }
    }

    // Greedy decode of one sequence: prompt tokens from start_pos, then n_gen sampled tokens
    // (Sampler with top_k = 1).  ids_out holds n_prompt + n_gen ids.
    void decode_greedy(uint32_t seq, const uint32_t* prompt, uint32_t n_prompt, uint32_t n_gen, uint32_t start_pos,
                       uint32_t* ids_out, float* gaps_out) {
        if (mode_ >= 1 && fused_available() && n_gen > 0) {
            // The device loop also runs the layers for the last sampled token (its KV entry is written); ids are the same.
            if (decode_greedy_device(seq, prompt, n_prompt, 0, n_gen, start_pos, ids_out, gaps_out, nullptr)) return;
        }
        Sampler sampler = greedy_sampler(42);
        std::vector<float> logits(cfg_.vocab);
        uint32_t pos = start_pos;
        const float* hidden = nullptr;
        for (uint32_t i = 0; i < n_prompt; ++i) {
            ids_out[i] = prompt[i];
            hidden = forward_token(seq, pos++, prompt[i]);
        }
        for (uint32_t g = 0; g < n_gen; ++g) {
            if (!hidden) throw std::invalid_argument("decode_greedy needs at least one prompt token");
            logits_from_hidden(hidden, logits.data());
            const uint32_t next = (uint32_t)sampler.sample(logits.data(), logits.size());
            if (gaps_out) gaps_out[g] = top2_gap(logits);
            ids_out[n_prompt + g] = next;
            if (g + 1 < n_gen) hidden = forward_token(seq, pos++, next);
        }
    }

    // ---- row-batched variable-length decode (forward.rs:1729-2140) ----------------------------
    // One step for `rows` sequences: token_ids[r] is the input token of sequence seq_ids[r] whose
    // cache currently holds kv_lens[r] tokens; afterwards each holds kv_lens[r] + 1.
    // d_hidden_out receives [rows][d_model].
    const float* forward_batched(const uint32_t* seq_ids, const uint32_t* kv_lens, const uint32_t* token_ids, uint32_t rows) {
        if (rows == 0) throw std::invalid_argument("empty batch");
        if (kvcfg_.is_enabled()) throw std::invalid_argument("batched decode requires the dense KV cache");
        ensure_workspace(rows);
        const uint32_t D = cfg_.d_model, KV = cfg_.kv_heads * cfg_.head_dim, F = cfg_.ffn;
        const uint32_t PRE = M40LLM_STREAM_PREFILL, DEC = M40LLM_STREAM_DECODE;
        float* a = ws_.scratch_a.f32();
        float* b = ws_.scratch_b.f32();
        // decode-stream work of the previous step must not overlap the embedding writes (prefill stream)
        M40H_TRY(m40llm_stream_wait_for_stream(ctx_, PRE, DEC));
        for (uint32_t r = 0; r < rows; ++r) {
            if (kv_lens[r] + 1 > cfg_.max_seq_len) throw std::out_of_range("sequence would exceed max_seq_len");
            embed(token_ids[r], a + (size_t)r * D);
        }
        for (uint32_t l = 0; l < cfg_.n_layers; ++l) {
            const LayerWeights& w = layers_[l];
            // plan for this layer: slot ids and lengths after the append
            std::vector<DecodeRequestState> reqs;
            for (uint32_t r = 0; r < rows; ++r)
                reqs.push_back(DecodeRequestState::active(r, kv_slot(seq_ids[r], l), kv_lens[r] + 1));
            DeviceDecodeBatchPlan plan(ctx_, DecodeBatchPlan::from_requests(reqs));
            M40H_TRY(m40llm_rms_norm_f32_weighted_async(ctx_, a, w.attn_norm, ws_.xn.ptr(), rows, D, cfg_.rms_eps, cfg_.norm_weight_dtype));
            M40H_TRY(m40llm_stream_wait_for_stream(ctx_, PRE, DEC));
            M40H_TRY(m40llm_gemm_f32xf16_gguf_f32(ctx_, ws_.xn.ptr(), w.wq, ws_.q.ptr(), (int)rows, (int)D, (int)D));
            M40H_TRY(m40llm_gemm_f32xf16_gguf_f32(ctx_, ws_.xn.ptr(), w.wk, ws_.k.ptr(), (int)rows, (int)KV, (int)D));
            M40H_TRY(m40llm_gemm_f32xf16_gguf_f32(ctx_, ws_.xn.ptr(), w.wv, ws_.v.ptr(), (int)rows, (int)KV, (int)D));
            M40H_TRY(m40llm_stream_wait_for_stream(ctx_, DEC, PRE));
            for (uint32_t r = 0; r < rows; ++r) {
                float* qr = ws_.q.f32((size_t)r * D);
                float* kr = ws_.k.f32((size_t)r * KV);
                float* vr = ws_.v.f32((size_t)r * KV);
                if (cfg_.has_qkv_bias) {
                    M40H_TRY(m40llm_residual_add_f32_async(ctx_, qr, w.bq, qr, D));
                    M40H_TRY(m40llm_residual_add_f32_async(ctx_, kr, w.bk, kr, KV));
                    M40H_TRY(m40llm_residual_add_f32_async(ctx_, vr, w.bv, vr, KV));
                }
                const uint32_t pos = kv_lens[r];
                M40H_TRY(m40llm_rope_f32_inplace_layout_async(ctx_, qr, 1, cfg_.q_heads, cfg_.head_dim, pos, cfg_.rope_base,
                                                              cfg_.rope_scale, cfg_.rope_layout));
                M40H_TRY(m40llm_kvcache_append_token_f32_rope_k_at_layout_async(ctx_, kv_, kv_slot(seq_ids[r], l), kr, vr, pos, pos,
                                                                                cfg_.rope_base, cfg_.rope_scale, cfg_.rope_layout));
            }
            M40H_TRY(plan.dispatch_attention_async(kv_, ws_.q.ptr(), cfg_.q_heads, ws_.ctx_out.ptr()));
            M40H_TRY(m40llm_stream_wait_for_stream(ctx_, PRE, DEC));
            M40H_TRY(m40llm_gemm_f32xf16_gguf_f32(ctx_, ws_.ctx_out.ptr(), w.wo, ws_.y_attn.ptr(), (int)rows, (int)D, (int)D));
            M40H_TRY(m40llm_stream_wait_for_stream(ctx_, DEC, PRE));
            M40H_TRY(m40llm_residual_add_f32_async(ctx_, a, ws_.y_attn.ptr(), ws_.x1.ptr(), (size_t)rows * D));
            M40H_TRY(m40llm_rms_norm_f32_weighted_async(ctx_, ws_.x1.ptr(), w.ffn_norm, ws_.x1n.ptr(), rows, D, cfg_.rms_eps, cfg_.norm_weight_dtype));
            M40H_TRY(m40llm_stream_wait_for_stream(ctx_, PRE, DEC));
            M40H_TRY(m40llm_gemm_f32xf16_gguf_f32(ctx_, ws_.x1n.ptr(), w.wgate, ws_.gate.ptr(), (int)rows, (int)F, (int)D));
            M40H_TRY(m40llm_gemm_f32xf16_gguf_f32(ctx_, ws_.x1n.ptr(), w.wup, ws_.up.ptr(), (int)rows, (int)F, (int)D));
            M40H_TRY(m40llm_stream_wait_for_stream(ctx_, DEC, PRE));
            M40H_TRY(m40llm_swiglu_f32_async(ctx_, ws_.gate.ptr(), ws_.up.ptr(), ws_.hid.ptr(), (size_t)rows * F));
            M40H_TRY(m40llm_stream_wait_for_stream(ctx_, PRE, DEC));
            M40H_TRY(m40llm_gemm_f32xf16_gguf_f32(ctx_, ws_.hid.ptr(), w.wdown, ws_.y_mlp.ptr(), (int)rows, (int)D, (int)F));
            M40H_TRY(m40llm_stream_wait_for_stream(ctx_, DEC, PRE));
            M40H_TRY(m40llm_residual_add_f32_async(ctx_, ws_.x1.ptr(), ws_.y_mlp.ptr(), b, (size_t)rows * D));
            M40H_TRY(m40llm_stream_synchronize(ctx_, DEC));   // the plan's device arrays are freed at scope end
            std::swap(a, b);
        }
        return a;
    }

    // logits for `rows` hidden rows -> host [rows][vocab]
    void logits_from_hidden_rows(const float* d_hidden, uint32_t rows, float* host_logits) {
        const uint32_t PRE = M40LLM_STREAM_PREFILL, DEC = M40LLM_STREAM_DECODE;
        M40H_TRY(m40llm_stream_wait_for_stream(ctx_, PRE, DEC));
        M40H_TRY(m40llm_rms_norm_f32_weighted_async(ctx_, d_hidden, out_norm_, ws_.norm_hidden.ptr(), rows, cfg_.d_model,
                                                    cfg_.rms_eps, cfg_.norm_weight_dtype));
        M40H_TRY(m40llm_stream_wait_for_stream(ctx_, PRE, DEC));
        M40H_TRY(m40llm_gemm_f32xf16_gguf_f32(ctx_, ws_.norm_hidden.ptr(), lm_head_, ws_.logits.ptr(), (int)rows,
                                              (int)cfg_.vocab, (int)cfg_.d_model));
        M40H_TRY(m40llm_stream_synchronize(ctx_, PRE));
        M40H_TRY(m40llm_memcpy_d2h(ctx_, host_logits, ws_.logits.ptr(), (size_t)rows * cfg_.vocab * 4));
    }

    // ---- device-driven row-batched greedy loop (modes 1 and 2; rows <= 16, dense cache) -------------------------
    // Per step: every layer as five fused calls on the decode stream, output norm + lm_head, then the greedy pick,
    // the length increment and the next embedding on the device.  Nothing is read back until the end.
    bool batched_fused_available(uint32_t rows) const {
        return !kvcfg_.is_enabled() && rows >= 1 && rows <= 16 && cfg_.d_model % 256 == 0 && cfg_.ffn % 256 == 0 &&
               (cfg_.head_dim == 64 || cfg_.head_dim == 128);   // the lengths-on-device attention serves these two
    }
    void batched_layer_fused(uint32_t l, const uint32_t* slots_dev, const uint32_t* lens_dev, uint32_t rows, uint32_t hint,
                             const float* d_x, float* d_out) {
        const LayerWeights& w = layers_[l];
        const uint32_t D = cfg_.d_model, F = cfg_.ffn;
        M40H_TRY(m40llm_ext_batched_norm_qkv_rope_append_async(ctx_, kv_, slots_dev, lens_dev, rows, d_x, w.attn_norm,
                                                               cfg_.norm_weight_dtype, cfg_.rms_eps, w.wq, w.wk, w.wv, w.bq, w.bk,
                                                               w.bv, D, cfg_.q_heads, cfg_.rope_base, cfg_.rope_scale,
                                                               cfg_.rope_layout, ws_.q.ptr()));
        M40H_TRY(m40llm_ext_attention_last_token_f32_gqa_batched_lens_dev_async(ctx_, kv_, slots_dev, lens_dev, 1, rows, hint,
                                                                                ws_.q.ptr(), cfg_.q_heads, ws_.ctx_out.ptr()));
        M40H_TRY(m40llm_ext_batched_gemm_residual_f32xf16_async(ctx_, ws_.ctx_out.ptr(), w.wo, d_x, ws_.x1.ptr(), rows, (int)D, (int)D));
        // d_out is dead until the down projection writes it: the gate + up launch clears it on the side, and the down
        // projection adds its two halves of K into it
        M40H_TRY(m40llm_ext_batched_norm_gate_up_swiglu_clear_async(ctx_, ws_.x1.ptr(), w.ffn_norm, cfg_.norm_weight_dtype,
                                                                    cfg_.rms_eps, w.wgate, w.wup, ws_.hid.ptr(), rows, (int)F,
                                                                    (int)D, d_out, rows * D));
        M40H_TRY(m40llm_ext_batched_gemm_residual_onto_zero_f32xf16_async(ctx_, ws_.hid.ptr(), w.wdown, ws_.x1.ptr(), d_out, rows,
                                                                          (int)D, (int)F));
    }
    void enqueue_batched_step(uint32_t rows, uint32_t hint, float* hidden, float* other) {
        const uint32_t* slots = static_cast<const uint32_t*>(bslots_.ptr());
        uint32_t* lens = static_cast<uint32_t*>(blens_.ptr());
        float* a = hidden;
        float* b = other;
        for (uint32_t l = 0; l < cfg_.n_layers; ++l) {
            batched_layer_fused(l, slots + (size_t)l * rows, lens, rows, hint, a, b);
            std::swap(a, b);
        }
        M40H_TRY(m40llm_ext_batched_norm_gemm_f32xf16_async(ctx_, a, out_norm_, cfg_.norm_weight_dtype, cfg_.rms_eps, lm_head_,
                                                            ws_.logits.ptr(), rows, (int)cfg_.vocab, (int)cfg_.d_model));
        M40H_TRY(m40llm_ext_batched_greedy_step_async(ctx_, ws_.logits.ptr(), rows, cfg_.vocab,
                                                      static_cast<uint32_t*>(bstate_.ptr()), lens,
                                                      static_cast<uint32_t*>(bids_.ptr()), static_cast<float*>(bgaps_.ptr()),
                                                      tok_emb_, cfg_.d_model, hidden));
    }
    // One decode step for `rows` sequences (token r at position kv_lens[r] of sequence seq_ids[r]) with the logits of
    // every row brought to the host: what a serving loop that samples on the host needs per tick
    // (forward_one_token_all_layers_batched_for_sequences + logits_after_batched_forward, src/server.rs:664-711).
    // Fused kernels in groups of up to 16 rows when the host mode allows them, the reference's sequence otherwise.
    // greedy / picks / picked (all null, or all given): rows marked greedy get their token picked on the device (first
    // index of the maximum, as a top_k = 1 sampler picks) when the top-1 / top-2 logit gap clears the tie guard; such
    // rows set picked[r] = 1 and their logits are not copied.  Every other row receives its logits.
    void batched_step_logits(const uint32_t* seq_ids, const uint32_t* kv_lens, const uint32_t* tokens, uint32_t rows,
                             float* host_logits, const uint8_t* greedy = nullptr, uint32_t* picks = nullptr,
                             uint8_t* picked = nullptr) {
        if (picked) std::fill(picked, picked + rows, (uint8_t)0);
        if (rows == 0) throw std::invalid_argument("empty batch");
        for (uint32_t r = 0; r < rows; ++r) {
            if (kv_lens[r] + 1 > cfg_.max_seq_len) throw std::out_of_range("sequence would exceed max_seq_len");
            if (seq_ids[r] >= cfg_.max_sequences) throw std::out_of_range("sequence id out of range");
            if (tokens[r] >= cfg_.vocab) throw std::out_of_range("token id out of range");
        }
        const bool batched_attention = !kvcfg_.is_enabled() && (cfg_.head_dim == 64 || cfg_.head_dim == 128);
        if (rows == 1 || !batched_attention) {
            // one request, or a cache / head size the batched attention does not serve: request by request
            // (scheduler_can_use_batched_attention -> DecodeSchedulerRequest::step, src/server.rs:457-480, 649-661)
            for (uint32_t r = 0; r < rows; ++r) {
                const float* h = forward_token(seq_ids[r], kv_lens[r], tokens[r]);
                logits_from_hidden(h, host_logits + (size_t)r * cfg_.vocab);
            }
            return;
        }
        if (!(mode_ >= 1 && batched_fused_available(rows < 16 ? rows : 16))) {
            const float* hidden = forward_batched(seq_ids, kv_lens, tokens, rows);
            logits_from_hidden_rows(hidden, rows, host_logits);
            return;
        }
        for (uint32_t r0 = 0; r0 < rows; r0 += 16) {
            const uint32_t n = rows - r0 < 16 ? rows - r0 : 16;
            ensure_workspace(n);
            std::vector<uint32_t> table((size_t)cfg_.n_layers * n + 2 * n);   // slots per layer, then lengths, then tokens
            uint32_t longest = 0;
            for (uint32_t l = 0; l < cfg_.n_layers; ++l)
                for (uint32_t r = 0; r < n; ++r) table[(size_t)l * n + r] = kv_slot(seq_ids[r0 + r], l);
            for (uint32_t r = 0; r < n; ++r) {
                table[(size_t)cfg_.n_layers * n + r] = kv_lens[r0 + r];
                table[(size_t)cfg_.n_layers * n + n + r] = tokens[r0 + r];
                longest = kv_lens[r0 + r] > longest ? kv_lens[r0 + r] : longest;
            }
            sync_all();   // the table buffer of the previous group may still be read
            if (tick_table_cap_ < table.size()) {
                tick_table_ = DeviceBuf(ctx_, table.size() * 4);
                tick_table_cap_ = table.size();
            }
            M40H_TRY(m40llm_memcpy_h2d(ctx_, tick_table_.ptr(), table.data(), table.size() * 4));
            const uint32_t* slots = tick_table_.u32();
            const uint32_t* lens = tick_table_.u32((size_t)cfg_.n_layers * n);
            const uint32_t* toks = tick_table_.u32((size_t)cfg_.n_layers * n + n);
            float* a = ws_.scratch_a.f32();
            float* b = ws_.scratch_b.f32();
            M40H_TRY(m40llm_ext_embed_rows_async(ctx_, tok_emb_, toks, n, cfg_.vocab, cfg_.d_model, a));
            const uint32_t hint = len_hint_for(longest);
            for (uint32_t l = 0; l < cfg_.n_layers; ++l) {
                batched_layer_fused(l, slots + (size_t)l * n, lens, n, hint, a, b);
                std::swap(a, b);
            }
            M40H_TRY(m40llm_ext_batched_norm_gemm_f32xf16_async(ctx_, a, out_norm_, cfg_.norm_weight_dtype, cfg_.rms_eps, lm_head_,
                                                                ws_.logits.ptr(), n, (int)cfg_.vocab, (int)cfg_.d_model));
            bool any_greedy = false;
            for (uint32_t r = 0; r < n && greedy && picks && picked; ++r) any_greedy = any_greedy || greedy[r0 + r];
            std::vector<uint32_t> idx(n);
            std::vector<float> gap(n, 0.0f);
            if (any_greedy) {
                M40H_TRY(m40llm_ext_argmax_f32_async(ctx_, ws_.logits.ptr(), n, cfg_.vocab, ws_.argmax_idx.u32(),
                                                     ws_.argmax_gap.f32()));
            }
            M40H_TRY(m40llm_stream_synchronize(ctx_, M40LLM_STREAM_DECODE));
            if (any_greedy) {
                M40H_TRY(m40llm_memcpy_d2h(ctx_, idx.data(), ws_.argmax_idx.ptr(), (size_t)n * 4));
                M40H_TRY(m40llm_memcpy_d2h(ctx_, gap.data(), ws_.argmax_gap.ptr(), (size_t)n * 4));
            }
            for (uint32_t r = 0; r < n; ++r) {
                if (any_greedy && greedy[r0 + r] && gap[r] >= tie_guard_) {
                    picks[r0 + r] = idx[r];
                    picked[r0 + r] = 1;
                } else {
                    M40H_TRY(m40llm_memcpy_d2h(ctx_, host_logits + (size_t)(r0 + r) * cfg_.vocab, ws_.logits.f32((size_t)r * cfg_.vocab),
                                               (size_t)cfg_.vocab * 4));
                }
            }
        }
    }

    // Returns false when a pick was a near-tie (the caller then repeats the decode on the host-sampled path).
    bool decode_batch_device(const uint32_t* seq_ids, const uint32_t* kv_lens, const uint32_t* first_tokens, uint32_t rows,
                             uint32_t warmup, uint32_t steps, uint32_t* ids_out, float* gaps_out, double* elapsed_ms) {
        const uint32_t total = warmup + steps;
        uint32_t max_len = 0;
        for (uint32_t r = 0; r < rows; ++r) {
            if (kv_lens[r] + total > cfg_.max_seq_len) throw std::out_of_range("sequence would exceed max_seq_len");
            if (seq_ids[r] >= cfg_.max_sequences) throw std::out_of_range("sequence id out of range");
            max_len = kv_lens[r] > max_len ? kv_lens[r] : max_len;
        }
        ensure_workspace(rows);
        // device state: slot ids per layer, lengths, per-row step counters, picks and gaps
        std::vector<uint32_t> slots((size_t)cfg_.n_layers * rows);
        for (uint32_t l = 0; l < cfg_.n_layers; ++l)
            for (uint32_t r = 0; r < rows; ++r) slots[(size_t)l * rows + r] = kv_slot(seq_ids[r], l);
        std::vector<uint32_t> state(2 + rows, 0);
        state[1] = total;
        sync_all();
        drop_batch_graph();
        bslots_ = DeviceBuf(ctx_, slots.size() * 4); blens_ = DeviceBuf(ctx_, (size_t)rows * 4);
        bstate_ = DeviceBuf(ctx_, state.size() * 4);
        bids_ = DeviceBuf(ctx_, (size_t)rows * total * 4); bgaps_ = DeviceBuf(ctx_, (size_t)rows * total * 4);
        M40H_TRY(m40llm_memcpy_h2d(ctx_, bslots_.ptr(), slots.data(), slots.size() * 4));
        M40H_TRY(m40llm_memcpy_h2d(ctx_, blens_.ptr(), kv_lens, (size_t)rows * 4));
        M40H_TRY(m40llm_memcpy_h2d(ctx_, bstate_.ptr(), state.data(), state.size() * 4));
        float* hidden = ws_.scratch_a.f32();
        float* other = ws_.scratch_b.f32();
        for (uint32_t r = 0; r < rows; ++r) embed(first_tokens[r], hidden + (size_t)r * cfg_.d_model);
        M40H_TRY(m40llm_stream_wait_for_stream(ctx_, M40LLM_STREAM_DECODE, M40LLM_STREAM_PREFILL));
        auto run = [&](uint32_t first_step, uint32_t n_steps) {
            uint32_t done = 0;
            while (done < n_steps) {
                const uint32_t longest = max_len + first_step + done;       // tokens held by the longest row before the step
                const uint32_t hint = len_hint_for(longest);                // >= longest + 1
                uint32_t n = n_steps - done;
                if (hint < cfg_.max_seq_len && longest + n > hint) n = hint - longest;
                if (mode_ >= 2) {
                    if (!bgraph_ || bgraph_rows_ != rows || bgraph_hint_ != hint || bgraph_ws_generation_ != ws_.generation) {
                        drop_batch_graph();
                        M40H_TRY(m40llm_stream_synchronize(ctx_, M40LLM_STREAM_DECODE));
                        M40H_TRY(m40llm_cuda_graph_begin_capture(ctx_, M40LLM_STREAM_DECODE));
                        try {
                            enqueue_batched_step(rows, hint, hidden, other);
                        } catch (...) {
                            m40llm_cuda_graph_cancel_capture(ctx_, M40LLM_STREAM_DECODE);
                            throw;
                        }
                        M40H_TRY(m40llm_cuda_graph_end_capture(ctx_, M40LLM_STREAM_DECODE, &bgraph_));
                        bgraph_rows_ = rows; bgraph_hint_ = hint; bgraph_ws_generation_ = ws_.generation;
                    }
                    for (uint32_t i = 0; i < n; ++i) M40H_TRY(m40llm_cuda_graph_launch(ctx_, bgraph_, M40LLM_STREAM_DECODE));
                } else {
                    for (uint32_t i = 0; i < n; ++i) enqueue_batched_step(rows, hint, hidden, other);
                }
                done += n;
            }
        };
        if (warmup) run(0, warmup);
        sync_all();
        const auto t0 = std::chrono::steady_clock::now();
        run(warmup, steps);
        sync_all();
        const auto t1 = std::chrono::steady_clock::now();
        if (elapsed_ms) *elapsed_ms = std::chrono::duration<double, std::milli>(t1 - t0).count();
        std::vector<float> gaps((size_t)rows * total);
        M40H_TRY(m40llm_memcpy_d2h(ctx_, ids_out, bids_.ptr(), (size_t)rows * total * 4));
        M40H_TRY(m40llm_memcpy_d2h(ctx_, gaps.data(), bgaps_.ptr(), gaps.size() * 4));
        drop_batch_graph();       // the graph holds pointers into the per-call state buffers
        bool ok = true;
        for (size_t i = 0; i < gaps.size(); ++i) {
            if (gaps_out) gaps_out[i] = gaps[i];
            if (!(gaps[i] >= tie_guard_)) ok = false;
        }
        return ok;
    }
    void drop_batch_graph() {
        if (bgraph_) m40llm_cuda_graph_destroy(bgraph_);
        bgraph_ = nullptr;
    }

    // `steps` greedy steps for a batch of sequences whose caches already hold kv_lens[r] tokens;
    // first_tokens[r] is the input of step 0.  ids_out: [rows][steps], gaps_out (optional) likewise.
    void decode_batch_greedy(const uint32_t* seq_ids, const uint32_t* kv_lens, const uint32_t* first_tokens,
                             uint32_t rows, uint32_t steps, uint32_t* ids_out, float* gaps_out) {
        if (mode_ >= 1 && batched_fused_available(rows)) {
            if (decode_batch_device(seq_ids, kv_lens, first_tokens, rows, 0, steps, ids_out, gaps_out, nullptr)) return;
            // near-tie somewhere: redo on the host-sampled path (same cache rows are rewritten)
        }
        std::vector<uint32_t> lens(kv_lens, kv_lens + rows), toks(first_tokens, first_tokens + rows);
        std::vector<float> logits((size_t)rows * cfg_.vocab);
        std::vector<Sampler> samplers(rows, greedy_sampler(42));
        for (uint32_t s = 0; s < steps; ++s) {
            const float* hidden = forward_batched(seq_ids, lens.data(), toks.data(), rows);
            logits_from_hidden_rows(hidden, rows, logits.data());
            for (uint32_t r = 0; r < rows; ++r) {
                const float* lr = logits.data() + (size_t)r * cfg_.vocab;
                const uint32_t next = (uint32_t)samplers[r].sample(lr, cfg_.vocab);
                ids_out[(size_t)r * steps + s] = next;
                if (gaps_out) gaps_out[(size_t)r * steps + s] = top2_gap(lr, cfg_.vocab);
                toks[r] = next;
                lens[r] += 1;
            }
        }
    }

    // Greedy decode with a timed region: prompt and `warmup` steps untimed, then `steps` steps between two full
    // synchronisations of both streams.
    void decode_timed(uint32_t seq, const uint32_t* prompt, uint32_t n_prompt, uint32_t warmup, uint32_t steps,
                      uint32_t* ids_out, double* elapsed_ms) {
        if (n_prompt == 0) throw std::invalid_argument("decode_timed needs a prompt");
        last_timed_host_fallback_ = false;
        if (mode_ >= 1 && fused_available()) {
            if (decode_greedy_device(seq, prompt, n_prompt, warmup, steps, 0, ids_out, nullptr, elapsed_ms)) return;
            // a device pick was a near tie: the whole run (warm-up and timed steps) is redone through the host sampler,
            // which rewrites the same cache rows; last_timed_host_fallback() tells the caller which path was timed
            last_timed_host_fallback_ = true;
        }
        std::vector<float> logits(cfg_.vocab);
        Sampler sampler = greedy_sampler(42);
        uint32_t pos = 0;
        const float* hidden = nullptr;
        for (uint32_t i = 0; i < n_prompt; ++i) {
            ids_out[i] = prompt[i];
            hidden = forward_token(seq, pos++, prompt[i]);
        }
        auto step = [&](uint32_t out_index) {
            logits_from_hidden(hidden, logits.data());
            const uint32_t next = (uint32_t)sampler.sample(logits.data(), logits.size());
            ids_out[out_index] = next;
            hidden = forward_token(seq, pos++, next);
        };
        for (uint32_t w = 0; w < warmup; ++w) step(n_prompt + w);
        sync_all();
        const auto t0 = std::chrono::steady_clock::now();
        for (uint32_t s = 0; s < steps; ++s) step(n_prompt + warmup + s);
        sync_all();
        const auto t1 = std::chrono::steady_clock::now();
        if (elapsed_ms) *elapsed_ms = std::chrono::duration<double, std::milli>(t1 - t0).count();
    }

    void decode_batch_timed(const uint32_t* seq_ids, const uint32_t* kv_lens, const uint32_t* first_tokens, uint32_t rows,
                            uint32_t warmup, uint32_t steps, uint32_t* ids_out, double* elapsed_ms) {
        last_timed_host_fallback_ = false;
        if (mode_ >= 1 && batched_fused_available(rows)) {
            if (decode_batch_device(seq_ids, kv_lens, first_tokens, rows, warmup, steps, ids_out, nullptr, elapsed_ms)) return;
            last_timed_host_fallback_ = true;   // as in decode_timed: redo everything on the host-sampled path
        }
        std::vector<uint32_t> lens(kv_lens, kv_lens + rows), toks(first_tokens, first_tokens + rows);
        std::vector<float> logits((size_t)rows * cfg_.vocab);
        std::vector<Sampler> samplers(rows, greedy_sampler(42));
        const uint32_t total = warmup + steps;
        auto step = [&](uint32_t s) {
            const float* hidden = forward_batched(seq_ids, lens.data(), toks.data(), rows);
            logits_from_hidden_rows(hidden, rows, logits.data());
            for (uint32_t r = 0; r < rows; ++r) {
                const uint32_t next = (uint32_t)samplers[r].sample(logits.data() + (size_t)r * cfg_.vocab, cfg_.vocab);
                ids_out[(size_t)r * total + s] = next;
                toks[r] = next;
                lens[r] += 1;
            }
        };
        for (uint32_t w = 0; w < warmup; ++w) step(w);
        sync_all();
        const auto t0 = std::chrono::steady_clock::now();
        for (uint32_t s = 0; s < steps; ++s) step(warmup + s);
        sync_all();
        const auto t1 = std::chrono::steady_clock::now();
        if (elapsed_ms) *elapsed_ms = std::chrono::duration<double, std::milli>(t1 - t0).count();
    }

    // true when the last decode_timed / decode_batch_timed call measured the host-sampled path because a device-side
    // greedy pick was a near tie
    bool last_timed_host_fallback() const { return last_timed_host_fallback_; }

    void sync_all() {
        M40H_TRY(m40llm_stream_synchronize(ctx_, M40LLM_STREAM_PREFILL));
        M40H_TRY(m40llm_stream_synchronize(ctx_, M40LLM_STREAM_DECODE));
    }

    static float top2_gap(const float* l, size_t n) {
        float a = -INFINITY, b = -INFINITY;
        for (size_t i = 0; i < n; ++i) {
            if (l[i] > a) { b = a; a = l[i]; }
            else if (l[i] > b) b = l[i];
        }
        return a - b;
    }
    static float top2_gap(const std::vector<float>& l) { return top2_gap(l.data(), l.size()); }

    ForwardWorkspace& workspace() { return ws_; }
    const std::vector<LayerWeights>& layers() const { return layers_; }
    const void* out_norm() const { return out_norm_; }
    const void* lm_head() const { return lm_head_; }
    const void* tok_emb() const { return tok_emb_; }
    const KvCompressionConfig& kv_config() const { return kvcfg_; }

private:
    // Attention dispatch on the KV-compression mode (src/infer/kv.rs:433-765).
    void run_attention(uint32_t layer, uint32_t slot, uint32_t seq_len, const float* d_q, float* d_out) {
        (void)layer;
        if (kvcfg_.mode == KvCompressMode::Off) {
            M40H_TRY(m40llm_attention_last_token_f32_gqa_async(ctx_, kv_, slot, d_q, cfg_.q_heads, seq_len, d_out));
            return;
        }
        if (kvcfg_.mode == KvCompressMode::BlockSelectExact &&
            kvcfg_.effective_exact_old_backing() == KvExactOldBacking::Fp16KQ4V &&
            kvcfg_.effective_exact_old_attention() == KvExactOldAttention::Fp16KQ4VDirect) {
            if (kv_selection::enabled() && seq_len > kvcfg_.recent_window) {
                // telemetry twin: q-head 0 only, host-side re-scoring (kv.rs:523-539)
                uint32_t blocks[2048], start[2048], end[2048], count = 0, total = 0;
                float scores[2048];
                if (m40llm_kvcache_debug_select_old_blocks(ctx_, kv_, slot, d_q, cfg_.q_heads, seq_len, kvcfg_.recent_window,
                                                           kvcfg_.block_size, kvcfg_.top_blocks, blocks, scores, start, end,
                                                           &count, 2048, &total) == 0) {
                    std::vector<KvSelectedBlock> sel;
                    for (uint32_t i = 0; i < count; ++i) sel.push_back({i, blocks[i], scores[i], start[i], end[i]});
                    kv_selection::record_scored_timed(std::move(sel), total, kvcfg_.top_blocks, std::nullopt);
                }
            }
            M40H_TRY(m40llm_attention_last_token_f32_gqa_block_select_exact_fp16_k_q4_v_old_direct_async(
                ctx_, kv_, slot, d_q, cfg_.q_heads, seq_len, kvcfg_.recent_window, kvcfg_.block_size, kvcfg_.top_blocks, d_out));
            return;
        }
        throw std::invalid_argument("KV compression mode not built: only off and block-select-exact/fp16-k-q4-v-direct");
    }

    M40llmCudaContext* ctx_;
    ModelConfig cfg_;
    std::vector<LayerWeights> layers_;
    const void* out_norm_;
    const void* lm_head_;
    const void* tok_emb_;
    KvCompressionConfig kvcfg_;
    M40llmKVCache* kv_ = nullptr;
    ForwardWorkspace ws_;
    PrefillWorkspace pws_;
    uint32_t mode_ = 0;
    bool last_timed_host_fallback_ = false;
    float tie_guard_ = kGreedyTieGuard;
    DeviceBuf state_;
    DeviceBuf top2_;
    static constexpr uint32_t kTop2Capacity = 1u << 16;
    uint32_t state_cap_ = 0;
    DeviceBuf bslots_, blens_, bstate_, bids_, bgaps_;
    DeviceBuf tick_table_;
    size_t tick_table_cap_ = 0;
    M40llmCudaGraphExec* bgraph_ = nullptr;
    uint32_t bgraph_rows_ = 0, bgraph_hint_ = 0, bgraph_ws_generation_ = 0;
    M40llmCudaGraphExec* graph_ = nullptr;
    uint32_t graph_seq_ = 0, graph_hint_ = 0, graph_ws_generation_ = 0;
    float* graph_hidden_ = nullptr;
};

}  // namespace m40host
