// C entry points of the host layer (see include/m40llm_host.h).
#include "../../include/m40llm_host.h"

#include <cstdio>
#include <cstring>
#include <exception>
#include <string>

#include "decode.hpp"
#include "decode_batch.hpp"
#include "gguf_loader.hpp"
#include "kv_compression.hpp"
#include "kv_selection.hpp"
#include "model.hpp"
#include "sampling.hpp"
#include "scheduler.hpp"

using namespace m40host;

namespace {
thread_local std::string g_last_error;

template <typename F>
auto guarded(F&& f, decltype(f()) on_error) -> decltype(f()) {
    try {
        return f();
    } catch (const std::exception& e) {
        g_last_error = e.what();
    } catch (...) {
        g_last_error = "unknown error";
    }
    return on_error;
}

void put_err(char* err, size_t n, const std::string& msg) {
    if (!err || n == 0) return;
    std::snprintf(err, n, "%s", msg.c_str());
}

KvCompressionConfig to_cpp(const M40HostKvConfig& c) {
    KvCompressionConfig k;
    k.mode = static_cast<KvCompressMode>(c.mode);
    k.recent_window = c.recent_window;
    k.block_size = c.block_size;
    k.top_blocks = c.top_blocks;
    k.representatives = c.representatives;
    k.representative_policy = static_cast<KvRepresentativePolicy>(c.representative_policy);
    k.exact_old_backing = static_cast<KvExactOldBacking>(c.exact_old_backing);
    k.exact_old_attention = static_cast<KvExactOldAttention>(c.exact_old_attention);
    return k;
}
void to_c(const KvCompressionConfig& k, M40HostKvConfig* c) {
    c->mode = (uint32_t)k.mode;
    c->recent_window = k.recent_window;
    c->block_size = k.block_size;
    c->top_blocks = k.top_blocks;
    c->representatives = k.representatives;
    c->representative_policy = (uint32_t)k.representative_policy;
    c->exact_old_backing = (uint32_t)k.exact_old_backing;
    c->exact_old_attention = (uint32_t)k.exact_old_attention;
}

StoppingCriteria make_stopping(int64_t max_tokens, int64_t eos_id, const uint32_t* stop_ids, size_t n_stop, int with_stop_ids) {
    std::optional<size_t> mt;
    if (max_tokens >= 0) mt = (size_t)max_tokens;
    if (with_stop_ids) return StoppingCriteria::with_stop_ids(mt, std::vector<uint32_t>(stop_ids, stop_ids + n_stop));
    std::optional<uint32_t> eos;
    if (eos_id >= 0) eos = (uint32_t)eos_id;
    return StoppingCriteria::make(mt, eos);
}

struct PlanHolder {
    DecodeBatchPlan plan;
};
}  // namespace

struct M40HostModel {
    std::unique_ptr<DecodeModel> m;
};
struct M40HostScheduler {
    std::unique_ptr<DecodeScheduler> s;
};
struct M40HostGguf {
    gguf::Model model;
    std::string json;
};
struct M40HostGgufWeights {
    std::unique_ptr<GgufWeights> w;
};

extern "C" {

const char* m40host_last_error(void) { return g_last_error.c_str(); }

// ---- sampling ----------------------------------------------------------------------------------
void* m40host_sampler_create(float temperature, int64_t top_k, float top_p, uint64_t seed) {
    SamplerConfig c;
    c.temperature = temperature;
    if (top_k >= 0) c.top_k = (size_t)top_k;
    if (top_p > 0.0f) c.top_p = top_p;
    c.seed = seed;
    return new Sampler(c);
}
void* m40host_greedy_sampler(uint64_t seed) { return new Sampler(greedy_sampler(seed)); }
int64_t m40host_sampler_sample(void* s, const float* logits, size_t n) {
    return guarded([&]() -> int64_t { return (int64_t) static_cast<Sampler*>(s)->sample(logits, n); }, -1);
}
int64_t m40host_sampler_sample_greedy(void* s, const float* logits, size_t n) {
    return guarded([&]() -> int64_t { return (int64_t) static_cast<Sampler*>(s)->sample_greedy(logits, n); }, -1);
}
void m40host_sampler_destroy(void* s) { delete static_cast<Sampler*>(s); }

// ---- stopping / decode loop -------------------------------------------------------------------
int m40host_should_stop(int64_t max_tokens, int64_t eos_id, const uint32_t* stop_ids, size_t n_stop, int with_stop_ids,
                        const uint32_t* generated, size_t n_generated) {
    const StoppingCriteria s = make_stopping(max_tokens, eos_id, stop_ids, n_stop, with_stop_ids);
    return s.should_stop(std::vector<uint32_t>(generated, generated + n_generated)) ? 1 : 0;
}

int64_t m40host_decode_loop(const uint32_t* prompt, size_t n_prompt, void* sampler, int64_t max_tokens, int64_t eos_id,
                            const uint32_t* stop_ids, size_t n_stop, int with_stop_ids, size_t vocab,
                            m40host_logits_fn logits_fn, void* user, uint32_t* ids_out, size_t ids_capacity) {
    return guarded(
        [&]() -> int64_t {
            const StoppingCriteria s = make_stopping(max_tokens, eos_id, stop_ids, n_stop, with_stop_ids);
            auto fn = [&](const std::vector<uint32_t>& ids) {
                std::vector<float> logits(vocab);
                if (logits_fn(user, ids.data(), ids.size(), logits.data(), vocab) != 0)
                    throw std::runtime_error("logits callback failed");
                return logits;
            };
            std::vector<uint32_t> ids =
                decode_loop_with(std::vector<uint32_t>(prompt, prompt + n_prompt), *static_cast<Sampler*>(sampler), s, fn);
            if (ids.size() > ids_capacity) throw std::runtime_error("ids_out too small");
            std::memcpy(ids_out, ids.data(), ids.size() * sizeof(uint32_t));
            return (int64_t)ids.size();
        },
        -1);
}

// ---- pool ------------------------------------------------------------------------------------------
void* m40host_pool_create(uint32_t capacity) { return new DecodeSequencePool(capacity); }
void m40host_pool_destroy(void* p) { delete static_cast<DecodeSequencePool*>(p); }
uint32_t m40host_pool_capacity(void* p) { return static_cast<DecodeSequencePool*>(p)->capacity(); }
size_t m40host_pool_available(void* p) { return static_cast<DecodeSequencePool*>(p)->available(); }
void* m40host_pool_try_lease(void* p) {
    auto lease = static_cast<DecodeSequencePool*>(p)->try_lease();
    if (!lease) return nullptr;
    return new DecodeSequenceLease(std::move(*lease));
}
uint32_t m40host_lease_sequence_id(void* l) { return static_cast<DecodeSequenceLease*>(l)->sequence_id(); }
void m40host_lease_release(void* l) { delete static_cast<DecodeSequenceLease*>(l); }

// ---- batch plan ------------------------------------------------------------------------------------
void* m40host_batch_plan_from_requests(const uint64_t* request_ids, const uint32_t* sequence_ids, const uint32_t* kv_lens,
                                       const uint32_t* status, size_t n) {
    return guarded(
        [&]() -> void* {
            std::vector<DecodeRequestState> reqs;
            for (size_t i = 0; i < n; ++i)
                reqs.push_back({request_ids[i], sequence_ids[i], kv_lens[i], static_cast<DecodeRequestStatus>(status[i])});
            return new PlanHolder{DecodeBatchPlan::from_requests(reqs)};
        },
        nullptr);
}
void m40host_batch_plan_destroy(void* p) { delete static_cast<PlanHolder*>(p); }
uint32_t m40host_batch_plan_size(void* p) { return static_cast<PlanHolder*>(p)->plan.batch_size(); }
void m40host_batch_plan_sequence_ids(void* p, uint32_t* out) {
    const auto v = static_cast<PlanHolder*>(p)->plan.sequence_ids();
    std::memcpy(out, v.data(), v.size() * 4);
}
void m40host_batch_plan_sequence_lens(void* p, uint32_t* out) {
    const auto v = static_cast<PlanHolder*>(p)->plan.sequence_lens();
    std::memcpy(out, v.data(), v.size() * 4);
}
uint32_t m40host_batch_plan_total_q_tokens(void* p) { return static_cast<PlanHolder*>(p)->plan.metadata().total_q_tokens(); }
uint32_t m40host_batch_plan_total_kv_tokens(void* p) { return static_cast<PlanHolder*>(p)->plan.metadata().total_kv_tokens(); }
uint64_t m40host_batch_plan_total_attention_cells(void* p) {
    return static_cast<PlanHolder*>(p)->plan.metadata().total_attention_cells();
}
uint32_t m40host_batch_plan_query_len(void* p, size_t i) { return static_cast<PlanHolder*>(p)->plan.metadata().sequences().at(i).query_len; }
int64_t m40host_batch_plan_index_for_request(void* p, uint64_t id) {
    auto r = static_cast<PlanHolder*>(p)->plan.batch_index_for_request(id);
    return r ? (int64_t)*r : -1;
}
int64_t m40host_batch_plan_output_offset_f32(void* p, uint64_t id, uint32_t q_heads, uint32_t head_dim) {
    auto r = static_cast<PlanHolder*>(p)->plan.output_offset_f32(id, q_heads, head_dim);
    return r ? (int64_t)*r : -1;
}
int m40host_batch_plan_dispatch_attention(void* p, M40llmCudaContext* ctx, const M40llmKVCache* kv, const void* d_q,
                                          uint32_t q_heads, void* d_out, int async) {
    return guarded(
        [&]() -> int {
            DeviceDecodeBatchPlan dev(ctx, static_cast<PlanHolder*>(p)->plan);
            int rc = async ? dev.dispatch_attention_async(kv, d_q, q_heads, d_out) : dev.dispatch_attention(kv, d_q, q_heads, d_out);
            // the device arrays must outlive the kernels that read them
            if (rc == 0 && async) rc = m40llm_stream_synchronize(ctx, M40LLM_STREAM_DECODE);
            return rc;
        },
        -100);
}
int m40host_batch_metadata_check(const uint32_t* seq_lens, const uint32_t* kv_lens, const uint32_t* query_lens, size_t n,
                                 uint32_t* total_q, uint32_t* total_kv, uint64_t* cells) {
    return guarded(
        [&]() -> int {
            std::vector<BatchSequence> s;
            for (size_t i = 0; i < n; ++i) s.push_back({seq_lens[i], kv_lens[i], query_lens[i]});
            const BatchMetadata m = BatchMetadata::make(std::move(s));
            if (total_q) *total_q = m.total_q_tokens();
            if (total_kv) *total_kv = m.total_kv_tokens();
            if (cells) *cells = m.total_attention_cells();
            return 0;
        },
        -1);
}

// ---- KV config ---------------------------------------------------------------------------------------
void m40host_kvcfg_default(M40HostKvConfig* out) { to_c(KvCompressionConfig(), out); }
void m40host_kvcfg_dense_reference(M40HostKvConfig* out) { to_c(KvCompressionConfig::dense_reference(), out); }
void m40host_kvcfg_for_mode(uint32_t mode, M40HostKvConfig* out) { to_c(KvCompressionConfig::for_mode(static_cast<KvCompressMode>(mode)), out); }
int m40host_kvcfg_validate(const M40HostKvConfig* cfg, char* err, size_t n) {
    const std::string e = to_cpp(*cfg).validate();
    put_err(err, n, e);
    return e.empty() ? 0 : -1;
}
int m40host_kvcfg_validate_runtime_support(const M40HostKvConfig* cfg, uint32_t max_seq_len, uint32_t head_dim, char* err,
                                           size_t n) {
    const std::string e = to_cpp(*cfg).validate_runtime_support(max_seq_len, head_dim);
    put_err(err, n, e);
    return e.empty() ? 0 : -1;
}
uint32_t m40host_kvcfg_effective_backing(const M40HostKvConfig* cfg) { return (uint32_t)to_cpp(*cfg).effective_exact_old_backing(); }
uint32_t m40host_kvcfg_effective_attention(const M40HostKvConfig* cfg) { return (uint32_t)to_cpp(*cfg).effective_exact_old_attention(); }
void m40host_kvcfg_set_runtime(const M40HostKvConfig* cfg) { set_runtime_config(to_cpp(*cfg)); }
void m40host_kvcfg_get_runtime(M40HostKvConfig* out) { to_c(runtime_config(), out); }
void* m40host_kvcfg_scoped_push(const M40HostKvConfig* cfg) { return new ScopedRuntimeConfig(to_cpp(*cfg)); }
void m40host_kvcfg_scoped_pop(void* g) { delete static_cast<ScopedRuntimeConfig*>(g); }

// ---- selection telemetry ----------------------------------------------------------------------------
int m40host_kvsel_enabled(void) { return kv_selection::enabled() ? 1 : 0; }
void m40host_kvsel_reset(void) { kv_selection::reset(); }
void m40host_kvsel_set_attention_context(int64_t layer, int64_t token) {
    kv_selection::set_attention_context(layer < 0 ? std::nullopt : std::optional<uint32_t>((uint32_t)layer),
                                        token < 0 ? std::nullopt : std::optional<uint32_t>((uint32_t)token));
}
void m40host_kvsel_record(const uint32_t* blocks, size_t n, uint32_t total, uint32_t top) {
    kv_selection::record(std::vector<uint32_t>(blocks, blocks + n), total, top);
}
void m40host_kvsel_record_scored_timed(const uint32_t* blocks, const float* scores, const uint32_t* starts,
                                       const uint32_t* ends, size_t n, uint32_t total, uint32_t top, float elapsed_ms) {
    std::vector<KvSelectedBlock> v;
    for (size_t i = 0; i < n; ++i) v.push_back({(uint32_t)i, blocks[i], scores[i], starts[i], ends[i]});
    kv_selection::record_scored_timed(std::move(v), total, top,
                                      elapsed_ms < 0 ? std::nullopt : std::optional<float>(elapsed_ms));
}
int m40host_kvsel_snapshot(uint32_t* selected_out, size_t capacity, size_t* n_selected, uint32_t* total, uint32_t* top,
                           size_t* n_records) {
    const auto s = kv_selection::snapshot();
    if (!s) return 0;
    const size_t n = std::min(capacity, s->selected_block_indices.size());
    if (selected_out) std::memcpy(selected_out, s->selected_block_indices.data(), n * 4);
    if (n_selected) *n_selected = s->selected_block_indices.size();
    if (total) *total = s->total_old_blocks;
    if (top) *top = s->top_blocks;
    if (n_records) *n_records = s->selection_records.size();
    return 1;
}
int m40host_kvsel_snapshot_record(size_t index, int64_t* layer, int64_t* token, uint32_t* ranks, uint32_t* blocks,
                                  float* scores, uint32_t* starts, uint32_t* ends, size_t capacity, size_t* n,
                                  uint32_t* total, uint32_t* top, float* elapsed_ms) {
    const auto s = kv_selection::snapshot();
    if (!s || index >= s->selection_records.size()) return -1;
    const auto& r = s->selection_records[index];
    if (layer) *layer = r.layer ? (int64_t)*r.layer : -1;
    if (token) *token = r.token ? (int64_t)*r.token : -1;
    const size_t m = std::min(capacity, r.selected_blocks.size());
    for (size_t i = 0; i < m; ++i) {
        if (ranks) ranks[i] = r.selected_blocks[i].rank;
        if (blocks) blocks[i] = r.selected_blocks[i].block_index;
        if (scores) scores[i] = r.selected_blocks[i].score;
        if (starts) starts[i] = r.selected_blocks[i].absolute_start;
        if (ends) ends[i] = r.selected_blocks[i].absolute_end;
    }
    if (n) *n = r.selected_blocks.size();
    if (total) *total = r.total_old_blocks;
    if (top) *top = r.top_blocks;
    if (elapsed_ms) *elapsed_ms = r.selection_elapsed_ms ? *r.selection_elapsed_ms : -1.0f;
    return 0;
}
int m40host_kvsel_should_capture_attention(void) { return kv_selection::should_capture_attention() ? 1 : 0; }
void m40host_kvsel_record_attention(float recent_mass, float selected_old_mass) {
    KvAttentionTelemetrySummary a;
    a.recent.prob_mass = recent_mass;
    a.selected_old_exact.prob_mass = selected_old_mass;
    kv_selection::record_attention(std::move(a));
}
size_t m40host_kvsel_attention_count(void) {
    const auto s = kv_selection::snapshot();
    return s ? s->attentions.size() : 0;
}

// ---- model -------------------------------------------------------------------------------------------
M40HostModel* m40host_model_create(M40llmCudaContext* ctx, const M40HostModelConfig* cfg, const M40HostLayerWeights* layers,
                                   const void* out_norm, const void* lm_head, const void* tok_emb,
                                   const M40HostKvConfig* kv_cfg) {
    return guarded(
        [&]() -> M40HostModel* {
            if (!ctx || !cfg || !layers || !out_norm || !lm_head || !tok_emb) throw std::invalid_argument("null argument");
            ModelConfig c{cfg->n_layers, cfg->d_model, cfg->q_heads, cfg->kv_heads, cfg->head_dim, cfg->ffn, cfg->vocab,
                          cfg->rms_eps, cfg->rope_base, cfg->rope_scale, cfg->rope_layout, cfg->has_qkv_bias,
                          cfg->norm_weight_dtype, cfg->max_seq_len, cfg->max_sequences};
            std::vector<LayerWeights> lw(cfg->n_layers);
            for (uint32_t l = 0; l < cfg->n_layers; ++l) {
                const auto& s = layers[l];
                lw[l] = {s.wq, s.wk, s.wv, s.wo, s.wgate, s.wup, s.wdown, s.bq, s.bk, s.bv, s.attn_norm, s.ffn_norm};
                const int nb = (s.bq != nullptr) + (s.bk != nullptr) + (s.bv != nullptr);
                if (nb != 0 && nb != 3) throw std::invalid_argument("Q/K/V attention biases must be all present or all absent");
                if (cfg->has_qkv_bias && nb != 3) throw std::invalid_argument("has_qkv_bias set but a bias pointer is null");
            }
            const KvCompressionConfig k = kv_cfg ? to_cpp(*kv_cfg) : KvCompressionConfig::dense_reference();
            auto* h = new M40HostModel();
            h->m = std::make_unique<DecodeModel>(ctx, c, lw.data(), out_norm, lm_head, tok_emb, k);
            return h;
        },
        nullptr);
}
void m40host_model_destroy(M40HostModel* m) { delete m; }
M40llmKVCache* m40host_model_kv(M40HostModel* m) { return m->m->kv(); }
uint32_t m40host_model_kv_slot(M40HostModel* m, uint32_t seq, uint32_t layer) {
    return guarded([&]() -> uint32_t { return m->m->kv_slot(seq, layer); }, 0xffffffffu);
}
int m40host_model_set_mode(M40HostModel* m, uint32_t mode) {
    if (mode > 2) return -1;
    m->m->set_mode(mode);
    return 0;
}
int m40host_model_forward_token(M40HostModel* m, uint32_t seq, uint32_t pos, uint32_t token, float* hidden_host,
                                float* logits_host) {
    return guarded(
        [&]() -> int {
            DecodeModel& d = *m->m;
            const float* h = d.forward_token(seq, pos, token);
            if (hidden_host) {
                M40H_TRY(m40llm_stream_synchronize(d.ctx(), M40LLM_STREAM_DECODE));
                M40H_TRY(m40llm_memcpy_d2h(d.ctx(), hidden_host, h, (size_t)d.config().d_model * 4));
            }
            if (logits_host) d.logits_from_hidden(h, logits_host);
            return 0;
        },
        -100);
}
int m40host_model_decode_greedy(M40HostModel* m, uint32_t seq, const uint32_t* prompt, uint32_t n_prompt, uint32_t n_gen,
                                uint32_t start_pos, uint32_t* ids_out, float* gaps_out) {
    return guarded([&]() -> int { m->m->decode_greedy(seq, prompt, n_prompt, n_gen, start_pos, ids_out, gaps_out); return 0; }, -100);
}
int m40host_model_decode_timed(M40HostModel* m, uint32_t seq, const uint32_t* prompt, uint32_t n_prompt, uint32_t warmup,
                               uint32_t steps, uint32_t* ids_out, double* elapsed_ms) {
    return guarded([&]() -> int { m->m->decode_timed(seq, prompt, n_prompt, warmup, steps, ids_out, elapsed_ms); return 0; }, -100);
}
int m40host_model_decode_batch_timed(M40HostModel* m, const uint32_t* seq_ids, const uint32_t* kv_lens,
                                     const uint32_t* first_tokens, uint32_t rows, uint32_t warmup, uint32_t steps,
                                     uint32_t* ids_out, double* elapsed_ms) {
    return guarded(
        [&]() -> int {
            m->m->decode_batch_timed(seq_ids, kv_lens, first_tokens, rows, warmup, steps, ids_out, elapsed_ms);
            return 0;
        },
        -100);
}
int m40host_model_last_timed_host_fallback(M40HostModel* m) { return m && m->m->last_timed_host_fallback() ? 1 : 0; }
int m40host_model_set_tie_guard(M40HostModel* m, float guard) {
    if (!m) return -1;
    m->m->set_tie_guard(guard);
    return 0;
}
int m40host_model_forward_batched(M40HostModel* m, const uint32_t* seq_ids, const uint32_t* kv_lens, const uint32_t* tokens,
                                  uint32_t rows, float* hidden_host, float* logits_host) {
    return guarded(
        [&]() -> int {
            DecodeModel& d = *m->m;
            const float* h = d.forward_batched(seq_ids, kv_lens, tokens, rows);
            if (hidden_host) {
                M40H_TRY(m40llm_stream_synchronize(d.ctx(), M40LLM_STREAM_DECODE));
                M40H_TRY(m40llm_memcpy_d2h(d.ctx(), hidden_host, h, (size_t)rows * d.config().d_model * 4));
            }
            if (logits_host) d.logits_from_hidden_rows(h, rows, logits_host);
            return 0;
        },
        -100);
}
int m40host_model_decode_batch_greedy(M40HostModel* m, const uint32_t* seq_ids, const uint32_t* kv_lens,
                                      const uint32_t* first_tokens, uint32_t rows, uint32_t steps, uint32_t* ids_out,
                                      float* gaps_out) {
    return guarded(
        [&]() -> int { m->m->decode_batch_greedy(seq_ids, kv_lens, first_tokens, rows, steps, ids_out, gaps_out); return 0; }, -100);
}

int m40host_model_forward_prefill(M40HostModel* m, const uint32_t* seq_ids, const uint32_t* lens, const uint32_t* tokens,
                                  uint32_t batch, float* hidden_last_host, float* logits_last_host) {
    return guarded(
        [&]() -> int {
            if (!m || !seq_ids || !lens || !tokens) throw std::invalid_argument("null argument");
            DecodeModel& d = *m->m;
            const float* h = d.forward_prefill(seq_ids, lens, tokens, batch);
            const size_t D = d.config().d_model, V = d.config().vocab;
            size_t row = 0;
            for (uint32_t i = 0; i < batch; ++i) {
                row += lens[i];
                const float* last = h + (row - 1) * D;
                if (hidden_last_host) M40H_TRY(m40llm_memcpy_d2h(d.ctx(), hidden_last_host + i * D, last, D * 4));
                if (logits_last_host) d.logits_from_hidden(last, logits_last_host + i * V);
            }
            return 0;
        },
        -100);
}

// ---- GGUF ingestion ------------------------------------------------------------------------------------
M40HostGguf* m40host_gguf_open(const char* path) {
    return guarded(
        [&]() -> M40HostGguf* {
            if (!path) throw std::invalid_argument("null path");
            gguf::MappedFile file(path);
            auto g = std::make_unique<M40HostGguf>();
            g->model = gguf::parse(file.data(), file.size());
            g->json = gguf::describe_json(g->model);
            return g.release();
        },
        nullptr);
}
M40HostGguf* m40host_gguf_parse(const void* bytes, size_t n) {
    return guarded(
        [&]() -> M40HostGguf* {
            if (!bytes && n) throw std::invalid_argument("null bytes");
            auto g = std::make_unique<M40HostGguf>();
            g->model = gguf::parse(static_cast<const uint8_t*>(bytes), n);
            g->json = gguf::describe_json(g->model);
            return g.release();
        },
        nullptr);
}
void m40host_gguf_close(M40HostGguf* g) { delete g; }
size_t m40host_gguf_describe_json(const M40HostGguf* g, char* buf, size_t capacity) {
    if (!g) return 0;
    if (buf && capacity) {
        const size_t n = g->json.size() < capacity - 1 ? g->json.size() : capacity - 1;
        std::memcpy(buf, g->json.data(), n);
        buf[n] = 0;
    }
    return g->json.size() + 1;
}
int m40host_gguf_embedding_row(const M40HostGguf* g, uint64_t token_id, uint64_t* byte_offset, uint64_t* row_bytes,
                               uint32_t* dtype_raw) {
    return guarded(
        [&]() -> int {
            if (!g) throw std::invalid_argument("null handle");
            const gguf::Config cfg = gguf::config_from_metadata(g->model.metadata, g->model.tensors);
            if (g->model.data_offset > g->model.file_len) throw gguf::Error("GGUF data_offset beyond file size");
            const gguf::Views views = gguf::build_views(g->model.tensors, g->model.file_len - g->model.data_offset);
            const gguf::EmbeddingRow r = gguf::embedding_row(views, cfg, token_id);
            if (byte_offset) *byte_offset = r.byte_offset;
            if (row_bytes) *row_bytes = r.row_bytes;
            if (dtype_raw) *dtype_raw = r.dtype;
            return 0;
        },
        -1);
}

M40HostGgufWeights* m40host_gguf_load(M40llmCudaContext* ctx, const char* path) {
    return guarded(
        [&]() -> M40HostGgufWeights* {
            if (!ctx || !path) throw std::invalid_argument("null argument");
            auto h = std::make_unique<M40HostGgufWeights>();
            h->w = std::make_unique<GgufWeights>(ctx, path);
            return h.release();
        },
        nullptr);
}
void m40host_gguf_weights_free(M40HostGgufWeights* w) { delete w; }
uint64_t m40host_gguf_weights_len(const M40HostGgufWeights* w) { return w ? w->w->weights_len() : 0; }
const void* m40host_gguf_weights_base(const M40HostGgufWeights* w) { return w ? w->w->base() : nullptr; }
const void* m40host_gguf_tensor_ptr(const M40HostGgufWeights* w, const char* name) {
    return guarded(
        [&]() -> const void* {
            if (!w || !name) throw std::invalid_argument("null argument");
            const void* p = w->w->tensor_ptr(name);
            if (!p) throw gguf::Error(std::string("no tensor named '") + name + "'");
            return p;
        },
        nullptr);
}
int m40host_gguf_load_token_embedding_f32(const M40HostGgufWeights* w, uint64_t token_id, void* d_out_f32) {
    return guarded(
        [&]() -> int {
            if (!w) throw std::invalid_argument("null handle");
            w->w->load_token_embedding_f32(token_id, d_out_f32);
            return 0;
        },
        -1);
}
M40HostModel* m40host_model_from_gguf(M40HostGgufWeights* w, uint32_t max_seq_len, uint32_t max_sequences,
                                      const M40HostKvConfig* kv_cfg) {
    return guarded(
        [&]() -> M40HostModel* {
            if (!w) throw std::invalid_argument("null handle");
            const KvCompressionConfig k = kv_cfg ? to_cpp(*kv_cfg) : KvCompressionConfig::dense_reference();
            auto h = std::make_unique<M40HostModel>();
            h->m = w->w->make_model(max_seq_len, max_sequences, k);
            return h.release();
        },
        nullptr);
}

// ---- continuous-batching decode scheduler -----------------------------------------------------------------
M40HostScheduler* m40host_scheduler_create_for_model(M40HostModel* model, uint32_t sequence_slots) {
    return guarded(
        [&]() -> M40HostScheduler* {
            if (!model) throw std::invalid_argument("null model");
            DecodeModel* d = model->m.get();
            const ModelConfig& c = d->config();
            if (sequence_slots == 0 || sequence_slots > c.max_sequences) sequence_slots = c.max_sequences;
            SchedulerEngine e;
            e.vocab = c.vocab;
            e.max_seq_len = c.max_seq_len;
            e.prefill = [d](const std::vector<SchedulerPrefillItem>& items, float* logits_out) {
                const ModelConfig& cfg = d->config();
                if (d->packed_prefill_available()) {
                    for (size_t i0 = 0; i0 < items.size();) {   // at most 64 prompts and 65535 rows per packed call
                        std::vector<uint32_t> seqs, lens, toks;
                        size_t i = i0;
                        while (i < items.size() && seqs.size() < 64 && toks.size() + items[i].len <= 65535u) {
                            seqs.push_back(items[i].sequence_id);
                            lens.push_back(items[i].len);
                            toks.insert(toks.end(), items[i].tokens, items[i].tokens + items[i].len);
                            ++i;
                        }
                        if (i == i0) throw std::invalid_argument("prompt longer than one packed prefill call takes");
                        const float* h = d->forward_prefill(seqs.data(), lens.data(), toks.data(), (uint32_t)seqs.size());
                        size_t row = 0;
                        for (size_t j = 0; j < seqs.size(); ++j) {
                            row += lens[j];
                            d->logits_from_hidden(h + (row - 1) * cfg.d_model, logits_out + (i0 + j) * (size_t)cfg.vocab);
                        }
                        i0 = i;
                    }
                } else {   // token by token (DecodeSchedulerRequest::step, server.rs:300-329)
                    for (size_t i = 0; i < items.size(); ++i) {
                        const float* h = nullptr;
                        for (uint32_t p = 0; p < items[i].len; ++p) h = d->forward_token(items[i].sequence_id, p, items[i].tokens[p]);
                        d->logits_from_hidden(h, logits_out + i * (size_t)cfg.vocab);
                    }
                }
            };
            e.decode = [d](const std::vector<SchedulerDecodeItem>& items, float* logits_out) {
                std::vector<uint32_t> seqs, lens, toks;
                for (const auto& it : items) {
                    seqs.push_back(it.sequence_id);
                    lens.push_back(it.kv_len);
                    toks.push_back(it.token);
                }
                d->batched_step_logits(seqs.data(), lens.data(), toks.data(), (uint32_t)items.size(), logits_out);
            };
            e.decode_pick = [d](const std::vector<SchedulerDecodeItem>& items, const uint8_t* greedy, float* logits_out,
                                uint32_t* picks_out, uint8_t* picked_out) {
                std::vector<uint32_t> seqs, lens, toks;
                for (const auto& it : items) {
                    seqs.push_back(it.sequence_id);
                    lens.push_back(it.kv_len);
                    toks.push_back(it.token);
                }
                d->batched_step_logits(seqs.data(), lens.data(), toks.data(), (uint32_t)items.size(), logits_out, greedy, picks_out,
                                       picked_out);
            };
            auto h = std::make_unique<M40HostScheduler>();
            h->s = std::make_unique<DecodeScheduler>(std::move(e), sequence_slots);
            return h.release();
        },
        nullptr);
}
M40HostScheduler* m40host_scheduler_create_with_engine(uint32_t vocab, uint32_t max_seq_len, uint32_t sequence_slots,
                                                       m40host_sched_prefill_fn prefill_fn, m40host_sched_decode_fn decode_fn,
                                                       void* user) {
    return guarded(
        [&]() -> M40HostScheduler* {
            if (!prefill_fn || !decode_fn) throw std::invalid_argument("null engine callback");
            SchedulerEngine e;
            e.vocab = vocab;
            e.max_seq_len = max_seq_len;
            e.prefill = [prefill_fn, user](const std::vector<SchedulerPrefillItem>& items, float* logits_out) {
                std::vector<uint32_t> seqs, lens, toks;
                for (const auto& it : items) {
                    seqs.push_back(it.sequence_id);
                    lens.push_back(it.len);
                    toks.insert(toks.end(), it.tokens, it.tokens + it.len);
                }
                if (prefill_fn(user, seqs.data(), lens.data(), toks.data(), (uint32_t)items.size(), logits_out) != 0)
                    throw std::runtime_error("prefill callback reported an error");
            };
            e.decode = [decode_fn, user](const std::vector<SchedulerDecodeItem>& items, float* logits_out) {
                std::vector<uint32_t> seqs, lens, toks;
                for (const auto& it : items) {
                    seqs.push_back(it.sequence_id);
                    lens.push_back(it.kv_len);
                    toks.push_back(it.token);
                }
                if (decode_fn(user, seqs.data(), lens.data(), toks.data(), (uint32_t)items.size(), logits_out) != 0)
                    throw std::runtime_error("decode callback reported an error");
            };
            auto h = std::make_unique<M40HostScheduler>();
            h->s = std::make_unique<DecodeScheduler>(std::move(e), sequence_slots);
            return h.release();
        },
        nullptr);
}
void m40host_scheduler_destroy(M40HostScheduler* s) { delete s; }
int64_t m40host_scheduler_submit(M40HostScheduler* s, const uint32_t* prompt, size_t n_prompt, int64_t max_tokens,
                                 const uint32_t* stop_ids, size_t n_stop, float temperature, int64_t top_k, float top_p,
                                 uint64_t seed) {
    return guarded(
        [&]() -> int64_t {
            if (!s) throw std::invalid_argument("null scheduler");
            SamplerConfig c;
            c.temperature = temperature;
            if (top_k >= 0) c.top_k = (size_t)top_k;
            if (top_p > 0.0f) c.top_p = top_p;
            c.seed = seed;
            std::vector<uint32_t> stops(stop_ids, stop_ids + (stop_ids ? n_stop : 0));
            return (int64_t)s->s->submit(prompt, n_prompt, max_tokens >= 0 ? std::optional<size_t>((size_t)max_tokens) : std::nullopt,
                                         std::move(stops), c);
        },
        -1);
}
int m40host_scheduler_cancel(M40HostScheduler* s, uint64_t request_id) { return s && s->s->cancel(request_id) ? 1 : 0; }
int m40host_scheduler_tick(M40HostScheduler* s, M40HostTickReport* report) {
    return guarded(
        [&]() -> int {
            if (!s) throw std::invalid_argument("null scheduler");
            const SchedulerTickReport r = s->s->tick();
            if (report) *report = M40HostTickReport{r.prefill_rows, r.prefill_tokens, r.decode_rows, r.completed, r.cancelled, r.failed};
            return 0;
        },
        -1);
}
uint32_t m40host_scheduler_state(M40HostScheduler* s, uint64_t request_id) { return s ? (uint32_t)s->s->state(request_id) : 0; }
uint32_t m40host_scheduler_sequence_of(M40HostScheduler* s, uint64_t request_id) { return s ? s->s->sequence_of(request_id) : 0xffffffffu; }
size_t m40host_scheduler_active(M40HostScheduler* s) { return s ? s->s->active() : 0; }
size_t m40host_scheduler_available_slots(M40HostScheduler* s) { return s ? s->s->available_slots() : 0; }
int64_t m40host_scheduler_generated(M40HostScheduler* s, uint64_t request_id, uint32_t* ids_out, size_t capacity) {
    if (!s) return -1;
    const std::vector<uint32_t> g = s->s->generated(request_id);
    for (size_t i = 0; i < g.size() && i < capacity; ++i) ids_out[i] = g[i];
    return (int64_t)g.size();
}
size_t m40host_scheduler_error(M40HostScheduler* s, uint64_t request_id, char* buf, size_t capacity) {
    if (!s) return 0;
    const std::string e = s->s->error_of(request_id);
    put_err(buf, capacity, e);
    return e.size();
}

}  // extern "C"
