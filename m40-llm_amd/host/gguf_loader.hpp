// GGUF ingestion, device side: the data section of a file goes into one device allocation, every tensor is a view
// into it (base + offset, src/infer/tensor_views.rs:86-104), and a decoder model is assembled from the mapped
// tensors.  Follows src/infer/load.rs:10-92 (from_gguf), src/infer/mapping.rs:12-50 (pointer bounds),
// src/infer/embeddings.rs:14-143 (embedding row -> f32) and the decode-time validation of
// src/infer/mapping.rs:495-540.  No tensor is repacked or converted: the bytes the file holds are the bytes the
// kernels read.
#pragma once

#include <memory>
#include <string>
#include <vector>

#include "gguf.hpp"
#include "model.hpp"

namespace m40host {

class GgufWeights {
public:
    // Parses and validates the whole file before anything is allocated on the device.
    GgufWeights(M40llmCudaContext* ctx, const std::string& path) : ctx_(ctx), path_(path) {
        if (!ctx) throw std::invalid_argument("null context");
        {
            gguf::MappedFile file(path);
            model_ = gguf::parse(file.data(), file.size());
        }
        if (model_.data_offset > model_.file_len)
            throw gguf::Error("GGUF data_offset " + std::to_string(model_.data_offset) + " beyond file size " +
                              std::to_string(model_.file_len));
        config_ = gguf::config_from_metadata(model_.metadata, model_.tensors);
        weights_len_ = model_.file_len - model_.data_offset;
        views_ = gguf::build_views(model_.tensors, weights_len_);
        void* base = nullptr;
        const int rc = m40llm_ext_upload_file_range(ctx, path.c_str(), model_.data_offset, weights_len_, &base);
        if (rc != 0) throw std::runtime_error("m40llm_ext_upload_file_range -> " + std::to_string(rc));
        base_ = static_cast<const char*>(base);
    }
    ~GgufWeights() {
        for (void* p : extras_) (void)m40llm_device_free(ctx_, p);
        if (base_) (void)m40llm_device_free(ctx_, const_cast<char*>(base_));
    }
    GgufWeights(const GgufWeights&) = delete;
    GgufWeights& operator=(const GgufWeights&) = delete;

    M40llmCudaContext* ctx() const { return ctx_; }
    const gguf::Model& model() const { return model_; }
    const gguf::Config& config() const { return config_; }
    const gguf::Views& views() const { return views_; }
    uint64_t weights_len() const { return weights_len_; }
    const void* base() const { return base_; }

    // Device address of a tensor, or nullptr when the file has no tensor of that name.
    const void* tensor_ptr(const std::string& name) const {
        const auto it = views_.find(name);
        if (it == views_.end()) return nullptr;
        if (it->second.byte_offset + it->second.nbytes > weights_len_)   // mapping.rs:27-37; build_views has checked it
            throw gguf::Error("tensor '" + name + "' device span exceeds weights length");
        return base_ + it->second.byte_offset;
    }

    // One token's embedding as f32 on the device (embeddings.rs:14-143).  F16 rows are widened and Q8_0 rows
    // dequantised (d * q per 34-byte block) by kernels; the reference does the Q8_0 case on the host.
    void load_token_embedding_f32(uint64_t token_id, void* d_out_f32) const {
        if (!d_out_f32) throw std::invalid_argument("null output");
        const gguf::EmbeddingRow r = gguf::embedding_row(views_, config_, token_id);
        const void* d_row = base_ + r.byte_offset;
        if (r.dtype == gguf::kF16Code) M40H_TRY(m40llm_f16_to_f32(ctx_, d_row, d_out_f32, config_.embedding_length));
        else M40H_TRY(m40llm_q80_to_f32(ctx_, d_row, d_out_f32, config_.embedding_length));
    }

    // A decoder over these weights.  The file must pass the reference's decode-time validation
    // (mapping.rs:495-540: every layer maps, the output projection has the layers' d_model).  Beyond that this
    // build runs F16 projection weights and an F16 embedding table only, needs the final norm tensor, one norm
    // dtype for the whole model and Q/K/V biases in all layers or in none; a layer without a norm tensor gets a
    // weight of ones (forward.rs:317-325 runs the unweighted norm there, which computes the same values).
    // The model reads the weights in place and must be destroyed before this object.
    std::unique_ptr<DecodeModel> make_model(uint32_t max_seq_len, uint32_t max_sequences, const KvCompressionConfig& kvcfg) {
        const gguf::Config& c = config_;
        const auto [d_model, hidden] = gguf::validate_standard_layers(views_, c);
        const gguf::LmHead head = gguf::map_lm_head(views_, c);
        if (head.d_model != d_model)
            throw gguf::Error("lm_head d_model " + std::to_string(head.d_model) + " != layer d_model " + std::to_string(d_model));
        if (head.vocab != c.vocab_size)
            throw gguf::Error("lm_head vocab " + std::to_string(head.vocab) + " != vocab_size " + std::to_string(c.vocab_size));
        const std::string out_norm = gguf::map_output_norm(views_, c);
        if (out_norm.empty()) throw gguf::Error("output norm tensor not found; this build requires output_norm.weight");

        std::vector<gguf::LayerNames> names;
        for (uint32_t l = 0; l < c.block_count; ++l) names.push_back(gguf::map_standard_layer(views_, c, l));
        auto require_f16 = [&](const std::string& name) {
            if (views_.at(name).dtype != gguf::kF16Code)
                throw gguf::Error("tensor " + name + " is " + gguf::dtype_name(views_.at(name).dtype) +
                                  "; this build runs F16 projection and embedding tensors only");
        };
        require_f16(names[0].tok_embeddings);
        uint32_t norm_dtype = views_.at(out_norm).dtype;
        size_t with_bias = 0;
        for (const auto& n : names) {
            for (const std::string* w : {&n.wq, &n.wk, &n.wv, &n.wo, &n.w_gate, &n.w_up, &n.w_down}) require_f16(*w);
            for (const std::string* w : {&n.attn_norm, &n.ffn_norm})
                if (!w->empty() && views_.at(*w).dtype != norm_dtype)
                    throw gguf::Error("norm tensors mix F16 and F32; this build needs one norm dtype per model");
            const int nb = !n.bq.empty() + !n.bk.empty() + !n.bv.empty();
            if (nb != 0 && nb != 3) throw gguf::Error("Q/K/V attention biases must be all present or all absent");
            with_bias += nb == 3;
        }
        if (with_bias != 0 && with_bias != names.size())
            throw gguf::Error("Q/K/V attention biases present in some layers only");

        ModelConfig mc{};
        mc.n_layers = c.block_count;
        mc.d_model = c.embedding_length;
        mc.q_heads = c.attention_head_count;
        mc.kv_heads = c.attention_head_count_kv;
        mc.head_dim = c.attention_key_length;
        mc.ffn = static_cast<uint32_t>(hidden);
        mc.vocab = c.vocab_size;
        mc.rms_eps = c.layer_norm_epsilon;
        mc.rope_base = c.rope_freq_base;
        mc.rope_scale = c.rope_freq_scale;
        mc.rope_layout = c.rope_layout();
        mc.has_qkv_bias = with_bias != 0;
        mc.norm_weight_dtype = norm_dtype == gguf::kF32Code ? 1u : 0u;
        mc.max_seq_len = max_seq_len ? max_seq_len : c.context_length;
        mc.max_sequences = max_sequences ? max_sequences : 1;

        const void* ones = nullptr;
        auto norm_or_ones = [&](const std::string& name) -> const void* {
            if (!name.empty()) return tensor_ptr(name);
            if (!ones) ones = make_ones(mc.d_model, mc.norm_weight_dtype);
            return ones;
        };
        std::vector<LayerWeights> lw(mc.n_layers);
        for (uint32_t l = 0; l < mc.n_layers; ++l) {
            const auto& n = names[l];
            lw[l] = LayerWeights{tensor_ptr(n.wq), tensor_ptr(n.wk), tensor_ptr(n.wv), tensor_ptr(n.wo), tensor_ptr(n.w_gate),
                                 tensor_ptr(n.w_up), tensor_ptr(n.w_down), n.bq.empty() ? nullptr : tensor_ptr(n.bq),
                                 n.bk.empty() ? nullptr : tensor_ptr(n.bk), n.bv.empty() ? nullptr : tensor_ptr(n.bv),
                                 norm_or_ones(n.attn_norm), norm_or_ones(n.ffn_norm)};
        }
        return std::make_unique<DecodeModel>(ctx_, mc, lw.data(), tensor_ptr(out_norm), tensor_ptr(head.name),
                                             tensor_ptr(names[0].tok_embeddings), kvcfg);
    }

private:
    const void* make_ones(uint32_t n, uint32_t f32) {
        void* p = nullptr;
        if (f32) {
            const std::vector<float> host(n, 1.0f);
            M40H_TRY(m40llm_upload_weights(ctx_, host.data(), host.size() * 4, &p));
        } else {
            const std::vector<uint16_t> host(n, 0x3c00);   // 1.0 in f16
            M40H_TRY(m40llm_upload_weights(ctx_, host.data(), host.size() * 2, &p));
        }
        extras_.push_back(p);
        return p;
    }

    M40llmCudaContext* ctx_;
    std::string path_;
    gguf::Model model_;
    gguf::Config config_;
    gguf::Views views_;
    uint64_t weights_len_ = 0;
    const char* base_ = nullptr;
    std::vector<void*> extras_;
};

}  // namespace m40host
