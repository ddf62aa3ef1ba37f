// KV-compression configuration: modes, exact-old backing / attention enums, validation and the
// process-wide + scoped (thread-local) runtime configuration.  Mirrors src/kv_compression.rs.
#pragma once

#include <cstdint>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <optional>
#include <string>

namespace m40host {

enum class KvCompressMode : uint32_t { Off = 0, DenseRecentOnly, BlockSelectExact, RecentOnly, BlockSummary, BlockSelectLossy };
enum class KvRepresentativePolicy : uint32_t { Last = 0, Stride = 1 };       // as_ffi(): 0 / 1
enum class KvExactOldBacking : uint32_t { Dense = 0, Q8 = 1, Fp16KQ4V = 2 };  // as_ffi(): 0 / 1 / 2 (src/cuda.rs:849-855)
enum class KvExactOldAttention : uint32_t { Staged = 0, Q8Direct = 1, Fp16KQ4VDirect = 2 };

inline const char* backing_str(KvExactOldBacking b) {
    switch (b) {
        case KvExactOldBacking::Dense: return "dense";
        case KvExactOldBacking::Q8: return "q8";
        default: return "fp16-k-q4-v";
    }
}
inline const char* attention_str(KvExactOldAttention a) {
    switch (a) {
        case KvExactOldAttention::Staged: return "staged";
        case KvExactOldAttention::Q8Direct: return "q8-direct";
        default: return "fp16-k-q4-v-direct";
    }
}
inline const char* mode_debug_str(KvCompressMode m) {
    switch (m) {
        case KvCompressMode::Off: return "Off";
        case KvCompressMode::DenseRecentOnly: return "DenseRecentOnly";
        case KvCompressMode::BlockSelectExact: return "BlockSelectExact";
        case KvCompressMode::RecentOnly: return "RecentOnly";
        case KvCompressMode::BlockSummary: return "BlockSummary";
        default: return "BlockSelectLossy";
    }
}

struct KvCompressionConfig {
    // defaults of src/kv_compression.rs:85-98
    KvCompressMode mode = KvCompressMode::BlockSelectExact;
    uint32_t recent_window = 1024;
    uint32_t block_size = 32;
    uint32_t top_blocks = 8;
    uint32_t representatives = 0;
    KvRepresentativePolicy representative_policy = KvRepresentativePolicy::Last;
    KvExactOldBacking exact_old_backing = KvExactOldBacking::Fp16KQ4V;
    KvExactOldAttention exact_old_attention = KvExactOldAttention::Fp16KQ4VDirect;

    bool operator==(const KvCompressionConfig& o) const {
        return mode == o.mode && recent_window == o.recent_window && block_size == o.block_size &&
               top_blocks == o.top_blocks && representatives == o.representatives &&
               representative_policy == o.representative_policy && exact_old_backing == o.exact_old_backing &&
               exact_old_attention == o.exact_old_attention;
    }

    static KvCompressionConfig dense_reference() {
        KvCompressionConfig c;
        c.mode = KvCompressMode::Off;
        c.exact_old_backing = KvExactOldBacking::Dense;
        c.exact_old_attention = KvExactOldAttention::Staged;
        return c;
    }
    static KvCompressionConfig for_mode(KvCompressMode mode) {
        KvCompressionConfig c = mode == KvCompressMode::BlockSelectExact ? KvCompressionConfig() : dense_reference();
        c.mode = mode;
        return c;
    }
    bool is_enabled() const { return mode != KvCompressMode::Off; }

    KvExactOldBacking effective_exact_old_backing() const {
        if (exact_old_backing != KvExactOldBacking::Dense) return exact_old_backing;
        const char* v = std::getenv("M40LLM_KV_EXACT_OLD_BACKING");
        if (v && (!std::strcmp(v, "q8") || !std::strcmp(v, "Q8"))) return KvExactOldBacking::Q8;
        if (v && (!std::strcmp(v, "fp16-k-q4-v") || !std::strcmp(v, "FP16-K-Q4-V"))) return KvExactOldBacking::Fp16KQ4V;
        return KvExactOldBacking::Dense;
    }
    KvExactOldAttention effective_exact_old_attention() const {
        if (exact_old_attention != KvExactOldAttention::Staged) return exact_old_attention;
        const char* v = std::getenv("M40LLM_KV_EXACT_OLD_ATTENTION");
        if (v && (!std::strcmp(v, "q8-direct") || !std::strcmp(v, "Q8-DIRECT") || !std::strcmp(v, "direct-q8")))
            return KvExactOldAttention::Q8Direct;
        if (v && (!std::strcmp(v, "fp16-k-q4-v-direct") || !std::strcmp(v, "FP16-K-Q4-V-DIRECT") ||
                  !std::strcmp(v, "direct-fp16-k-q4-v")))
            return KvExactOldAttention::Fp16KQ4VDirect;
        return KvExactOldAttention::Staged;
    }
    bool uses_compressed_exact_old_backing() const {
        return mode == KvCompressMode::BlockSelectExact && effective_exact_old_backing() != KvExactOldBacking::Dense;
    }

    // Returns an empty string when valid, else the reference's error text.
    std::string validate() const {
        if (recent_window == 0) return "kv_recent_window must be > 0";
        if (block_size == 0) return "kv_compress_block must be > 0";
        if ((mode == KvCompressMode::BlockSelectExact || mode == KvCompressMode::BlockSelectLossy) && top_blocks == 0)
            return "kv_compress_top_blocks must be > 0 for block-select modes";
        const KvExactOldBacking backing =
            mode == KvCompressMode::BlockSelectExact ? effective_exact_old_backing() : exact_old_backing;
        const KvExactOldAttention attention =
            mode == KvCompressMode::BlockSelectExact ? effective_exact_old_attention() : exact_old_attention;
        if (backing != KvExactOldBacking::Dense && mode != KvCompressMode::BlockSelectExact)
            return std::string("kv_exact_old_backing=") + backing_str(backing) +
                   " requires kv_compress_mode=block-select-exact";
        if (attention == KvExactOldAttention::Q8Direct && backing != KvExactOldBacking::Q8)
            return "kv_exact_old_attention=q8-direct requires kv_exact_old_backing=q8";
        if (attention == KvExactOldAttention::Fp16KQ4VDirect && backing != KvExactOldBacking::Fp16KQ4V)
            return "kv_exact_old_attention=fp16-k-q4-v-direct requires kv_exact_old_backing=fp16-k-q4-v";
        return "";
    }

    std::string validate_runtime_support(uint32_t max_seq_len, uint32_t head_dim) const {
        std::string e = validate();
        if (!e.empty()) return e;
        if (mode == KvCompressMode::Off) return "";
        if (max_seq_len == 0) return "compressed KV requires model context_length > 0";
        if (recent_window > max_seq_len)
            return "kv_recent_window " + std::to_string(recent_window) + " exceeds model context_length " +
                   std::to_string(max_seq_len) + "; use a smaller --kv-recent-window or --kv-compress-mode off";
        if (block_size > max_seq_len)
            return "kv_compress_block " + std::to_string(block_size) + " exceeds model context_length " +
                   std::to_string(max_seq_len);
        if ((mode == KvCompressMode::BlockSelectExact || mode == KvCompressMode::BlockSelectLossy) && top_blocks > 64)
            return "kv_compress_top_blocks " + std::to_string(top_blocks) + " exceeds the CUDA block-select limit of 64";
        switch (mode) {
            case KvCompressMode::Off: return "";
            case KvCompressMode::DenseRecentOnly:
            case KvCompressMode::RecentOnly:
            case KvCompressMode::BlockSummary:
            case KvCompressMode::BlockSelectLossy:
                if (head_dim != 64)
                    return std::string(mode_debug_str(mode)) + " currently requires head_dim=64, got head_dim=" +
                           std::to_string(head_dim);
                return "";
            case KvCompressMode::BlockSelectExact: {
                const auto backing = effective_exact_old_backing();
                const auto attention = effective_exact_old_attention();
                if (head_dim == 64) return "";
                if (head_dim == 128 && backing == KvExactOldBacking::Fp16KQ4V &&
                    attention == KvExactOldAttention::Fp16KQ4VDirect)
                    return "";
                return "block-select-exact currently requires head_dim=64, or head_dim=128 with --kv-exact-old-backing "
                       "fp16-k-q4-v and --kv-exact-old-attention fp16-k-q4-v-direct; got head_dim=" +
                       std::to_string(head_dim) + " backing=" + backing_str(backing) + " attention=" +
                       attention_str(attention);
            }
        }
        return "";
    }
};

namespace detail {
inline std::mutex& runtime_mu() { static std::mutex m; return m; }
inline KvCompressionConfig& runtime_cfg() { static KvCompressionConfig c; return c; }
inline std::optional<KvCompressionConfig>& scoped_cfg() {
    thread_local std::optional<KvCompressionConfig> c;
    return c;
}
}  // namespace detail

inline void set_runtime_config(const KvCompressionConfig& c) {
    std::lock_guard<std::mutex> g(detail::runtime_mu());
    detail::runtime_cfg() = c;
}
inline KvCompressionConfig runtime_config() {
    if (detail::scoped_cfg()) return *detail::scoped_cfg();
    std::lock_guard<std::mutex> g(detail::runtime_mu());
    return detail::runtime_cfg();
}
// RAII guard: shadows the process-wide configuration on this thread
class ScopedRuntimeConfig {
public:
    explicit ScopedRuntimeConfig(const KvCompressionConfig& c) : previous_(detail::scoped_cfg()) { detail::scoped_cfg() = c; }
    ~ScopedRuntimeConfig() { detail::scoped_cfg() = previous_; }
    ScopedRuntimeConfig(const ScopedRuntimeConfig&) = delete;
    ScopedRuntimeConfig& operator=(const ScopedRuntimeConfig&) = delete;

private:
    std::optional<KvCompressionConfig> previous_;
};

}  // namespace m40host
