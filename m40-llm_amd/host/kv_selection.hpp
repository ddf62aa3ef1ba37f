// Process-global recorder of selected old blocks and attention-mass telemetry.
// Mirrors src/kv_selection.rs (types :3-82, capture policy :104-152, recorder :154-276).
#pragma once

#include <algorithm>
#include <cctype>
#include <cstdint>
#include <cstdlib>
#include <mutex>
#include <optional>
#include <set>
#include <string>
#include <vector>

namespace m40host {

struct KvAttentionGroupStats {
    float prob_mass = 0, logit_max = 0, logit_mean = 0;
    uint32_t count = 0;
};
struct KvSelectedBlock {
    uint32_t rank, block_index;
    float score;
    uint32_t absolute_start, absolute_end;
};
struct KvSelectionRecord {
    std::optional<uint32_t> layer, token;
    std::vector<KvSelectedBlock> selected_blocks;
    uint32_t total_old_blocks, top_blocks;
    std::optional<float> selection_elapsed_ms;
};
struct KvAttentionBlockMass {
    uint32_t block_index;
    float prob_mass, logit_max, logit_mean;
    uint32_t count;
};
struct KvAttentionTopEntry {
    std::string group;
    std::optional<uint32_t> block_index, token_position;
    float score, probability;
};
struct KvAttentionTelemetrySummary {
    KvAttentionGroupStats recent, selected_old_exact, summary, representatives, other;
    std::optional<float> needle_block_mass;
    std::vector<KvAttentionBlockMass> selected_block_masses;
    std::vector<KvAttentionTopEntry> top_entries;
};
struct KvAttentionTelemetryRecord {
    std::optional<uint32_t> layer, token;
    KvAttentionTelemetrySummary attention;
};
struct KvSelectionSummary {
    std::vector<uint32_t> selected_block_indices;   // ascending, unique
    uint32_t total_old_blocks, top_blocks;
    std::vector<KvSelectionRecord> selection_records;
    std::optional<KvAttentionTelemetrySummary> attention;
    std::vector<KvAttentionTelemetryRecord> attentions;
};

namespace kv_selection {

namespace detail {
struct State {
    std::set<uint32_t> selected;
    std::vector<KvSelectionRecord> selection_records;
    uint32_t total_old_blocks = 0, top_blocks = 0;
    std::vector<KvAttentionTelemetryRecord> attentions;
    std::optional<uint32_t> current_layer, current_token;
};
inline std::mutex& mu() { static std::mutex m; return m; }
inline State& state() { static State s; return s; }

struct CapturePolicy {
    enum Kind { First, All, Layer, Token, LayerToken } kind = First;
    uint32_t layer = 0, token = 0;
    static std::string trim(const std::string& s) {
        size_t a = 0, b = s.size();
        while (a < b && std::isspace((unsigned char)s[a])) ++a;
        while (b > a && std::isspace((unsigned char)s[b - 1])) --b;
        return s.substr(a, b - a);
    }
    static bool ieq(const std::string& a, const char* b) {
        std::string l = a;
        std::transform(l.begin(), l.end(), l.begin(), [](unsigned char c) { return std::tolower(c); });
        return l == b;
    }
    static std::optional<uint32_t> parse_u32(const std::string& s) {
        if (s.empty()) return std::nullopt;
        for (char c : s)
            if (!std::isdigit((unsigned char)c)) return std::nullopt;
        try {
            unsigned long long v = std::stoull(s);
            if (v > 0xffffffffull) return std::nullopt;
            return (uint32_t)v;
        } catch (...) { return std::nullopt; }
    }
    static CapturePolicy from_env() {
        CapturePolicy p;
        const char* raw = std::getenv("M40LLM_KV_ATTENTION_CAPTURE");
        if (!raw) return p;
        const std::string value = trim(raw);
        if (ieq(value, "all")) { p.kind = All; return p; }
        if (ieq(value, "first") || value.empty()) return p;
        std::optional<uint32_t> layer, token;
        size_t pos = 0;
        while (pos <= value.size()) {
            size_t comma = value.find(',', pos);
            if (comma == std::string::npos) comma = value.size();
            const std::string part = trim(value.substr(pos, comma - pos));
            const size_t colon = part.find(':');
            if (colon != std::string::npos) {
                const std::string key = trim(part.substr(0, colon)), val = trim(part.substr(colon + 1));
                if (key == "layer") layer = parse_u32(val);
                else if (key == "token") token = parse_u32(val);
            }
            pos = comma + 1;
        }
        if (layer && token) { p.kind = LayerToken; p.layer = *layer; p.token = *token; }
        else if (layer) { p.kind = Layer; p.layer = *layer; }
        else if (token) { p.kind = Token; p.token = *token; }
        return p;
    }
    bool matches(std::optional<uint32_t> l, std::optional<uint32_t> t) const {
        switch (kind) {
            case First: case All: return true;
            case Layer: return l && *l == layer;
            case Token: return t && *t == token;
            default: return l && *l == layer && t && *t == token;
        }
    }
};
}  // namespace detail

inline bool enabled() {
    const char* v = std::getenv("M40LLM_KV_SELECTION_TELEMETRY");
    if (!v) return false;
    const std::string s = v;
    return s == "1" || s == "true" || s == "TRUE" || s == "yes" || s == "YES";
}
inline std::optional<uint32_t> needle_block() {
    const char* v = std::getenv("M40LLM_KV_TELEMETRY_NEEDLE_BLOCK");
    return v ? detail::CapturePolicy::parse_u32(v) : std::nullopt;
}
inline void reset() {
    std::lock_guard<std::mutex> g(detail::mu());
    detail::state() = detail::State();
}
inline void set_attention_context(std::optional<uint32_t> layer, std::optional<uint32_t> token) {
    std::lock_guard<std::mutex> g(detail::mu());
    detail::state().current_layer = layer;
    detail::state().current_token = token;
}
inline void record_scored_timed(std::vector<KvSelectedBlock> blocks, uint32_t total_old_blocks, uint32_t top_blocks,
                                std::optional<float> elapsed_ms) {
    std::lock_guard<std::mutex> g(detail::mu());
    auto& s = detail::state();
    s.total_old_blocks = std::max(s.total_old_blocks, total_old_blocks);
    s.top_blocks = std::max(s.top_blocks, top_blocks);
    for (const auto& b : blocks) s.selected.insert(b.block_index);
    s.selection_records.push_back({s.current_layer, s.current_token, std::move(blocks), total_old_blocks, top_blocks, elapsed_ms});
}
inline void record_scored(std::vector<KvSelectedBlock> blocks, uint32_t total_old_blocks, uint32_t top_blocks) {
    record_scored_timed(std::move(blocks), total_old_blocks, top_blocks, std::nullopt);
}
inline void record(const std::vector<uint32_t>& selected_blocks, uint32_t total_old_blocks, uint32_t top_blocks) {
    std::vector<KvSelectedBlock> scored;
    for (size_t r = 0; r < selected_blocks.size(); ++r) scored.push_back({(uint32_t)r, selected_blocks[r], 0.0f, 0, 0});
    record_scored(std::move(scored), total_old_blocks, top_blocks);
}
inline bool has_attention() {
    std::lock_guard<std::mutex> g(detail::mu());
    return !detail::state().attentions.empty();
}
inline bool should_capture_attention() {
    if (!enabled()) return false;
    const auto policy = detail::CapturePolicy::from_env();
    std::lock_guard<std::mutex> g(detail::mu());
    const auto& s = detail::state();
    if (policy.kind == detail::CapturePolicy::First && !s.attentions.empty()) return false;
    return policy.matches(s.current_layer, s.current_token);
}
inline void record_attention(KvAttentionTelemetrySummary attention) {
    const auto policy = detail::CapturePolicy::from_env();
    std::lock_guard<std::mutex> g(detail::mu());
    auto& s = detail::state();
    if (policy.kind == detail::CapturePolicy::First && !s.attentions.empty()) return;
    s.attentions.push_back({s.current_layer, s.current_token, std::move(attention)});
}
inline std::optional<KvSelectionSummary> snapshot() {
    std::lock_guard<std::mutex> g(detail::mu());
    const auto& s = detail::state();
    if (s.total_old_blocks == 0 && s.selected.empty() && s.attentions.empty()) return std::nullopt;
    KvSelectionSummary out;
    out.selected_block_indices.assign(s.selected.begin(), s.selected.end());
    out.total_old_blocks = s.total_old_blocks;
    out.top_blocks = s.top_blocks;
    out.selection_records = s.selection_records;
    if (!s.attentions.empty()) out.attention = s.attentions.front().attention;
    out.attentions = s.attentions;
    return out;
}

}  // namespace kv_selection
}  // namespace m40host
