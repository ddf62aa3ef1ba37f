// Decode loop helpers: stopping criteria for EOS / stop ids / max_tokens and the minimal
// host-side loop that consumes logits from a callback.  Mirrors src/decode.rs of the reference
// (StoppingCriteria :10-54, decode_loop_with :59-108); the tokenizer is outside the hot path,
// so the loop starts from prompt token ids.
#pragma once

#include <algorithm>
#include <cstdint>
#include <functional>
#include <optional>
#include <stdexcept>
#include <vector>

#include "sampling.hpp"

namespace m40host {

struct StoppingCriteria {
    std::optional<size_t> max_tokens;
    std::optional<uint32_t> eos_id;
    std::vector<uint32_t> stop_ids;

    static StoppingCriteria make(std::optional<size_t> max_tokens, std::optional<uint32_t> eos_id) {
        StoppingCriteria s;
        s.max_tokens = max_tokens;
        s.eos_id = eos_id;
        if (eos_id) s.stop_ids.push_back(*eos_id);
        return s;
    }
    static StoppingCriteria with_stop_ids(std::optional<size_t> max_tokens, std::vector<uint32_t> stop_ids) {
        StoppingCriteria s;
        s.max_tokens = max_tokens;
        if (!stop_ids.empty()) s.eos_id = stop_ids.front();
        std::sort(stop_ids.begin(), stop_ids.end());
        stop_ids.erase(std::unique(stop_ids.begin(), stop_ids.end()), stop_ids.end());
        s.stop_ids = std::move(stop_ids);
        return s;
    }
    bool is_stop_id(uint32_t id) const { return std::find(stop_ids.begin(), stop_ids.end(), id) != stop_ids.end(); }
    bool should_stop(const std::vector<uint32_t>& generated) const {
        if (max_tokens && generated.size() >= *max_tokens) return true;
        if (!generated.empty() && is_stop_id(generated.back())) return true;
        return false;
    }
};

// logits_fn receives every id so far and returns the logits of the last position.
inline std::vector<uint32_t> decode_loop_with(std::vector<uint32_t> ids, Sampler sampler,
                                              const StoppingCriteria& stopping,
                                              const std::function<std::vector<float>(const std::vector<uint32_t>&)>& logits_fn) {
    const size_t start_len = ids.size();
    std::vector<uint32_t> generated;
    for (;;) {
        if (stopping.should_stop(generated)) break;
        std::vector<float> logits = logits_fn(ids);
        if (logits.empty()) throw std::runtime_error("logits_fn returned empty logits");
        const uint32_t next = static_cast<uint32_t>(sampler.sample(logits.data(), logits.size()));
        ids.push_back(next);
        generated.push_back(next);
        if (stopping.is_stop_id(next)) break;
        if (stopping.max_tokens && generated.size() >= *stopping.max_tokens) break;
        if (!stopping.max_tokens && !stopping.eos_id && generated.size() > 4 * std::max<size_t>(start_len, 1) &&
            generated.size() > 4096) {
            throw std::runtime_error("decode_loop_with: refusing to continue without stopping criteria");
        }
    }
    return ids;
}

}  // namespace m40host
