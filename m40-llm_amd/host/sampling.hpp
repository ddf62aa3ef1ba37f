// Host-side sampling: softmax with temperature, greedy, top-k, top-p, xorshift64* RNG.
// Mirrors src/sampling.rs of the reference (Sampler::sample :40-97, sample_greedy :99-112,
// softmax_temp :114-140, XorShift64Star :142-165).
#pragma once

#include <algorithm>
#include <cmath>
#include <cstdint>
#include <cstring>
#include <limits>
#include <optional>
#include <stdexcept>
#include <utility>
#include <vector>

namespace m40host {

struct SamplerConfig {
    float temperature = 1.0f;            // 1.0 => pure softmax
    std::optional<size_t> top_k;
    std::optional<float> top_p;          // 0 < p <= 1
    uint64_t seed = 42;
};

class XorShift64Star {
public:
    explicit XorShift64Star(uint64_t seed) : state_(seed) {}
    uint64_t next_u64() {
        uint64_t x = state_;
        x ^= x >> 12;
        x ^= x << 25;
        x ^= x >> 27;
        state_ = x;
        return x * 0x2545F4914F6CDD1DULL;
    }
    float next_f32() {
        const uint32_t mant = static_cast<uint32_t>(next_u64() >> 41);  // 23 bits
        return static_cast<float>(mant) / static_cast<float>(1u << 23);
    }

private:
    uint64_t state_;
};

// f32::total_cmp(a, b) == Greater
inline bool total_cmp_greater(float a, float b) {
    int32_t ia, ib;
    std::memcpy(&ia, &a, 4);
    std::memcpy(&ib, &b, 4);
    ia ^= static_cast<int32_t>(static_cast<uint32_t>(ia >> 31) >> 1);
    ib ^= static_cast<int32_t>(static_cast<uint32_t>(ib >> 31) >> 1);
    return ia > ib;
}

inline std::vector<float> softmax_temp(const float* logits, size_t n, float temperature) {
    const float t = temperature <= 0.0f ? 1e-6f : temperature;
    const float inv_t = 1.0f / t;
    float max_logit = -std::numeric_limits<float>::infinity();
    for (size_t i = 0; i < n; ++i) {
        const float v = logits[i] * inv_t;
        if (v > max_logit || max_logit != max_logit) max_logit = v;  // f32::max ignores NaN
    }
    std::vector<float> exps(n);
    float sum = 0.0f;
    for (size_t i = 0; i < n; ++i) {
        float x = std::exp(logits[i] * inv_t - max_logit);
        if (!(std::isfinite(x) && x > 0.0f)) x = 0.0f;
        exps[i] = x;
        sum += x;
    }
    if (sum <= 0.0f || !std::isfinite(sum)) return std::vector<float>(n, 0.0f);
    for (auto& x : exps) x = x / sum;
    return exps;
}

class Sampler {
public:
    explicit Sampler(SamplerConfig cfg) : cfg_(cfg), rng_(cfg.seed == 0 ? 1 : cfg.seed) {}

    size_t sample_greedy(const float* logits, size_t n) const {
        if (n == 0) throw std::invalid_argument("empty logits");
        size_t max_i = 0;
        float max_v = -std::numeric_limits<float>::infinity();
        for (size_t i = 0; i < n; ++i)
            if (logits[i] > max_v) { max_v = logits[i]; max_i = i; }
        return max_i;
    }

    size_t sample(const float* logits, size_t n) {
        if (n == 0) throw std::invalid_argument("empty logits");
        std::vector<float> probs = softmax_temp(logits, n, cfg_.temperature);
        for (auto& p : probs)
            if (!std::isfinite(p) || p < 0.0f) p = 0.0f;
        if (cfg_.top_k && *cfg_.top_k == 1 && n > 1 && !cfg_.top_p) {
            // top_k = 1 keeps the first element of a stable descending sort: the first index of the
            // maximum.  One pass instead of the O(V log V) sort; same result, same RNG consumption.
            size_t best = 0;
            for (size_t i = 1; i < n; ++i)
                if (total_cmp_greater(probs[i], probs[best])) best = i;
            if (!(probs[best] > 0.0f)) return sample_greedy(logits, n);
            (void)rng_.next_f32();
            return best;
        }
        std::vector<std::pair<size_t, float>> items(n);
        for (size_t i = 0; i < n; ++i) items[i] = {i, probs[i]};
        auto by_prob_desc = [](const std::pair<size_t, float>& a, const std::pair<size_t, float>& b) {
            return total_cmp_greater(a.second, b.second);
        };
        bool sorted_desc = false;
        if (cfg_.top_k) {
            const size_t k = *cfg_.top_k;
            if (k > 0 && k < items.size()) {
                std::stable_sort(items.begin(), items.end(), by_prob_desc);
                items.resize(k);
                sorted_desc = true;
            }
        }
        if (cfg_.top_p) {
            if (!sorted_desc) {
                std::stable_sort(items.begin(), items.end(), by_prob_desc);
                sorted_desc = true;
            }
            float cum = 0.0f;
            size_t keep = 0;
            for (const auto& it : items) {
                cum += it.second;
                keep += 1;
                if (cum >= *cfg_.top_p) break;
            }
            items.resize(std::max<size_t>(keep, 1));
        }
        if (!sorted_desc) std::stable_sort(items.begin(), items.end(), by_prob_desc);
        bool nonzero = false;
        for (const auto& it : items) nonzero = nonzero || it.second > 0.0f;
        if (!nonzero) return sample_greedy(logits, n);
        float sum = 0.0f;
        for (const auto& it : items) sum += it.second;
        float r = rng_.next_f32() * std::max(sum, std::numeric_limits<float>::epsilon());
        for (const auto& it : items) {
            if (r <= it.second) return it.first;
            r -= it.second;
        }
        return n - 1;
    }

    const SamplerConfig& config() const { return cfg_; }

private:
    SamplerConfig cfg_;
    XorShift64Star rng_;
};

// Convenience of src/decode.rs:111-117
inline Sampler greedy_sampler(uint64_t seed) {
    SamplerConfig c;
    c.top_k = 1;
    c.seed = seed;
    return Sampler(c);
}

}  // namespace m40host
