// Decode batching: sequence-slot pool with leases, request state, per-step batch plan with packed
// offsets, and the device-side plan that dispatches the variable-length batched attention.
// Mirrors src/decode_batch.rs (pool :14-85, request state :87-140, plan :142-220, device plan
// :222-355) and BatchMetadata::new of src/infer/batch.rs:276-355.
#pragma once

#include <cstdint>
#include <deque>
#include <memory>
#include <mutex>
#include <optional>
#include <stdexcept>
#include <string>
#include <vector>

#include "../../include/m40llm.h"

namespace m40host {

using DecodeRequestId = uint64_t;

class DecodeSequencePool;

class DecodeSequenceLease {
public:
    DecodeSequenceLease() = default;
    DecodeSequenceLease(uint32_t id, std::shared_ptr<struct PoolInner> inner) : id_(id), inner_(std::move(inner)) {}
    DecodeSequenceLease(DecodeSequenceLease&& o) noexcept : id_(o.id_), inner_(std::move(o.inner_)) {}
    DecodeSequenceLease& operator=(DecodeSequenceLease&& o) noexcept {
        release();
        id_ = o.id_;
        inner_ = std::move(o.inner_);
        return *this;
    }
    DecodeSequenceLease(const DecodeSequenceLease&) = delete;
    DecodeSequenceLease& operator=(const DecodeSequenceLease&) = delete;
    ~DecodeSequenceLease() { release(); }
    uint32_t sequence_id() const { return id_; }
    void release();

private:
    uint32_t id_ = 0;
    std::shared_ptr<struct PoolInner> inner_;
};

struct PoolInner {
    std::mutex mu;
    std::deque<uint32_t> free;   // FIFO: returned slots go to the back
    uint32_t capacity = 0;
};

inline void DecodeSequenceLease::release() {
    if (!inner_) return;
    std::lock_guard<std::mutex> g(inner_->mu);
    inner_->free.push_back(id_);
    inner_.reset();
}

class DecodeSequencePool {
public:
    explicit DecodeSequencePool(uint32_t capacity) : inner_(std::make_shared<PoolInner>()) {
        inner_->capacity = capacity;
        for (uint32_t i = 0; i < capacity; ++i) inner_->free.push_back(i);
    }
    uint32_t capacity() const { return inner_->capacity; }
    size_t available() const {
        std::lock_guard<std::mutex> g(inner_->mu);
        return inner_->free.size();
    }
    std::optional<DecodeSequenceLease> try_lease() {
        std::lock_guard<std::mutex> g(inner_->mu);
        if (inner_->free.empty()) return std::nullopt;
        const uint32_t id = inner_->free.front();
        inner_->free.pop_front();
        return DecodeSequenceLease(id, inner_);
    }

private:
    std::shared_ptr<PoolInner> inner_;
};

enum class DecodeRequestStatus : uint32_t { Active = 0, Completed = 1, Cancelled = 2 };

struct DecodeRequestState {
    DecodeRequestId request_id;
    uint32_t sequence_id;
    uint32_t kv_len;
    DecodeRequestStatus status;
    static DecodeRequestState active(DecodeRequestId r, uint32_t s, uint32_t l) { return {r, s, l, DecodeRequestStatus::Active}; }
    static DecodeRequestState completed(DecodeRequestId r, uint32_t s, uint32_t l) { return {r, s, l, DecodeRequestStatus::Completed}; }
    static DecodeRequestState cancelled(DecodeRequestId r, uint32_t s, uint32_t l) { return {r, s, l, DecodeRequestStatus::Cancelled}; }
    bool is_active() const { return status == DecodeRequestStatus::Active; }
};

struct BatchSequence {
    uint32_t seq_len, kv_len, query_len;
};

struct PackedSequenceOffsets {
    uint32_t token_offset, q_offset, kv_offset;
    uint64_t attention_offset;
};

// Exclusive-prefix packed offsets with overflow checks (src/infer/batch.rs:276-355).
class BatchMetadata {
public:
    static BatchMetadata make(std::vector<BatchSequence> sequences) {
        if (sequences.empty()) throw std::invalid_argument("batch metadata requires at least one sequence");
        BatchMetadata m;
        uint32_t token_sum = 0, q_sum = 0, kv_sum = 0;
        uint64_t attention_sum = 0;
        m.token_offsets_.push_back(0);
        m.q_offsets_.push_back(0);
        m.kv_offsets_.push_back(0);
        m.attention_offsets_.push_back(0);
        for (size_t idx = 0; idx < sequences.size(); ++idx) {
            const BatchSequence& s = sequences[idx];
            const std::string at = "sequence " + std::to_string(idx);
            if (s.seq_len == 0) throw std::invalid_argument(at + " has zero seq_len");
            if (s.query_len == 0) throw std::invalid_argument(at + " has zero query_len");
            if (s.kv_len == 0) throw std::invalid_argument(at + " has zero kv_len");
            if (s.query_len > s.seq_len)
                throw std::invalid_argument(at + " query_len " + std::to_string(s.query_len) + " exceeds seq_len " +
                                            std::to_string(s.seq_len));
            if (s.kv_len < s.query_len)
                throw std::invalid_argument(at + " kv_len " + std::to_string(s.kv_len) + " is smaller than query_len " +
                                            std::to_string(s.query_len));
            m.offsets_.push_back({token_sum, q_sum, kv_sum, attention_sum});
            if (__builtin_add_overflow(token_sum, s.seq_len, &token_sum))
                throw std::overflow_error("token_offsets overflow after " + at);
            if (__builtin_add_overflow(q_sum, s.query_len, &q_sum)) throw std::overflow_error("q_offsets overflow after " + at);
            if (__builtin_add_overflow(kv_sum, s.kv_len, &kv_sum)) throw std::overflow_error("kv_offsets overflow after " + at);
            if (__builtin_add_overflow(attention_sum, (uint64_t)s.query_len * (uint64_t)s.kv_len, &attention_sum))
                throw std::overflow_error("attention_offsets overflow after " + at);
            m.token_offsets_.push_back(token_sum);
            m.q_offsets_.push_back(q_sum);
            m.kv_offsets_.push_back(kv_sum);
            m.attention_offsets_.push_back(attention_sum);
        }
        m.sequences_ = std::move(sequences);
        return m;
    }
    const std::vector<BatchSequence>& sequences() const { return sequences_; }
    const std::vector<PackedSequenceOffsets>& offsets() const { return offsets_; }
    const std::vector<uint32_t>& q_offsets() const { return q_offsets_; }
    const std::vector<uint32_t>& kv_offsets() const { return kv_offsets_; }
    uint32_t total_tokens() const { return token_offsets_.back(); }
    uint32_t total_q_tokens() const { return q_offsets_.back(); }
    uint32_t total_kv_tokens() const { return kv_offsets_.back(); }
    uint64_t total_attention_cells() const { return attention_offsets_.back(); }

private:
    std::vector<BatchSequence> sequences_;
    std::vector<PackedSequenceOffsets> offsets_;
    std::vector<uint32_t> token_offsets_, q_offsets_, kv_offsets_;
    std::vector<uint64_t> attention_offsets_;
};

struct DecodeBatchEntry {
    DecodeRequestId request_id;
    uint32_t sequence_id;
    uint32_t kv_len;
    size_t batch_index;
};

class DecodeBatchPlan {
public:
    static DecodeBatchPlan from_requests(const std::vector<DecodeRequestState>& requests) {
        std::vector<DecodeRequestState> active;
        for (const auto& r : requests)
            if (r.is_active()) active.push_back(r);
        if (active.empty()) throw std::invalid_argument("decode batch requires at least one active request");
        DecodeBatchPlan p;
        std::vector<BatchSequence> sequences;
        for (size_t i = 0; i < active.size(); ++i) {
            const auto& r = active[i];
            if (r.kv_len == 0)
                throw std::invalid_argument("active request " + std::to_string(r.request_id) + " has zero kv_len");
            p.entries_.push_back({r.request_id, r.sequence_id, r.kv_len, i});
            sequences.push_back({r.kv_len, r.kv_len, 1});
        }
        p.metadata_ = BatchMetadata::make(std::move(sequences));
        return p;
    }
    const std::vector<DecodeBatchEntry>& entries() const { return entries_; }
    const BatchMetadata& metadata() const { return metadata_; }
    uint32_t batch_size() const { return static_cast<uint32_t>(entries_.size()); }
    std::vector<uint32_t> sequence_ids() const {
        std::vector<uint32_t> v;
        for (const auto& e : entries_) v.push_back(e.sequence_id);
        return v;
    }
    std::vector<uint32_t> sequence_lens() const {
        std::vector<uint32_t> v;
        for (const auto& e : entries_) v.push_back(e.kv_len);
        return v;
    }
    std::optional<size_t> batch_index_for_request(DecodeRequestId id) const {
        for (const auto& e : entries_)
            if (e.request_id == id) return e.batch_index;
        return std::nullopt;
    }
    std::optional<size_t> output_offset_f32(DecodeRequestId id, uint32_t q_heads, uint32_t head_dim) const {
        size_t per_item;
        if (__builtin_mul_overflow((size_t)q_heads, (size_t)head_dim, &per_item)) return std::nullopt;
        auto idx = batch_index_for_request(id);
        if (!idx) return std::nullopt;
        size_t off;
        if (__builtin_mul_overflow(*idx, per_item, &off)) return std::nullopt;
        return off;
    }

private:
    std::vector<DecodeBatchEntry> entries_;
    BatchMetadata metadata_;
};

// Device copy of (sequence ids, lengths) + dispatch of the batched attention entry point.
class DeviceDecodeBatchPlan {
public:
    DeviceDecodeBatchPlan(M40llmCudaContext* ctx, DecodeBatchPlan plan) : ctx_(ctx), plan_(std::move(plan)) {
        const size_t bytes = (size_t)plan_.batch_size() * sizeof(uint32_t);
        if (m40llm_device_malloc(ctx_, bytes, &d_ids_) != 0 || m40llm_device_malloc(ctx_, bytes, &d_lens_) != 0) {
            cleanup();
            throw std::runtime_error("decode_batch: device allocation failed");
        }
        const auto ids = plan_.sequence_ids();
        const auto lens = plan_.sequence_lens();
        if (m40llm_memcpy_h2d(ctx_, d_ids_, ids.data(), bytes) != 0 || m40llm_memcpy_h2d(ctx_, d_lens_, lens.data(), bytes) != 0) {
            cleanup();
            throw std::runtime_error("decode_batch: metadata upload failed");
        }
    }
    DeviceDecodeBatchPlan(const DeviceDecodeBatchPlan&) = delete;
    DeviceDecodeBatchPlan& operator=(const DeviceDecodeBatchPlan&) = delete;
    ~DeviceDecodeBatchPlan() { cleanup(); }
    const DecodeBatchPlan& plan() const { return plan_; }
    const uint32_t* d_sequence_ids() const { return static_cast<const uint32_t*>(d_ids_); }
    const uint32_t* d_sequence_lens() const { return static_cast<const uint32_t*>(d_lens_); }
    // q and out packed [batch][q_heads][head_dim] in plan.entries() order
    int dispatch_attention(const M40llmKVCache* kv, const void* d_q, uint32_t q_heads, void* d_out) const {
        return m40llm_attention_last_token_f32_gqa_batched(ctx_, kv, d_sequence_ids(), d_sequence_lens(),
                                                           plan_.batch_size(), d_q, q_heads, d_out);
    }
    int dispatch_attention_async(const M40llmKVCache* kv, const void* d_q, uint32_t q_heads, void* d_out) const {
        return m40llm_attention_last_token_f32_gqa_batched_async(ctx_, kv, d_sequence_ids(), d_sequence_lens(),
                                                                 plan_.batch_size(), d_q, q_heads, d_out);
    }

private:
    void cleanup() {
        if (d_ids_) m40llm_device_free(ctx_, d_ids_);
        if (d_lens_) m40llm_device_free(ctx_, d_lens_);
        d_ids_ = d_lens_ = nullptr;
    }
    M40llmCudaContext* ctx_;
    DecodeBatchPlan plan_;
    void* d_ids_ = nullptr;
    void* d_lens_ = nullptr;
};

}  // namespace m40host
