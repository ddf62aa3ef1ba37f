// Continuous-batching decode scheduler: requests arrive at any time, lease a sequence slot, are prefilled together,
// then take one batched decode step per tick until their stopping criteria fire; the slot returns to the pool.
//
// Follows the reference's server scheduler (src/server.rs:203-770) without its HTTP, tokenizer and channel plumbing:
//   submit        = enqueue_scheduler_request + DecodeSchedulerRequest::new (:231-290, :764-783): lease a sequence
//                   slot (no free slot -> the request is refused, nothing waits), build the stopping criteria
//                   (max_tokens + stop ids), give the request the next id;
//   tick          = the loop body of decode_scheduler_loop (:713-762) + process_scheduler_batch_tick (:604-711):
//                   cancelled requests leave; the rest split into complete / pending prefill / decode
//                   (split_scheduler_requests :536-556); pending prefills run as one packed prefill and sample their
//                   first token (process_scheduler_prefill_tick :559-602, finish_prefill :378-404); decode requests
//                   each contribute their newest token to one batched step and sample from their logits row
//                   (prepare_batch_token :331-348, finish_batch_token :406-433);
//   a request that finishes in a tick is reported then (send_complete), its lease dropped (slot to the back of the
//   free list, src/decode_batch.rs:75-85).
// The engine that runs the model is behind two callbacks (and an optional third that lets the engine pick the token of
// greedy requests itself), so the scheduling logic can be exercised without a GPU.
#pragma once

#include <cstdint>
#include <deque>
#include <functional>
#include <map>
#include <memory>
#include <optional>
#include <stdexcept>
#include <string>
#include <vector>

#include "decode.hpp"
#include "decode_batch.hpp"
#include "sampling.hpp"

namespace m40host {

struct SchedulerPrefillItem {
    uint32_t sequence_id;
    const uint32_t* tokens;
    uint32_t len;
};
struct SchedulerDecodeItem {
    uint32_t sequence_id;
    uint32_t kv_len;   // tokens the sequence's cache holds = position of `token`
    uint32_t token;
};

struct SchedulerEngine {
    uint32_t vocab = 0;
    uint32_t max_seq_len = 0;
    // logits_out: one row of `vocab` floats per item (the last prompt token's logits / the new token's logits)
    std::function<void(const std::vector<SchedulerPrefillItem>&, float* logits_out)> prefill;
    std::function<void(const std::vector<SchedulerDecodeItem>&, float* logits_out)> decode;
    // Optional.  Like decode, but rows flagged greedy (their sampler keeps only the top token) may be decided by the
    // engine: it stores the first index of the row's maximum in picks_out[r] and sets picked_out[r] = 1, and then need
    // not fill that row's logits (a model does so on the device when the top two logits are not a near tie).
    std::function<void(const std::vector<SchedulerDecodeItem>&, const uint8_t* greedy, float* logits_out, uint32_t* picks_out,
                       uint8_t* picked_out)>
        decode_pick;
};

enum class SchedulerRequestState : uint32_t { Unknown = 0, PendingPrefill = 1, Decoding = 2, Complete = 3, Cancelled = 4, Failed = 5 };

struct SchedulerTickReport {
    uint32_t prefill_rows = 0, prefill_tokens = 0, decode_rows = 0, completed = 0, cancelled = 0, failed = 0;
};

class DecodeScheduler {
public:
    DecodeScheduler(SchedulerEngine engine, uint32_t sequence_slots) : engine_(std::move(engine)), pool_(sequence_slots) {
        if (!engine_.prefill || !engine_.decode || engine_.vocab == 0) throw std::invalid_argument("scheduler engine incomplete");
    }

    uint32_t capacity() const { return pool_.capacity(); }
    size_t available_slots() const { return pool_.available(); }
    size_t active() const { return active_.size(); }

    // Returns the request id (1, 2, ...).  Throws when no sequence slot is free or the prompt is unusable.
    uint64_t submit(const uint32_t* prompt, size_t n_prompt, std::optional<size_t> max_tokens, std::vector<uint32_t> stop_ids,
                    SamplerConfig sampler) {
        if (n_prompt == 0 || !prompt) throw std::invalid_argument("empty prompt");
        if (engine_.max_seq_len && n_prompt > engine_.max_seq_len) throw std::invalid_argument("prompt longer than the context window");
        for (size_t i = 0; i < n_prompt; ++i)
            if (prompt[i] >= engine_.vocab) throw std::out_of_range("token id out of range");
        auto lease = pool_.try_lease();
        if (!lease) throw std::runtime_error("decode batching requires a sequence lease");   // server.rs:239-240
        auto r = std::make_unique<Request>(std::move(*lease), sampler);
        r->id = next_id_++;
        r->ids.assign(prompt, prompt + n_prompt);
        r->prompt_len = n_prompt;
        // max_tokens defaults to the context length (server.rs:248-251)
        r->stopping = StoppingCriteria::with_stop_ids(max_tokens ? max_tokens : std::optional<size_t>(engine_.max_seq_len ? engine_.max_seq_len : 32),
                                                      std::move(stop_ids));
        const uint64_t id = r->id;
        states_[id] = SchedulerRequestState::PendingPrefill;
        active_.push_back(std::move(r));
        return id;
    }

    // The request leaves at the start of the next tick (is_cancelled, server.rs:733-743); unknown or finished ids: false.
    bool cancel(uint64_t id) {
        for (auto& r : active_)
            if (r->id == id) {
                r->cancelled = true;
                return true;
            }
        return false;
    }

    SchedulerRequestState state(uint64_t id) const {
        const auto it = states_.find(id);
        return it == states_.end() ? SchedulerRequestState::Unknown : it->second;
    }
    uint32_t sequence_of(uint64_t id) const {
        for (const auto& r : active_)
            if (r->id == id) return r->lease.sequence_id();
        return 0xffffffffu;
    }
    // generated ids so far (any state); empty for unknown ids
    std::vector<uint32_t> generated(uint64_t id) const {
        for (const auto& r : active_)
            if (r->id == id) return r->generated;
        const auto it = results_.find(id);
        return it == results_.end() ? std::vector<uint32_t>() : it->second;
    }
    std::string error_of(uint64_t id) const {
        const auto it = errors_.find(id);
        return it == errors_.end() ? std::string() : it->second;
    }
    // the batch the next tick would decode, as the reference logs it (log_decode_batch_plan, server.rs:786-806)
    DecodeBatchPlan plan() const {
        std::vector<DecodeRequestState> states;
        for (const auto& r : active_) states.push_back(DecodeRequestState::active(r->id, r->lease.sequence_id(), (uint32_t)r->ids.size()));
        return DecodeBatchPlan::from_requests(states);
    }

    SchedulerTickReport tick() {
        SchedulerTickReport rep;
        // cancelled requests leave first
        for (auto it = active_.begin(); it != active_.end();) {
            if ((*it)->cancelled) {
                finish(**it, SchedulerRequestState::Cancelled);
                it = active_.erase(it);
                ++rep.cancelled;
            } else {
                ++it;
            }
        }
        if (active_.empty()) return rep;
        std::vector<std::unique_ptr<Request>> current;
        for (auto& r : active_) current.push_back(std::move(r));
        active_.clear();
        std::vector<std::unique_ptr<Request>> prefill, decode;
        for (auto& r : current) {   // split_scheduler_requests
            if (r->stopping.should_stop(r->generated)) {
                finish(*r, SchedulerRequestState::Complete);
                ++rep.completed;
            } else if (r->processed == 0 && r->generated.empty()) {
                prefill.push_back(std::move(r));
            } else {
                decode.push_back(std::move(r));
            }
        }
        if (!prefill.empty()) run_prefill(prefill, rep);
        if (!decode.empty()) run_decode(decode, rep);
        return rep;
    }

private:
    struct Request {
        Request(DecodeSequenceLease l, SamplerConfig s) : lease(std::move(l)), sampler(s) {}
        uint64_t id = 0;
        DecodeSequenceLease lease;
        Sampler sampler;
        StoppingCriteria stopping;
        std::vector<uint32_t> ids, generated;
        size_t prompt_len = 0, processed = 0;   // processed: tokens whose KV entries exist
        bool cancelled = false;
    };

    void finish(Request& r, SchedulerRequestState st, const std::string& err = std::string()) {
        states_[r.id] = st;
        results_[r.id] = r.generated;
        if (!err.empty()) errors_[r.id] = err;
        // the lease is dropped with the request: the slot goes to the back of the free list
    }

    // sample from a logits row, push the token, then complete or stay active (finish_prefill / finish_batch_token)
    void sample_and_route(std::unique_ptr<Request> r, const float* logits, SchedulerTickReport& rep, const uint32_t* pick = nullptr) {
        const uint32_t next = pick ? *pick : static_cast<uint32_t>(r->sampler.sample(logits, engine_.vocab));
        r->ids.push_back(next);
        r->generated.push_back(next);
        if (r->stopping.should_stop(r->generated)) {
            finish(*r, SchedulerRequestState::Complete);
            ++rep.completed;
        } else {
            states_[r->id] = SchedulerRequestState::Decoding;
            active_.push_back(std::move(r));
        }
    }

    void fail_all(std::vector<std::unique_ptr<Request>>& rs, const std::string& what, SchedulerTickReport& rep) {
        for (auto& r : rs) {
            finish(*r, SchedulerRequestState::Failed, what);
            ++rep.failed;
        }
        rs.clear();
    }

    void run_prefill(std::vector<std::unique_ptr<Request>>& rs, SchedulerTickReport& rep) {
        std::vector<SchedulerPrefillItem> items;
        for (const auto& r : rs) {
            items.push_back({r->lease.sequence_id(), r->ids.data(), (uint32_t)r->prompt_len});
            rep.prefill_tokens += (uint32_t)r->prompt_len;
        }
        rep.prefill_rows = (uint32_t)rs.size();
        logits_.resize(items.size() * (size_t)engine_.vocab);
        try {
            engine_.prefill(items, logits_.data());
        } catch (const std::exception& e) {
            fail_all(rs, std::string("batched prefill forward failed: ") + e.what(), rep);   // server.rs:592-596
            return;
        }
        for (size_t i = 0; i < rs.size(); ++i) {
            rs[i]->processed = rs[i]->prompt_len;
            sample_and_route(std::move(rs[i]), logits_.data() + i * (size_t)engine_.vocab, rep);
        }
    }

    void run_decode(std::vector<std::unique_ptr<Request>>& rs, SchedulerTickReport& rep) {
        // a sequence at the end of its context window cannot take another token
        std::vector<std::unique_ptr<Request>> ready;
        for (auto& r : rs) {
            if (engine_.max_seq_len && r->processed + 1 > engine_.max_seq_len) {
                finish(*r, SchedulerRequestState::Failed, "context window exhausted");
                ++rep.failed;
            } else {
                ready.push_back(std::move(r));
            }
        }
        if (ready.empty()) return;
        std::vector<SchedulerDecodeItem> items;
        for (const auto& r : ready)   // the next unprocessed token of each request (prepare_batch_token)
            items.push_back({r->lease.sequence_id(), (uint32_t)r->processed, r->ids[r->processed]});
        rep.decode_rows = (uint32_t)ready.size();
        logits_.resize(items.size() * (size_t)engine_.vocab);
        std::vector<uint8_t> greedy(ready.size(), 0), picked(ready.size(), 0);
        std::vector<uint32_t> picks(ready.size(), 0);
        try {
            if (engine_.decode_pick) {
                for (size_t i = 0; i < ready.size(); ++i) {
                    const SamplerConfig& c = ready[i]->sampler.config();
                    // the pick replaces the sample only where the request's next step samples (no prompt tokens left)
                    greedy[i] = c.top_k && *c.top_k == 1 && !c.top_p && ready[i]->processed + 1 == ready[i]->ids.size();
                }
                engine_.decode_pick(items, greedy.data(), logits_.data(), picks.data(), picked.data());
            } else {
                engine_.decode(items, logits_.data());
            }
        } catch (const std::exception& e) {
            fail_all(ready, std::string("batched decode forward failed: ") + e.what(), rep);   // server.rs:680-685
            return;
        }
        for (size_t i = 0; i < ready.size(); ++i) {
            auto& r = ready[i];
            r->processed += 1;
            if (r->processed < r->ids.size()) {   // still catching up with its own ids (finish_batch_token :410-412)
                active_.push_back(std::move(r));
                continue;
            }
            sample_and_route(std::move(r), logits_.data() + i * (size_t)engine_.vocab, rep, picked[i] ? &picks[i] : nullptr);
        }
    }

    SchedulerEngine engine_;
    DecodeSequencePool pool_;
    std::deque<std::unique_ptr<Request>> active_;
    std::map<uint64_t, SchedulerRequestState> states_;
    std::map<uint64_t, std::vector<uint32_t>> results_;
    std::map<uint64_t, std::string> errors_;
    std::vector<float> logits_;
    uint64_t next_id_ = 1;
};

}  // namespace m40host
