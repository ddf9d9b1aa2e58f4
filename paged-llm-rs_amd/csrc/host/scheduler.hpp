// What runs on the next step.  The scheduler decides and the engine executes:
// nothing here touches a tensor.  It admits requests, cuts prompts into
// portions under a token budget, puts one portion beside every running
// request's next token, takes pages from the cache manager, evicts the newest
// request when the pools run dry, and takes back the tokens that came out.
// (Reference: crates/pagedllm/src/scheduler.rs.)
#pragma once

#include <cstdint>
#include <deque>
#include <optional>
#include <utility>
#include <vector>

#include "cache.hpp"
#include "sampler.hpp"

namespace pl {

enum class Finish : int { None = 0, Stop = 1, Length = 2 };
enum class PlanKind : int { Idle = 0, Prefill = 1, Mixed = 2, Decode = 3, Refused = 4 };

// One request, from arrival to its last token (scheduler.rs:34-56).
struct Sequence {
    uint64_t id = 0;
    std::vector<uint32_t> history;  // everything the model has seen: prompt, then output
    size_t prompt_tokens = 0;
    Sampling sampling;
    size_t max_tokens = 0;
    std::vector<uint32_t> stop_tokens;
    Rng rng;
    std::vector<uint32_t> pending;  // fed on the next step
    size_t generated = 0;
    uint32_t preemptions = 0;
    size_t prompt_left = 0;         // non-zero only while a prompt runs a portion at a time
    Finish finish = Finish::None;
    int state_slot = -1;
    bool state_fresh = false;       // the slot has to be cleared before its first use
};

// The tokens one request contributes to a step.
struct PlanEntry {
    uint64_t id;
    size_t start;                   // position of the first token
    std::vector<uint32_t> tokens;
    bool wants_logits;              // at the last of these tokens
    int state_slot;
    bool state_fresh;
};

struct Plan {
    PlanKind kind = PlanKind::Idle;
    std::vector<uint64_t> ids;                          // requests a token comes back for, in row order
    std::vector<std::pair<uint64_t, size_t>> advanced;  // (id, tokens written)
    std::vector<PlanEntry> entries;
    uint64_t refused = 0;
};

struct FinishedInfo {
    uint64_t id;
    Finish finish;
    size_t prompt_tokens;
    size_t generated;
    uint32_t preemptions;
};

struct Outcome {
    std::vector<std::pair<uint64_t, uint32_t>> tokens;
    std::vector<FinishedInfo> finished;
};

// scheduler.rs:203-231
struct Metrics {
    uint64_t steps = 0, prefills = 0, tokens = 0, decode_rows = 0, admission_stalls = 0,
             preemptions = 0, mixed_steps = 0, decode_steps = 0, recomputed_tokens = 0,
             cached_tokens = 0, prefilled_tokens = 0;
};

class Scheduler {
public:
    // `chunk` 0 runs a prompt whole (prefill first); otherwise it is the most
    // tokens one step may carry.  `max_positions` 0 means no limit.
    Scheduler(CacheManager* cache, size_t max_batch, size_t chunk, size_t max_positions);

    void set_chunk(size_t tokens) { chunk_ = tokens; }
    size_t chunk() const { return chunk_; }
    void set_prefix_cache(bool enabled) { cache_->set_prefix_cache(enabled); }

    // Throws Error on an empty prompt or sampling parameters out of range.
    void submit(Sequence sequence);
    size_t waiting() const { return waiting_.size(); }
    size_t running() const { return running_.size(); }
    std::vector<uint64_t> running_ids() const;
    const Metrics& metrics() const { return metrics_; }
    size_t wasted_tokens() const;

    const Plan& plan();
    const Plan& last_plan() const { return plan_; }
    const Outcome& last_outcome() const { return outcome_; }
    // `sampled` is one token per id of the plan, in the same order.
    const Outcome& commit(const std::vector<uint32_t>& sampled);
    void cancel(uint64_t id);
    const Outcome& drain_finished();

    Sequence* sequence(uint64_t id);

private:
    std::optional<Plan> mixed();
    std::optional<Plan> admit();
    Plan decode();
    std::optional<Plan> refuse_unservable();
    void start_next_prompt();
    std::optional<size_t> newest_evictable(size_t protect) const;
    void preempt(size_t index);
    void retire(Outcome& outcome);
    std::optional<size_t> prompt_in_flight() const;
    PlanEntry entry_for(Sequence& s, size_t start, std::vector<uint32_t> tokens, bool wants);

    CacheManager* cache_;
    std::deque<Sequence> waiting_;
    std::vector<Sequence> running_;
    size_t max_batch_;
    size_t chunk_;
    size_t max_positions_;
    Metrics metrics_;
    Plan plan_;
    Outcome outcome_;
    std::optional<FinishedInfo> outcome_pending_refusal_;
};

}  // namespace pl
