// What runs on the next step.  The scheduler decides and the engine executes:
// nothing here touches a tensor.  A step is assembled out of one allowance of
// tokens and rows: first a row for every resident request's next token, then
// the tokens of prompts (the one part-way through, then newcomers) until the
// allowance is spent; pages come from the cache manager as rows are handed
// out, the newest request gives its pages up when the pools run dry, and the
// tokens that came out of a step are taken back in.  The policy (which request
// goes first, who is evicted, what is refused) is the reference's,
// crates/pagedllm/src/scheduler.rs, and its scenarios are the tests.
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
    // A step planned ahead (see plan_ahead): for every entry the row of the step before whose token it is
    // fed; the entry's own token is a placeholder.  Empty for every other step.
    std::vector<int> fed_rows;
    bool stalled = false;                               // planning it counted a stall of the queue's front (drop_ahead takes it back)
    bool launched = false;                              // the lengths in the cache have moved for it
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

    // Decoding a step ahead.  The tokens of a decoding step decide nothing about the next step but which
    // requests a stop token ends, so the next step can be on the device before they have been read:
    //   plan(); [run]; launched(); plan_ahead(); [run, fed on the device]; commit(tokens of the first);
    //   launched(); plan_ahead(); [run]; commit(tokens of the second); ...
    // `launched` says that the planned step is queued on the device: its tokens are as good as written
    // for everything queued behind it, so the lengths in the cache move now (commit does this itself
    // where nobody has).  `plan_ahead` gives the step behind a launched decoding step, or nothing when
    // that step is not known yet: the planner would bring the front of the queue in or turn it away, a
    // request is part-way through its prompt, the pools have no page for a row (then the ordinary
    // planner decides who gives way, after the commit), or a request waits while the launched step is some
    // resident's last by its budget or position (its pages come back at the commit, and the front may come in).
    // When it gives nothing it has taken nothing: the pages of its rows are counted first and taken only once the
    // step stands, so that the planner finds the pools as it would without steps ahead.  Otherwise it is a decoding step again: rows for
    // the residents in their order as far as the rows last, as the planner seats them.  Requests that the
    // launched step ends by their budget or the model's last position have no row in it; one that a stop
    // token ends has, and that row's token is dropped when it is committed (a resident that would have
    // had its row gets one a step later).  After the commit of the step before, the step planned ahead is the planned
    // step, and `plan` may not be asked until it is committed too.  `drop_ahead` forgets a step planned
    // ahead that was not launched after all.
    void launched();
    const Plan* plan_ahead();
    const Plan* ahead() const { return ahead_ ? &*ahead_ : nullptr; }
    void drop_ahead();
    // The planned step failed and will not be committed (its requests are cancelled by whoever saw it fail):
    // it is forgotten, and so is a step planned ahead of it.
    void abandon();
    const Outcome& last_outcome() const { return outcome_; }
    // `sampled` is one token per id of the plan, in the same order.
    const Outcome& commit(const std::vector<uint32_t>& sampled);
    void cancel(uint64_t id);
    const Outcome& drain_finished();

    Sequence* sequence(uint64_t id);

private:
    // A step under assembly: rows and tokens are handed out of one allowance, whoever asks.
    struct Assembly {
        Plan plan;
        size_t tokens_left;
        size_t rows_left;
        size_t decode_rows = 0;
        size_t prompt_tokens = 0;
        Assembly(size_t tokens, size_t rows) : tokens_left(tokens), rows_left(rows) {}
    };
    enum class WhenDry { GiveUp, EvictNewest };   // what seating does when a resident's next token has no page
    enum class Entry { PortionWise, Whole };      // how a newcomer's prompt will be fed

    bool turn_away_front();
    bool seat_residents(Assembly& step, WhenDry policy);
    bool feed_prompts(Assembly& step, Entry entry);
    std::optional<size_t> bring_in_front(Entry entry);
    void row_of_tokens(Assembly& step, Sequence& s, size_t first, size_t count, bool wants_logits);
    const Plan& publish(Assembly& step, PlanKind kind);
    void evict(size_t index);
    std::optional<size_t> newest_other_than(size_t keep) const;
    void retire(Outcome& outcome);
    std::optional<size_t> prompt_in_flight() const;

    CacheManager* cache_;
    std::deque<Sequence> waiting_;
    std::vector<Sequence> running_;
    size_t max_batch_;
    size_t chunk_;
    size_t max_positions_;
    Metrics metrics_;
    Plan plan_;
    std::optional<Plan> ahead_;
    Outcome outcome_;
    std::optional<FinishedInfo> outcome_pending_refusal_;
};

}  // namespace pl
