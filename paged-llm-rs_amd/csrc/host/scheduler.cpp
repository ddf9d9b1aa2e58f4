#include "scheduler.hpp"

#include <algorithm>

namespace pl {

Scheduler::Scheduler(CacheManager* cache, size_t max_batch, size_t chunk, size_t max_positions)
    : cache_(cache), max_batch_(std::max<size_t>(max_batch, 1)), chunk_(chunk), max_positions_(max_positions) {}

void Scheduler::submit(Sequence sequence) {
    if (sequence.history.empty()) throw Error("cannot generate from an empty prompt");
    sequence.prompt_tokens = sequence.history.size();
    sequence.pending = sequence.history;
    sequence.generated = 0;
    sequence.prompt_left = 0;
    sequence.finish = Finish::None;
    waiting_.push_back(std::move(sequence));
}

std::vector<uint64_t> Scheduler::running_ids() const {
    std::vector<uint64_t> ids;
    for (const Sequence& s : running_) ids.push_back(s.id);
    return ids;
}

size_t Scheduler::wasted_tokens() const {
    size_t total = 0;
    for (const Sequence& s : running_) total += cache_->wasted_tokens(s.id);
    return total;
}

Sequence* Scheduler::sequence(uint64_t id) {
    for (Sequence& s : running_)
        if (s.id == id) return &s;
    return nullptr;
}

std::optional<size_t> Scheduler::prompt_in_flight() const {
    for (size_t i = 0; i < running_.size(); ++i)
        if (running_[i].prompt_left > 0 && running_[i].finish == Finish::None) return i;
    return std::nullopt;
}

// ---------------------------------------------------------------------------
// Assembling a step.
//
// Three kinds of step come out of the same four moves.  With a token allowance
// (chunk > 0): seat the residents, giving the step up if one of them finds no
// page; feed prompts with what the residents left; if any prompt token went in,
// that is the step.  Without an allowance: bring the front prompt in whole and
// run it alone.  Whenever neither made a step: seat the residents again, this
// time evicting for pages, and decode.  (scheduler.rs:368-381 has the same order
// of preference as three separate planners.)
// ---------------------------------------------------------------------------
const Plan& Scheduler::plan() {
    if (!plan_.fed_rows.empty() || ahead_)
        throw Error("a step planned ahead is on the device: commit it before planning another");
    if (turn_away_front()) return plan_;
    if (chunk_ > 0) {
        // every row carries at least one token, so the allowance bounds the rows as well
        Assembly step(chunk_, std::min(max_batch_, chunk_));
        if (seat_residents(step, WhenDry::GiveUp) && feed_prompts(step, Entry::PortionWise))
            return publish(step, PlanKind::Mixed);
    } else {
        Assembly step(SIZE_MAX, 1);
        if (feed_prompts(step, Entry::Whole)) return publish(step, PlanKind::Prefill);
    }
    Assembly step(max_batch_, max_batch_);
    seat_residents(step, WhenDry::EvictNewest);
    return publish(step, step.plan.entries.empty() ? PlanKind::Idle : PlanKind::Decode);
}

// One row of the step: `count` tokens of `s` from position `first` of its history.
void Scheduler::row_of_tokens(Assembly& step, Sequence& s, size_t first, size_t count, bool wants_logits) {
    if (wants_logits) step.plan.ids.push_back(s.id);
    step.plan.advanced.emplace_back(s.id, count);
    step.plan.entries.push_back(PlanEntry{
        s.id, first, std::vector<uint32_t>(s.history.begin() + static_cast<long>(first),
                                           s.history.begin() + static_cast<long>(first + count)),
        wants_logits, s.state_slot, s.state_fresh});
    s.state_fresh = false;
    step.rows_left -= std::min<size_t>(step.rows_left, 1);
    step.tokens_left -= std::min(step.tokens_left, count);
}

// A row for the next token of every resident that has one to feed, in the order
// of arrival, as far as the rows last.  Each needs room for one more token in
// its pages.  Where the pools cannot give that: under GiveUp nothing is seated
// and false comes back (the caller then decodes instead, which may evict; a
// step that carried a prompt beside an incomplete set of residents would starve
// the one left out); under EvictNewest the newest resident other than the asker
// loses its pages and goes back to the front of the queue, and the asker tries
// again (scheduler.rs:625-676).  A request that is alone and still finds no page
// can never be served further and ends with what it has.
bool Scheduler::seat_residents(Assembly& step, WhenDry policy) {
    std::vector<uint64_t> seated;
    size_t index = 0;
    while (index < running_.size() && seated.size() < step.rows_left) {
        Sequence& s = running_[index];
        if (s.finish != Finish::None || s.pending.size() != 1) {   // done, or still taking its prompt in
            ++index;
            continue;
        }
        if (cache_->reserve(s.id, 1)) {
            seated.push_back(s.id);
            ++index;
            continue;
        }
        if (policy == WhenDry::GiveUp) return false;
        const auto victim = newest_other_than(index);
        if (!victim) {
            s.finish = Finish::Length;
            ++index;
            continue;
        }
        seated.erase(std::remove(seated.begin(), seated.end(), running_[*victim].id), seated.end());
        evict(*victim);
        if (*victim < index) --index;      // the asker has moved down by one
    }
    for (uint64_t id : seated) {
        Sequence* s = sequence(id);
        // the token to feed is the last of the history: what the step before produced
        row_of_tokens(step, *s, cache_->tokens(id), 1, true);
    }
    step.decode_rows = seated.size();
    return true;
}

// Prompt tokens into what is left of the step: first the prompt that an earlier
// step left part-way, then newcomers from the front of the queue, each from
// where its cached or already fed tokens end.  A prompt that does not fit
// whole gets what fits (what the pools can back, at most) and stays in flight;
// since only one prompt may be in flight, nothing follows it.  Only the row
// that holds a prompt's last token asks for logits.  True when at least one
// prompt token went in.  (The reference feeds a slice of one prompt a step,
// scheduler.rs:388-499; here short prompts share a step, so a batch of short
// requests fills in a few steps instead of one step a request.)
bool Scheduler::feed_prompts(Assembly& step, Entry entry) {
    std::optional<size_t> index = entry == Entry::PortionWise ? prompt_in_flight() : std::nullopt;
    // (The first prompt row goes in even when the residents have taken every row: a prompt in flight
    // must not wait for a resident to finish.)
    while (step.tokens_left > 0 && (step.prompt_tokens == 0 || step.rows_left > 0)) {
        if (!index) {
            // a newcomer takes its first pages only now, after the residents have theirs
            index = bring_in_front(entry);
            if (!index) break;
        }
        Sequence& s = running_[*index];
        const size_t fed = s.history.size() - s.prompt_left;
        const size_t take = cache_->reserve_up_to(s.id, std::min(step.tokens_left, s.prompt_left));
        if (take == 0) break;
        const bool completes = take == s.prompt_left;
        row_of_tokens(step, s, fed, take, completes);
        step.prompt_tokens += take;
        if (!completes) break;
        index.reset();
    }
    return step.prompt_tokens > 0;
}

// The front of the queue becomes a resident: a state slot, the pages of whatever
// prefix of its prompt the cache already holds, and pages of its own for what
// it needs at once (everything, when its prompt is to run whole; room for one
// token otherwise, so that even a fully cached prompt has somewhere to write).
// Where the pools or the slots cannot give that, everything is handed back, the
// request keeps its place and the stall is counted (scheduler.rs:503-589).
std::optional<size_t> Scheduler::bring_in_front(Entry entry) {
    if (waiting_.empty()) return std::nullopt;
    const size_t prompt_len = waiting_.front().pending.size();
    const bool room = entry == Entry::Whole ? cache_->fits_from_scratch(prompt_len) : cache_->min_available() > 0;
    if (!room || !cache_->state_slot_available()) {
        metrics_.admission_stalls += 1;
        return std::nullopt;
    }
    Sequence s = std::move(waiting_.front());
    waiting_.pop_front();
    s.state_slot = cache_->add_sequence(s.id);
    s.state_fresh = s.state_slot >= 0;
    const size_t shared = cache_->claim_prefix(s.id, s.pending.data(), s.pending.size());
    const size_t at_once = entry == Entry::Whole ? prompt_len - shared : 1;
    if (!cache_->reserve(s.id, at_once)) {
        cache_->free_sequence(s.id);
        s.state_slot = -1;
        s.pending = s.history;
        waiting_.push_front(std::move(s));
        metrics_.admission_stalls += 1;
        return std::nullopt;
    }
    metrics_.cached_tokens += shared;
    metrics_.prefilled_tokens += prompt_len - shared;
    metrics_.prefills += 1;
    s.prompt_left = std::max<size_t>(prompt_len - shared, 1);   // the last token is always fed: its logits are wanted
    s.pending.clear();                                          // nothing to decode until the prompt is in
    running_.push_back(std::move(s));
    return running_.size() - 1;
}

// The assembled step becomes the plan, and the counters learn of it.
const Plan& Scheduler::publish(Assembly& step, PlanKind kind) {
    plan_ = std::move(step.plan);
    plan_.kind = kind;
    if (kind == PlanKind::Idle) return plan_;
    metrics_.steps += 1;
    metrics_.decode_rows += step.decode_rows;
    if (step.decode_rows > 0) metrics_.decode_steps += 1;
    if (kind == PlanKind::Mixed) metrics_.mixed_steps += 1;
    return plan_;
}

// A prompt at the front that no amount of waiting will serve (more pages than
// the pools have in all, or more positions than the model knows) is answered at
// once with an empty result, so that it does not block the queue behind it
// (scheduler.rs:681-690).  The refusal is a step of its own: its commit reports it.
bool Scheduler::turn_away_front() {
    if (waiting_.empty()) return false;
    const size_t prompt_len = waiting_.front().pending.size();
    const size_t most_a_step = chunk_ > 0 ? chunk_ : prompt_len;
    const bool too_long = max_positions_ > 0 && prompt_len > max_positions_;
    if (!too_long && cache_->fits_in_total(prompt_len, most_a_step)) return false;
    Sequence s = std::move(waiting_.front());
    waiting_.pop_front();
    plan_ = Plan{};
    plan_.kind = PlanKind::Refused;
    plan_.refused = s.id;
    outcome_pending_refusal_ = FinishedInfo{s.id, Finish::Length, s.prompt_tokens, s.generated, s.preemptions};
    return true;
}

std::optional<size_t> Scheduler::newest_other_than(size_t keep) const {
    for (size_t i = running_.size(); i-- > 0;)
        if (i != keep && running_[i].finish == Finish::None) return i;
    return std::nullopt;
}

// A resident gives everything back and queues again at the front; when its turn
// comes it is fed its whole history, prompt and output so far, as a prompt, so
// the tokens it has already returned stay returned (scheduler.rs:700-712).
void Scheduler::evict(size_t index) {
    Sequence s = std::move(running_[index]);
    running_.erase(running_.begin() + static_cast<long>(index));
    cache_->free_sequence(s.id);
    s.state_slot = -1;
    s.pending = s.history;
    s.prompt_left = 0;
    s.preemptions += 1;
    metrics_.preemptions += 1;
    metrics_.recomputed_tokens += s.history.size();
    waiting_.push_front(std::move(s));
}

// The planned step is queued on the device.  Its rows' tokens are in the pages for
// everything that runs behind it: the lengths move, and pages that filled up get
// their names for the prefix cache (as far as the history names their tokens: a
// token that was fed on the device joins the history only at the commit of the
// step that chose it, and its page is named at the commit after).
void Scheduler::launched() {
    if (plan_.launched) return;
    plan_.launched = true;
    for (const auto& [id, written] : plan_.advanced) {
        Sequence* s = sequence(id);
        if (!s) continue;       // ended by a stop token of the step before, or cancelled
        cache_->advance(id, written);
        s->prompt_left = s->prompt_left > written ? s->prompt_left - written : 0;
        cache_->publish_full(id, s->history.data(), s->history.size());
    }
}

// The step behind a launched decoding step: a row for every request of that step
// which it cannot end but by a stop token, fed the token of its row there.
const Plan* Scheduler::plan_ahead() {
    if (ahead_) throw Error("a step is planned ahead already");
    if (plan_.kind != PlanKind::Decode || !plan_.launched || prompt_in_flight()) return nullptr;
    // Would the planner bring the front of the queue in (or turn it away)?  Then the next step is its to decide.
    // Whether there is room is asked where the planner asks: before the residents take their pages when prompts
    // run whole, after them under a token budget.
    // Nothing is taken from the pools before the step is known to stand: a plan given up half way would leave
    // its pages with the residents a step early, and the planner would then find less room for the queue's front
    // than it finds without steps planned ahead.
    const size_t groups = cache_->num_groups();
    std::vector<size_t> need(groups, 0);                          // pages the rows seated so far take, a group
    auto room_left = [&]() -> size_t {                            // (what min_available() will say once they have them)
        size_t least = SIZE_MAX;
        for (size_t g = 0; g < groups; ++g) {
            const size_t free_now = cache_->pool(g).available();
            least = std::min(least, free_now > need[g] ? free_now - need[g] : 0);
        }
        return least;
    };
    bool stalled = false;
    auto front_stalls = [&]() -> bool {
        if (waiting_.empty()) return true;
        const size_t prompt_len = waiting_.front().pending.size();
        const bool too_long = max_positions_ > 0 && prompt_len > max_positions_;
        if (too_long || !cache_->fits_in_total(prompt_len, chunk_ > 0 ? chunk_ : prompt_len)) return false;   // a refusal
        const bool room = chunk_ > 0 ? room_left() > 0 : cache_->fits_from_scratch(prompt_len);
        if (room && cache_->state_slot_available()) return false;
        stalled = true;
        return true;
    };
    if (chunk_ == 0 && !front_stalls()) return nullptr;
    // A row for every resident with a token to feed, in the order of arrival, as far as the rows last (as the
    // planner seats them): the token of its row in the launched step, which is not known yet, or, for a resident
    // that step had no row for, the token it has been holding.
    std::vector<std::pair<Sequence*, int>> seated;
    for (Sequence& s : running_) {
        if (seated.size() == max_batch_) break;
        if (s.finish != Finish::None) continue;                  // (leaves at the commit)
        if (s.pending.size() != 1) return nullptr;
        const auto at = std::find(plan_.ids.begin(), plan_.ids.end(), s.id);
        const int fed = at == plan_.ids.end() ? -1 : static_cast<int>(at - plan_.ids.begin());
        if (fed >= 0) {
            const bool last_token = s.generated + 1 >= s.max_tokens;
            const bool last_position = max_positions_ > 0 && s.history.size() + 1 > max_positions_;
            if (last_token || last_position) {
                // It leaves at the commit and its pages with it: a queue that stalls now may not stall then, and
                // bringing the front in is the planner's step.
                if (!waiting_.empty()) return nullptr;
                continue;
            }
        }
        for (size_t g = 0; g < groups; ++g) {
            need[g] += cache_->blocks_needed_in(s.id, g, 1);
            if (need[g] > cache_->pool(g).available()) return nullptr;   // who gives way is the planner's decision
        }
        seated.emplace_back(&s, fed);
    }
    if (seated.empty()) return nullptr;
    if (chunk_ > 0 && !front_stalls()) return nullptr;
    Plan next;
    next.kind = PlanKind::Decode;
    for (const auto& [seq, fed] : seated) {
        Sequence& s = *seq;
        if (!cache_->reserve(s.id, 1)) throw Error("a step planned ahead found no page where it had counted one");
        const size_t first = cache_->tokens(s.id);
        next.ids.push_back(s.id);
        next.advanced.emplace_back(s.id, 1);
        next.entries.push_back(PlanEntry{s.id, first, std::vector<uint32_t>(1, fed >= 0 ? 0u : s.history[first]), true,
                                         s.state_slot, false});
        next.fed_rows.push_back(fed);
    }
    if (stalled) metrics_.admission_stalls += 1;
    metrics_.steps += 1;
    metrics_.decode_steps += 1;
    metrics_.decode_rows += next.entries.size();
    next.stalled = stalled;
    ahead_ = std::move(next);
    return &*ahead_;
}

void Scheduler::drop_ahead() {
    if (!ahead_) return;
    metrics_.steps -= 1;
    metrics_.decode_steps -= 1;
    metrics_.decode_rows -= ahead_->entries.size();
    if (ahead_->stalled) metrics_.admission_stalls -= 1;
    ahead_.reset();           // (the pages reserved for its rows stay with their requests, whose next step needs them)
}

void Scheduler::abandon() {
    drop_ahead();
    plan_ = Plan{};
}

// The step ran.  The sampled tokens join their requests' histories and become
// what the next step feeds; requests that hit a stop token, their budget or the
// model's last position are retired (scheduler.rs:717-764).  A token for a
// request that is no longer there (a row of a step planned ahead, whose request
// the step before ended) is dropped.  The step planned ahead, if there is one,
// becomes the planned step.
const Outcome& Scheduler::commit(const std::vector<uint32_t>& sampled) {
    outcome_ = Outcome{};
    launched();
    const size_t count = std::min(plan_.ids.size(), sampled.size());
    for (size_t i = 0; i < count; ++i) {
        Sequence* s = sequence(plan_.ids[i]);
        if (!s) continue;
        const uint32_t token = sampled[i];
        s->pending.assign(1, token);
        s->history.push_back(token);
        s->generated += 1;
        metrics_.tokens += 1;
        if (std::find(s->stop_tokens.begin(), s->stop_tokens.end(), token) != s->stop_tokens.end()) {
            s->finish = Finish::Stop;  // the stop token is not part of the output
        } else {
            outcome_.tokens.emplace_back(s->id, token);
            if (s->generated >= s->max_tokens) s->finish = Finish::Length;
            // Feeding this token would put it at position history-1, which has to
            // be one the model knows.  (Not checked by the reference.)
            else if (max_positions_ > 0 && s->history.size() > max_positions_) s->finish = Finish::Length;
        }
    }
    if (plan_.kind == PlanKind::Refused && outcome_pending_refusal_) {
        outcome_.finished.push_back(*outcome_pending_refusal_);
        outcome_pending_refusal_.reset();
    }
    retire(outcome_);
    if (ahead_) {
        plan_ = std::move(*ahead_);
        ahead_.reset();
    } else {
        plan_ = Plan{};
    }
    return outcome_;
}

void Scheduler::cancel(uint64_t id) {
    for (auto it = waiting_.begin(); it != waiting_.end(); ++it) {
        if (it->id == id) {
            waiting_.erase(it);
            return;
        }
    }
    if (Sequence* s = sequence(id)) s->finish = Finish::Stop;
    Outcome dropped;
    retire(dropped);
}

// Finished requests leave the running set and their pages return to the pools (scheduler.rs:782-793).
void Scheduler::retire(Outcome& outcome) {
    size_t index = 0;
    while (index < running_.size()) {
        if (running_[index].finish == Finish::None) {
            ++index;
            continue;
        }
        Sequence s = std::move(running_[index]);
        running_.erase(running_.begin() + static_cast<long>(index));
        cache_->free_sequence(s.id);
        outcome.finished.push_back(FinishedInfo{s.id, s.finish, s.prompt_tokens, s.generated, s.preemptions});
    }
}

const Outcome& Scheduler::drain_finished() {
    outcome_ = Outcome{};
    retire(outcome_);
    return outcome_;
}

}  // namespace pl
