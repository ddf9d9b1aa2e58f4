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

PlanEntry Scheduler::entry_for(Sequence& s, size_t start, std::vector<uint32_t> tokens, bool wants) {
    PlanEntry e{s.id, start, std::move(tokens), wants, s.state_slot, s.state_fresh};
    s.state_fresh = false;
    return e;
}

// Refuse first, then (with a budget) a mixed step or else a plain decode, or
// (without one) a whole prompt or else a plain decode (scheduler.rs:368-381).
const Plan& Scheduler::plan() {
    if (auto refused = refuse_unservable()) {
        plan_ = std::move(*refused);
        return plan_;
    }
    if (chunk_ > 0) {
        if (auto step = mixed()) {
            plan_ = std::move(*step);
            return plan_;
        }
        plan_ = decode();
        return plan_;
    }
    if (auto step = admit()) {
        plan_ = std::move(*step);
        return plan_;
    }
    plan_ = decode();
    return plan_;
}

// One step carrying a portion of a prompt and every running request's next
// token (scheduler.rs:388-499).
std::optional<Plan> Scheduler::mixed() {
    const size_t budget = chunk_;
    // A prompt part-way through finishes before a new one starts.
    std::optional<size_t> index = prompt_in_flight();

    Plan step;
    step.kind = PlanKind::Mixed;
    // Decodes are taken first: they are what a client is watching.
    const size_t cap = std::min(max_batch_, budget);
    for (size_t row = 0; row < running_.size(); ++row) {
        if (step.entries.size() >= cap) break;
        Sequence& s = running_[row];
        if ((index && row == *index) || s.finish != Finish::None || s.pending.size() != 1) continue;
        if (!cache_->reserve(s.id, 1)) {
            // A resident that needs a page from a dry pool is a preemption, and
            // choosing the victim is the plain decode's job.  Give the step up
            // rather than run without this request.
            return std::nullopt;
        }
        step.ids.push_back(s.id);
        step.advanced.emplace_back(s.id, 1);
        step.entries.push_back(entry_for(s, cache_->tokens(s.id), {s.pending[0]}, true));
    }
    const size_t decodes = step.entries.size();

    // Whatever the decodes left goes to the prompt in flight; and where that prompt ends within the budget,
    // to the next waiting ones, as long as tokens and rows are left.  (The reference's step carries a slice
    // of one prompt; short prompts then enter one a step however large the budget, and a batch takes as many
    // steps to fill as it has requests.)  At most one prompt is left part-way by a step, so the next step
    // finds one prompt in flight, as the reference's does.
    size_t room = budget > decodes ? budget - decodes : 0;
    if (room == 0) return std::nullopt;
    bool any = false;
    while (room > 0 && (!any || step.entries.size() < cap)) {
        // A new prompt joins only now, after the residents have taken their pages.
        if (!index) {
            const size_t before = running_.size();
            start_next_prompt();
            if (running_.size() == before) break;
            index = before;
        }
        Sequence& s = running_[*index];
        const size_t done = s.history.size() - s.prompt_left;
        const size_t want = std::min(room, s.prompt_left);
        const size_t take = cache_->reserve_up_to(s.id, want);
        if (take == 0) break;
        const bool last = take == s.prompt_left;
        if (last) step.ids.push_back(s.id);  // only the last portion asks for logits
        step.advanced.emplace_back(s.id, take);
        step.entries.push_back(entry_for(
            s, done, std::vector<uint32_t>(s.history.begin() + done, s.history.begin() + done + take), last));
        any = true;
        room -= take;
        if (!last) break;
        index.reset();
    }
    if (!any) return std::nullopt;

    metrics_.steps += 1;
    metrics_.mixed_steps += 1;
    metrics_.decode_rows += decodes;
    if (decodes > 0) metrics_.decode_steps += 1;
    return step;
}

// Move the first waiting request into the running set without running it, so
// that its prompt can be fed a portion at a time (scheduler.rs:503-539).
void Scheduler::start_next_prompt() {
    if (waiting_.empty()) return;
    const size_t prompt_len = waiting_.front().pending.size();
    if (cache_->min_available() == 0 || !cache_->state_slot_available()) {
        metrics_.admission_stalls += 1;
        return;
    }
    Sequence s = std::move(waiting_.front());
    waiting_.pop_front();
    s.state_slot = cache_->add_sequence(s.id);
    s.state_fresh = s.state_slot >= 0;
    const size_t shared = cache_->claim_prefix(s.id, s.pending.data(), s.pending.size());
    // Claiming takes pages of its own, and a request whose whole prefix was
    // resident still needs somewhere to write the token it is about to produce.
    if (!cache_->reserve(s.id, 1)) {
        cache_->free_sequence(s.id);
        s.state_slot = -1;
        s.pending = s.history;
        waiting_.push_front(std::move(s));
        metrics_.admission_stalls += 1;
        return;
    }
    metrics_.cached_tokens += shared;
    metrics_.prefilled_tokens += prompt_len - shared;
    s.prompt_left = std::max<size_t>(prompt_len - shared, 1);
    s.pending.clear();
    metrics_.prefills += 1;
    running_.push_back(std::move(s));
}

// Give a waiting request its pages and run its whole prompt (scheduler.rs:548-589).
std::optional<Plan> Scheduler::admit() {
    if (waiting_.empty()) return std::nullopt;
    const size_t prompt_len = waiting_.front().pending.size();
    if (!cache_->fits_from_scratch(prompt_len) || !cache_->state_slot_available()) {
        metrics_.admission_stalls += 1;
        return std::nullopt;
    }
    Sequence s = std::move(waiting_.front());
    waiting_.pop_front();
    s.state_slot = cache_->add_sequence(s.id);
    s.state_fresh = s.state_slot >= 0;
    const size_t shared = cache_->claim_prefix(s.id, s.pending.data(), s.pending.size());
    if (!cache_->reserve(s.id, prompt_len - shared)) {
        // The cache gave way and there is still nothing: put it back rather
        // than admit it half served.
        cache_->free_sequence(s.id);
        s.state_slot = -1;
        s.pending = s.history;
        waiting_.push_front(std::move(s));
        metrics_.admission_stalls += 1;
        return std::nullopt;
    }
    metrics_.cached_tokens += shared;
    metrics_.prefilled_tokens += prompt_len - shared;

    Plan step;
    step.kind = PlanKind::Prefill;
    step.ids.push_back(s.id);
    step.advanced.emplace_back(s.id, prompt_len - shared);
    step.entries.push_back(
        entry_for(s, shared, std::vector<uint32_t>(s.pending.begin() + shared, s.pending.end()), true));
    s.pending.clear();
    running_.push_back(std::move(s));
    metrics_.steps += 1;
    metrics_.prefills += 1;
    return step;
}

// Advance every resident request by one token, evicting where the pools
// cannot supply the page one of them needs (scheduler.rs:625-676).
Plan Scheduler::decode() {
    std::vector<size_t> chosen;
    size_t index = 0;
    while (index < running_.size() && chosen.size() < max_batch_) {
        Sequence& s = running_[index];
        if (s.finish != Finish::None || s.pending.size() != 1) {
            ++index;
            continue;
        }
        if (cache_->reserve(s.id, 1)) {
            chosen.push_back(index);
            ++index;
            continue;
        }
        // Nothing left.  Evict the newest resident that is not this one and
        // come back to this request with the pages it freed.
        const auto victim = newest_evictable(index);
        if (!victim) {
            // Alone, and the pools cannot hold its next token: it ends here,
            // or nothing would ever free anything.  (The reference would idle
            // forever at this point.)
            s.finish = Finish::Length;
            ++index;
            continue;
        }
        preempt(*victim);
        chosen.erase(std::remove(chosen.begin(), chosen.end(), *victim), chosen.end());
        for (size_t& taken : chosen)
            if (taken > *victim) --taken;
        if (*victim < index) --index;
    }
    Plan step;
    if (chosen.empty()) return step;  // Idle
    step.kind = PlanKind::Decode;
    for (size_t i : chosen) {
        Sequence& s = running_[i];
        step.ids.push_back(s.id);
        step.advanced.emplace_back(s.id, 1);
        step.entries.push_back(entry_for(s, cache_->tokens(s.id), {s.pending[0]}, true));
    }
    metrics_.steps += 1;
    metrics_.decode_steps += 1;
    metrics_.decode_rows += step.ids.size();
    return step;
}

// Reject a waiting prompt the pools could never hold, or one past the longest
// position the model knows (scheduler.rs:681-690).
std::optional<Plan> Scheduler::refuse_unservable() {
    if (waiting_.empty()) return std::nullopt;
    const size_t prompt_len = waiting_.front().pending.size();
    const size_t budget = chunk_ > 0 ? chunk_ : prompt_len;
    const bool too_long = max_positions_ > 0 && prompt_len > max_positions_;
    if (!too_long && cache_->fits_in_total(prompt_len, budget)) return std::nullopt;
    Sequence s = std::move(waiting_.front());
    waiting_.pop_front();
    Plan step;
    step.kind = PlanKind::Refused;
    step.refused = s.id;
    outcome_pending_refusal_ = FinishedInfo{s.id, Finish::Length, s.prompt_tokens, s.generated, s.preemptions};
    return step;
}

std::optional<size_t> Scheduler::newest_evictable(size_t protect) const {
    for (size_t i = running_.size(); i-- > 0;)
        if (i != protect && running_[i].finish == Finish::None) return i;
    return std::nullopt;
}

// Take a request's pages back and put it at the front of the queue, to be
// recomputed from everything the model has seen (scheduler.rs:700-712).
void Scheduler::preempt(size_t index) {
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

// Record that a step ran: keep its tokens, retire what it finished
// (scheduler.rs:717-764).
const Outcome& Scheduler::commit(const std::vector<uint32_t>& sampled) {
    outcome_ = Outcome{};
    for (const auto& [id, written] : plan_.advanced) {
        Sequence* s = sequence(id);
        if (!s) continue;
        cache_->advance(id, written);
        s->prompt_left = s->prompt_left > written ? s->prompt_left - written : 0;
        // Name whatever this step filled.  Done here rather than in the step,
        // because only now is it known that the tokens are really there.
        cache_->publish_full(id, s->history.data(), s->history.size());
    }
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
    plan_ = Plan{};
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

// Hand every finished request's pages back to the pools (scheduler.rs:782-793).
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
