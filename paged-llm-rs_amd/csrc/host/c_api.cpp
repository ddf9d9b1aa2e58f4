// The C interface of the host runtime.  Every call returns 0 (or a count) on
// success and a negative number on failure; the message is read with
// plh_last_error().  Handles are opaque pointers.
#include <algorithm>
#include <cstring>
#include <string>

#include "cache.hpp"
#include "sampler.hpp"
#include "scheduler.hpp"

using namespace pl;

static thread_local std::string g_error;

template <typename F>
static long guarded(F&& f) {
    try {
        return f();
    } catch (const std::exception& e) {
        g_error = e.what();
        return -1;
    }
}

extern "C" {

const char* plh_last_error() { return g_error.c_str(); }
int plh_abi_version() { return 1; }

uint64_t plh_block_hash(int has_parent, uint64_t parent, const uint32_t* tokens, size_t count) {
    return block_hash(has_parent != 0, parent, tokens, count);
}

// ---- one pool ---------------------------------------------------------------
void* plh_pool_create(size_t total) { return new BlockPool(total); }
void plh_pool_destroy(void* p) { delete static_cast<BlockPool*>(p); }
int plh_pool_allocate(void* p) { return static_cast<BlockPool*>(p)->allocate(); }
int plh_pool_acquire_cached(void* p, uint64_t hash) { return static_cast<BlockPool*>(p)->acquire_cached(hash); }
void plh_pool_publish(void* p, int block, uint64_t hash) { static_cast<BlockPool*>(p)->publish(block, hash); }
long plh_pool_release(void* p, int block) {
    return guarded([&] { static_cast<BlockPool*>(p)->release(block); return 0L; });
}
void plh_pool_clear_cache(void* p) { static_cast<BlockPool*>(p)->clear_cache(); }
// which: 0 available, 1 total, 2 in_use, 3 cached_blocks, 4 handed_out, 5 hits, 6 misses, 7 evictions
static uint64_t pool_counter(const BlockPool& pool, int which) {
    switch (which) {
        case 0: return pool.available();
        case 1: return pool.total();
        case 2: return pool.in_use();
        case 3: return pool.cached_blocks();
        case 4: return pool.handed_out();
        case 5: return pool.hits();
        case 6: return pool.misses();
        case 7: return pool.evictions();
    }
    return 0;
}
uint64_t plh_pool_counter(void* p, int which) { return pool_counter(*static_cast<BlockPool*>(p), which); }

// ---- the cache manager ------------------------------------------------------
void* plh_cache_create(int groups, const int* block_size, const int* num_blocks, const int* window, int state_slots) {
    try {
        std::vector<GroupSpec> specs;
        for (int g = 0; g < groups; ++g) specs.push_back(GroupSpec{block_size[g], num_blocks[g], window[g]});
        return new CacheManager(std::move(specs), state_slots);
    } catch (const std::exception& e) {
        g_error = e.what();
        return nullptr;
    }
}
void plh_cache_destroy(void* c) { delete static_cast<CacheManager*>(c); }
long plh_cache_add_sequence(void* c, uint64_t id) {
    try {
        return static_cast<CacheManager*>(c)->add_sequence(id);
    } catch (const std::exception& e) {
        g_error = e.what();
        return -2;
    }
}
void plh_cache_free_sequence(void* c, uint64_t id) { static_cast<CacheManager*>(c)->free_sequence(id); }
int plh_cache_has(void* c, uint64_t id) { return static_cast<CacheManager*>(c)->has(id) ? 1 : 0; }
long plh_cache_tokens(void* c, uint64_t id) {
    return guarded([&] { return static_cast<long>(static_cast<CacheManager*>(c)->tokens(id)); });
}
long plh_cache_capacity(void* c, uint64_t id) {
    return guarded([&] { return static_cast<long>(static_cast<CacheManager*>(c)->capacity(id)); });
}
long plh_cache_blocks_needed(void* c, uint64_t id, size_t count) {
    return guarded([&] { return static_cast<long>(static_cast<CacheManager*>(c)->blocks_needed(id, count)); });
}
long plh_cache_reserve(void* c, uint64_t id, size_t count) {
    return guarded([&] { return static_cast<CacheManager*>(c)->reserve(id, count) ? 1L : 0L; });
}
long plh_cache_reserve_up_to(void* c, uint64_t id, size_t count) {
    return guarded([&] { return static_cast<long>(static_cast<CacheManager*>(c)->reserve_up_to(id, count)); });
}
long plh_cache_advance(void* c, uint64_t id, size_t count) {
    return guarded([&] { static_cast<CacheManager*>(c)->advance(id, count); return 0L; });
}
long plh_cache_slot_of(void* c, uint64_t id, size_t group, size_t position) {
    try {
        return static_cast<CacheManager*>(c)->slot_of(id, group, position);
    } catch (const std::exception& e) {
        g_error = e.what();
        return -2;
    }
}
long plh_cache_claim_prefix(void* c, uint64_t id, const uint32_t* prompt, size_t length) {
    return guarded([&] { return static_cast<long>(static_cast<CacheManager*>(c)->claim_prefix(id, prompt, length)); });
}
long plh_cache_publish_full(void* c, uint64_t id, const uint32_t* history, size_t length) {
    return guarded([&] { static_cast<CacheManager*>(c)->publish_full(id, history, length); return 0L; });
}
void plh_cache_set_prefix_cache(void* c, int enabled) { static_cast<CacheManager*>(c)->set_prefix_cache(enabled != 0); }
int plh_cache_sharing_possible(void* c) { return static_cast<CacheManager*>(c)->sharing_possible() ? 1 : 0; }
// Writes the logical page list of one group (-1 where the window has passed);
// returns its length, or a negative number when `cap` is too small or the id unknown.
long plh_cache_table(void* c, uint64_t id, size_t group, int* out, size_t cap) {
    return guarded([&] {
        const auto& blocks = static_cast<CacheManager*>(c)->table(id).blocks.at(group);
        if (blocks.size() > cap) throw Error("a table of " + std::to_string(blocks.size()) + " pages for room of " + std::to_string(cap));
        std::memcpy(out, blocks.data(), blocks.size() * sizeof(int));
        return static_cast<long>(blocks.size());
    });
}
// For a step of n requests: positions[i] = tokens the cache holds of request i (where its next
// token goes), and row i of `tables` (n rows of `width`, -1 beyond a request's pages) for one group.
// Returns 0, or the number of pages of the longest table when that is more than `width`.
// Either output may be null.
long plh_cache_fill_step(void* c, size_t n, const uint64_t* ids, int* positions, size_t group, int* tables,
                         size_t width) {
    return guarded([&] {
        auto* cache = static_cast<CacheManager*>(c);
        size_t widest = 0;
        for (size_t i = 0; i < n; ++i) {
            const SequenceTable& t = cache->table(ids[i]);
            if (t.tokens + 1 > cache->capacity(ids[i]))
                throw Error("request " + std::to_string(ids[i]) + " has no block for position " + std::to_string(t.tokens));
            if (positions) positions[i] = static_cast<int>(t.tokens);
            if (tables) widest = std::max(widest, t.blocks.at(group).size());
        }
        if (tables && widest > width) return static_cast<long>(widest);   // nothing is written: the rows need more room
        for (size_t i = 0; tables && i < n; ++i) {
            const auto& blocks = cache->table(ids[i]).blocks.at(group);
            int* row = tables + i * width;
            std::memcpy(row, blocks.data(), blocks.size() * sizeof(int));
            for (size_t b = blocks.size(); b < width; ++b) row[b] = -1;
        }
        return 0L;
    });
}
long plh_cache_table_len(void* c, uint64_t id, size_t group) {
    return guarded([&] { return static_cast<long>(static_cast<CacheManager*>(c)->table(id).blocks.at(group).size()); });
}
long plh_cache_state_slot(void* c, uint64_t id) {
    try {
        return static_cast<CacheManager*>(c)->table(id).state_slot;
    } catch (const std::exception& e) {
        g_error = e.what();
        return -2;
    }
}
long plh_cache_wasted_tokens(void* c, uint64_t id) {
    return guarded([&] { return static_cast<long>(static_cast<CacheManager*>(c)->wasted_tokens(id)); });
}
uint64_t plh_cache_counter(void* c, size_t group, int which) {
    return pool_counter(static_cast<CacheManager*>(c)->pool(group), which);
}
long plh_cache_live_sequences(void* c) { return static_cast<long>(static_cast<CacheManager*>(c)->live_sequences()); }
int plh_cache_free_state_slots(void* c) { return static_cast<CacheManager*>(c)->free_state_slots(); }
long plh_cache_holders(void* c, size_t group, int block) {
    return guarded([&] { return static_cast<long>(static_cast<CacheManager*>(c)->pool(group).holders(block)); });
}

// ---- the sampler ------------------------------------------------------------
uint64_t plh_rng_next_u64(uint64_t* state) {
    Rng rng(*state);
    const uint64_t v = rng.next_u64();
    *state = rng.state;
    return v;
}
float plh_rng_next_f32(uint64_t* state) {
    Rng rng(*state);
    const float v = rng.next_f32();
    *state = rng.state;
    return v;
}
const char* plh_sampling_problem(float temperature, int has_top_k, long top_k, int has_top_p, float top_p) {
    return sampling_problem(temperature, has_top_k, top_k, has_top_p, top_p);
}
long plh_sample(float temperature, int top_k, float top_p, const float* logits, size_t count, uint64_t* rng_state) {
    if (count == 0) {
        g_error = "cannot sample from an empty logit vector";
        return -1;
    }
    Sampling how{temperature, top_k, top_p};
    Rng rng(*rng_state);
    const uint32_t token = sample(how, logits, count, rng);
    *rng_state = rng.state;
    return token;
}

// ---- the scheduler ----------------------------------------------------------
void* plh_sched_create(void* cache, size_t max_batch, size_t chunk, size_t max_positions) {
    return new Scheduler(static_cast<CacheManager*>(cache), max_batch, chunk, max_positions);
}
void plh_sched_destroy(void* s) { delete static_cast<Scheduler*>(s); }
void plh_sched_set_chunk(void* s, size_t chunk) { static_cast<Scheduler*>(s)->set_chunk(chunk); }
void plh_sched_set_prefix_cache(void* s, int enabled) { static_cast<Scheduler*>(s)->set_prefix_cache(enabled != 0); }

long plh_sched_submit(void* s, uint64_t id, const uint32_t* prompt, size_t length, float temperature,
                      int has_top_k, long top_k, int has_top_p, float top_p, size_t max_tokens,
                      const uint32_t* stop, size_t stops, uint64_t seed) {
    return guarded([&] {
        const char* problem = sampling_problem(temperature, has_top_k, top_k, has_top_p, top_p);
        if (problem[0]) throw Error(problem);
        Sequence q;
        q.id = id;
        q.history.assign(prompt, prompt + length);
        q.sampling = Sampling{temperature, has_top_k ? static_cast<int>(std::min<long>(top_k, 1L << 30)) : 0,
                              has_top_p ? top_p : 1.f};
        q.max_tokens = max_tokens;
        q.stop_tokens.assign(stop, stop + stops);
        q.rng = Rng(seed);
        static_cast<Scheduler*>(s)->submit(std::move(q));
        return 0L;
    });
}

static void plan_sizes(const Plan& p, size_t* sizes) {
    size_t tokens = 0;
    for (const PlanEntry& e : p.entries) tokens += e.tokens.size();
    sizes[0] = p.entries.size();
    sizes[1] = tokens;
    sizes[2] = p.ids.size();
    sizes[3] = p.advanced.size();
}

static void plan_read(const Plan& p, uint64_t* entry_id, int* entry_start, int* entry_len, int* entry_wants,
                      int* entry_state_slot, int* entry_fresh, int* entry_fed_row, uint32_t* tokens, uint64_t* ids,
                      uint64_t* advanced_id, int* advanced_count, uint64_t* refused) {
    size_t at = 0;
    for (size_t i = 0; i < p.entries.size(); ++i) {
        const PlanEntry& e = p.entries[i];
        entry_id[i] = e.id;
        entry_start[i] = static_cast<int>(e.start);
        entry_len[i] = static_cast<int>(e.tokens.size());
        entry_wants[i] = e.wants_logits ? 1 : 0;
        entry_state_slot[i] = e.state_slot;
        entry_fresh[i] = e.state_fresh ? 1 : 0;
        entry_fed_row[i] = i < p.fed_rows.size() ? p.fed_rows[i] : -1;
        std::memcpy(tokens + at, e.tokens.data(), e.tokens.size() * sizeof(uint32_t));
        at += e.tokens.size();
    }
    for (size_t i = 0; i < p.ids.size(); ++i) ids[i] = p.ids[i];
    for (size_t i = 0; i < p.advanced.size(); ++i) {
        advanced_id[i] = p.advanced[i].first;
        advanced_count[i] = static_cast<int>(p.advanced[i].second);
    }
    *refused = p.refused;
}

// Decides the next step and keeps it; returns its kind.  sizes: entries, tokens
// (all entries together), ids, advanced.
long plh_sched_plan(void* s, size_t* sizes) {
    return guarded([&] {
        const Plan& p = static_cast<Scheduler*>(s)->plan();
        plan_sizes(p, sizes);
        return static_cast<long>(p.kind);
    });
}

// Reads the planned step; `which` 1 reads the step planned ahead instead.
void plh_sched_plan_read(void* s, int which, uint64_t* entry_id, int* entry_start, int* entry_len, int* entry_wants,
                         int* entry_state_slot, int* entry_fresh, int* entry_fed_row, uint32_t* tokens,
                         uint64_t* ids, uint64_t* advanced_id, int* advanced_count, uint64_t* refused) {
    const Scheduler* q = static_cast<Scheduler*>(s);
    const Plan* p = which == 1 ? q->ahead() : &q->last_plan();
    if (!p) return;
    plan_read(*p, entry_id, entry_start, entry_len, entry_wants, entry_state_slot, entry_fresh, entry_fed_row,
              tokens, ids, advanced_id, advanced_count, refused);
}

// The planned step is queued on the device: the lengths in the cache move.
long plh_sched_launched(void* s) {
    return guarded([&] { static_cast<Scheduler*>(s)->launched(); return 0L; });
}
// Plans the step behind the launched one, if it can be known: 1 and its sizes, else 0.
long plh_sched_plan_ahead(void* s, size_t* sizes) {
    return guarded([&]() -> long {
        const Plan* p = static_cast<Scheduler*>(s)->plan_ahead();
        if (!p) return 0L;
        plan_sizes(*p, sizes);
        return 1L;
    });
}
void plh_sched_drop_ahead(void* s) { static_cast<Scheduler*>(s)->drop_ahead(); }
void plh_sched_abandon(void* s) { static_cast<Scheduler*>(s)->abandon(); }
static void read_outcome_sizes(const Outcome& o, size_t* sizes) {
    sizes[0] = o.tokens.size();
    sizes[1] = o.finished.size();
}

long plh_sched_commit(void* s, const uint32_t* sampled, size_t count, size_t* sizes) {
    return guarded([&] {
        const Outcome& o = static_cast<Scheduler*>(s)->commit(std::vector<uint32_t>(sampled, sampled + count));
        read_outcome_sizes(o, sizes);
        return 0L;
    });
}
long plh_sched_drain_finished(void* s, size_t* sizes) {
    return guarded([&] {
        read_outcome_sizes(static_cast<Scheduler*>(s)->drain_finished(), sizes);
        return 0L;
    });
}
// Reads the outcome of the last commit or drain.
void plh_sched_outcome_read(void* s, uint64_t* token_id, uint32_t* token, uint64_t* finished_id, int* finish,
                            uint64_t* prompt_tokens, uint64_t* generated, uint32_t* preemptions) {
    const Outcome& o = static_cast<Scheduler*>(s)->last_outcome();
    for (size_t i = 0; i < o.tokens.size(); ++i) {
        token_id[i] = o.tokens[i].first;
        token[i] = o.tokens[i].second;
    }
    for (size_t i = 0; i < o.finished.size(); ++i) {
        finished_id[i] = o.finished[i].id;
        finish[i] = static_cast<int>(o.finished[i].finish);
        prompt_tokens[i] = o.finished[i].prompt_tokens;
        generated[i] = o.finished[i].generated;
        preemptions[i] = o.finished[i].preemptions;
    }
}
long plh_sched_cancel(void* s, uint64_t id) {
    return guarded([&] { static_cast<Scheduler*>(s)->cancel(id); return 0L; });
}
size_t plh_sched_waiting(void* s) { return static_cast<Scheduler*>(s)->waiting(); }
size_t plh_sched_running(void* s) { return static_cast<Scheduler*>(s)->running(); }
size_t plh_sched_running_ids(void* s, uint64_t* out, size_t cap) {
    const auto ids = static_cast<Scheduler*>(s)->running_ids();
    for (size_t i = 0; i < ids.size() && i < cap; ++i) out[i] = ids[i];
    return ids.size();
}
size_t plh_sched_wasted_tokens(void* s) { return static_cast<Scheduler*>(s)->wasted_tokens(); }
// steps, prefills, tokens, decode_rows, admission_stalls, preemptions, mixed_steps,
// decode_steps, recomputed_tokens, cached_tokens, prefilled_tokens
void plh_sched_metrics(void* s, uint64_t* out) {
    const Metrics& m = static_cast<Scheduler*>(s)->metrics();
    const uint64_t values[11] = {m.steps, m.prefills, m.tokens, m.decode_rows, m.admission_stalls, m.preemptions,
                                 m.mixed_steps, m.decode_steps, m.recomputed_tokens, m.cached_tokens, m.prefilled_tokens};
    std::memcpy(out, values, sizeof(values));
}
// Host sampling for one request with its own parameters and generator.
long plh_sched_sample(void* s, uint64_t id, const float* logits, size_t count) {
    return guarded([&]() -> long {
        if (count == 0) throw Error("cannot sample from an empty logit vector");
        Sequence* q = static_cast<Scheduler*>(s)->sequence(id);
        if (!q) throw Error("request " + std::to_string(id) + " left while its step was running");
        return sample(q->sampling, logits, count, q->rng);
    });
}
// What a device sampler needs for one request: its parameters, and (for a
// request that draws) the next number of its generator.  Greedy never moves it.
long plh_sched_sampling_of(void* s, uint64_t id, float* temperature, int* top_k, float* top_p, float* uniform) {
    return guarded([&]() -> long {
        Sequence* q = static_cast<Scheduler*>(s)->sequence(id);
        if (!q) throw Error("request " + std::to_string(id) + " left while its step was running");
        *temperature = q->sampling.temperature;
        *top_k = q->sampling.top_k;
        *top_p = q->sampling.top_p;
        *uniform = q->sampling.greedy() ? 0.f : q->rng.next_f32();
        return 0;
    });
}

}  // extern "C"
