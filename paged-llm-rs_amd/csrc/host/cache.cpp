#include "cache.hpp"

#include <algorithm>

namespace pl {

BlockHash block_hash(bool has_parent, BlockHash parent, const uint32_t* tokens, size_t count) {
    uint64_t hash = 0xcbf29ce484222325ULL;
    auto mix = [&hash](uint64_t value) {
        for (int i = 0; i < 8; ++i) {
            hash ^= (value >> (8 * i)) & 0xffULL;
            hash *= 0x00000100000001b3ULL;
        }
    };
    // The parent goes in first, so the same tokens after another prefix get another name.
    mix(has_parent ? parent : 0);
    mix(static_cast<uint64_t>(count));
    for (size_t i = 0; i < count; ++i) mix(static_cast<uint64_t>(tokens[i]));
    uint64_t z = hash + 0x9E3779B97F4A7C15ULL;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ULL;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBULL;
    return z ^ (z >> 31);
}

// ---------------------------------------------------------------------------

BlockPool::BlockPool(size_t total) : slots_(total), total_(total) {
    // Taken from the end, so the first page handed out is page zero.
    free_anonymous_.reserve(total);
    for (size_t i = total; i-- > 0;) free_anonymous_.push_back(static_cast<BlockId>(i));
}

BlockId BlockPool::allocate() {
    BlockId block;
    if (!free_anonymous_.empty()) {
        block = free_anonymous_.back();
        free_anonymous_.pop_back();
    } else if (!free_named_.empty()) {
        auto oldest = free_named_.begin();
        block = oldest->second;
        free_named_.erase(oldest);
        ++evictions_;
    } else {
        return kNoBlock;
    }
    forget(block);
    slots_[static_cast<size_t>(block)].holders = 1;
    ++handed_out_;
    return block;
}

BlockId BlockPool::acquire_cached(BlockHash hash) {
    auto found = cached_.find(hash);
    if (found == cached_.end()) return kNoBlock;
    const BlockId block = found->second;
    Slot& slot = slots_[static_cast<size_t>(block)];
    if (slot.holders == 0) {
        // Resident but unheld: no longer a candidate for eviction while somebody reads it.
        free_named_.erase(slot.released_at);
    }
    ++slot.holders;
    ++hits_;
    return block;
}

void BlockPool::publish(BlockId block, BlockHash hash) {
    auto found = cached_.find(hash);
    if (found != cached_.end() && found->second != block) {
        // Another request filled the same prefix first; its page keeps the name.
        return;
    }
    Slot& slot = slots_.at(static_cast<size_t>(block));
    if (slot.named && slot.hash != hash) forget(block);
    slot.named = true;
    slot.hash = hash;
    cached_[hash] = block;
}

void BlockPool::release(BlockId block) {
    if (block < 0 || static_cast<size_t>(block) >= slots_.size())
        throw Error("page " + std::to_string(block) + " released, which the pool does not hold");
    Slot& slot = slots_[static_cast<size_t>(block)];
    if (slot.holders == 0)
        throw Error("page " + std::to_string(block) + " released more often than it was taken");
    if (--slot.holders == 0) {
        slot.released_at = ++clock_;
        if (slot.named)
            free_named_[slot.released_at] = block;
        else
            free_anonymous_.push_back(block);
    }
}

void BlockPool::clear_cache() {
    for (Slot& slot : slots_) slot.named = false;
    cached_.clear();
    // Oldest first, so the page released last is the next one taken.
    for (auto& entry : free_named_) free_anonymous_.push_back(entry.second);
    free_named_.clear();
}

void BlockPool::forget(BlockId block) {
    Slot& slot = slots_[static_cast<size_t>(block)];
    if (!slot.named) return;
    slot.named = false;
    auto found = cached_.find(slot.hash);
    if (found != cached_.end() && found->second == block) cached_.erase(found);
}

// ---------------------------------------------------------------------------

CacheManager::CacheManager(std::vector<GroupSpec> groups, int state_slots)
    : groups_(std::move(groups)), state_slots_(state_slots) {
    if (groups_.empty() && state_slots_ <= 0)
        throw Error("a cache with neither pages nor state slots");
    for (const GroupSpec& g : groups_) {
        if (g.block_size < 1) throw Error("block size " + std::to_string(g.block_size) + ", which has to be at least one");
        if (g.num_blocks < 1) throw Error("a pool of " + std::to_string(g.num_blocks) + " pages");
        if (g.window < 0) throw Error("window " + std::to_string(g.window));
        pools_.emplace_back(static_cast<size_t>(g.num_blocks));
    }
    if (state_slots_ < 0) state_slots_ = 0;
    for (int i = state_slots_; i-- > 0;) free_state_slots_.push_back(i);
}

bool CacheManager::sharing_possible() const {
    if (groups_.empty() || state_slots_ > 0) return false;
    for (const GroupSpec& g : groups_)
        if (g.window != 0 || g.block_size != groups_[0].block_size) return false;
    return true;
}

void CacheManager::set_prefix_cache(bool enabled) {
    prefix_cache_ = enabled;
    if (!enabled)
        for (BlockPool& p : pools_) p.clear_cache();
}

int CacheManager::add_sequence(uint64_t id) {
    if (tables_.count(id)) throw Error("request " + std::to_string(id) + " is already resident");
    SequenceTable t;
    t.blocks.resize(groups_.size());
    if (state_slots_ > 0) {
        if (free_state_slots_.empty()) throw Error("no state slot is free");
        t.state_slot = free_state_slots_.back();
        free_state_slots_.pop_back();
    }
    const int slot = t.state_slot;
    tables_.emplace(id, std::move(t));
    return slot;
}

void CacheManager::free_sequence(uint64_t id) {
    auto found = tables_.find(id);
    if (found == tables_.end()) return;
    SequenceTable& t = found->second;
    for (size_t g = 0; g < groups_.size(); ++g)
        for (BlockId b : t.blocks[g])
            if (b != kNoBlock) pools_[g].release(b);
    if (t.state_slot >= 0) free_state_slots_.push_back(t.state_slot);
    tables_.erase(found);
}

const SequenceTable& CacheManager::table(uint64_t id) const {
    auto found = tables_.find(id);
    if (found == tables_.end()) throw Error("request " + std::to_string(id) + " is not resident");
    return found->second;
}

SequenceTable& CacheManager::table_mut(uint64_t id) {
    auto found = tables_.find(id);
    if (found == tables_.end()) throw Error("request " + std::to_string(id) + " is not resident");
    return found->second;
}

size_t CacheManager::capacity(uint64_t id) const {
    const SequenceTable& t = table(id);
    if (groups_.empty()) return SIZE_MAX;
    size_t least = SIZE_MAX;
    for (size_t g = 0; g < groups_.size(); ++g)
        least = std::min(least, t.blocks[g].size() * static_cast<size_t>(groups_[g].block_size));
    return least;
}

size_t CacheManager::needed_in_group(const SequenceTable& t, size_t g, size_t count) const {
    const size_t bs = static_cast<size_t>(groups_[g].block_size);
    const size_t wanted = t.tokens + count;
    const size_t have = t.blocks[g].size() * bs;
    if (wanted <= have) return 0;
    return (wanted - have + bs - 1) / bs;
}

size_t CacheManager::blocks_needed(uint64_t id, size_t count) const {
    const SequenceTable& t = table(id);
    size_t most = 0;
    for (size_t g = 0; g < groups_.size(); ++g) most = std::max(most, needed_in_group(t, g, count));
    return most;
}

bool CacheManager::reserve(uint64_t id, size_t count) {
    SequenceTable& t = table_mut(id);
    for (size_t g = 0; g < groups_.size(); ++g)
        if (needed_in_group(t, g, count) > pools_[g].available()) return false;
    for (size_t g = 0; g < groups_.size(); ++g) {
        const size_t need = needed_in_group(t, g, count);
        for (size_t i = 0; i < need; ++i) t.blocks[g].push_back(pools_[g].allocate());
    }
    return true;
}

size_t CacheManager::reserve_up_to(uint64_t id, size_t count) {
    SequenceTable& t = table_mut(id);
    for (size_t g = 0; g < groups_.size(); ++g) {
        const size_t need = needed_in_group(t, g, count);
        for (size_t i = 0; i < need; ++i) {
            const BlockId b = pools_[g].allocate();
            if (b == kNoBlock) break;
            t.blocks[g].push_back(b);
        }
    }
    const size_t cap = capacity(id);
    return std::min(count, cap > t.tokens ? cap - t.tokens : 0);
}

void CacheManager::advance(uint64_t id, size_t count) {
    SequenceTable& t = table_mut(id);
    if (t.tokens + count > capacity(id))
        throw Error(std::to_string(t.tokens + count) + " tokens written into " +
                    std::to_string(capacity(id)) + " of capacity");
    t.tokens += count;
    release_passed(t);
}

void CacheManager::release_passed(SequenceTable& t) {
    for (size_t g = 0; g < groups_.size(); ++g) {
        const size_t window = static_cast<size_t>(groups_[g].window);
        if (window == 0 || t.tokens < window) continue;
        // The next query sits at position t.tokens and reads keys from
        // t.tokens - window + 1 on; a page whose last position is below that is done.
        const size_t first_needed = t.tokens - window + 1;
        const size_t bs = static_cast<size_t>(groups_[g].block_size);
        const size_t dead = std::min(first_needed / bs, t.blocks[g].size());
        for (size_t b = 0; b < dead; ++b) {
            if (t.blocks[g][b] == kNoBlock) continue;
            pools_[g].release(t.blocks[g][b]);
            t.blocks[g][b] = kNoBlock;
        }
    }
}

long CacheManager::slot_of(uint64_t id, size_t group, size_t position) const {
    const SequenceTable& t = table(id);
    const size_t bs = static_cast<size_t>(groups_.at(group).block_size);
    const size_t index = position / bs;
    if (index >= t.blocks[group].size() || t.blocks[group][index] == kNoBlock) return -1;
    return static_cast<long>(t.blocks[group][index]) * static_cast<long>(bs) + static_cast<long>(position % bs);
}

size_t CacheManager::claim_prefix(uint64_t id, const uint32_t* prompt, size_t length) {
    if (!prefix_cache_ || !sharing_possible()) return 0;
    SequenceTable& t = table_mut(id);
    if (t.tokens != 0 || !t.blocks[0].empty()) throw Error("a prefix is claimed by an empty table only");
    const size_t bs = static_cast<size_t>(groups_[0].block_size);
    // The prompt's last page is left alone even when full, so the step has at
    // least one token to run and the request owns the page it writes next.
    const size_t pages = (length + bs - 1) / bs;
    const size_t candidates = pages > 0 ? pages - 1 : 0;
    bool has_parent = false;
    BlockHash parent = 0;
    size_t shared = 0;
    std::vector<BlockId> taken(groups_.size());
    for (size_t index = 0; index < candidates; ++index) {
        const BlockHash hash = block_hash(has_parent, parent, prompt + index * bs, bs);
        size_t got = 0;
        for (; got < groups_.size(); ++got) {
            taken[got] = pools_[got].acquire_cached(hash);
            if (taken[got] == kNoBlock) break;
        }
        if (got < groups_.size()) {
            for (size_t g = 0; g < got; ++g) pools_[g].release(taken[g]);
            pools_[0].record_miss();
            break;
        }
        for (size_t g = 0; g < groups_.size(); ++g) t.blocks[g].push_back(taken[g]);
        t.hashes.push_back(hash);
        t.tokens += bs;
        shared += bs;
        has_parent = true;
        parent = hash;
    }
    return shared;
}

void CacheManager::publish_full(uint64_t id, const uint32_t* history, size_t length) {
    if (!prefix_cache_ || !sharing_possible()) return;
    SequenceTable& t = table_mut(id);
    const size_t bs = static_cast<size_t>(groups_[0].block_size);
    const size_t full = std::min(t.tokens / bs, t.blocks[0].size());
    while (t.hashes.size() < full) {
        const size_t index = t.hashes.size();
        const size_t start = index * bs;
        if (start + bs > length) break;
        const bool has_parent = !t.hashes.empty();
        const BlockHash hash = block_hash(has_parent, has_parent ? t.hashes.back() : 0, history + start, bs);
        t.hashes.push_back(hash);
        for (size_t g = 0; g < groups_.size(); ++g) pools_[g].publish(t.blocks[g][index], hash);
    }
}

size_t CacheManager::wasted_tokens(uint64_t id) const {
    const SequenceTable& t = table(id);
    if (groups_.empty()) return 0;
    return t.blocks[0].size() * static_cast<size_t>(groups_[0].block_size) - t.tokens;
}

size_t CacheManager::min_available() const {
    size_t least = SIZE_MAX;
    for (const BlockPool& p : pools_) least = std::min(least, p.available());
    return groups_.empty() ? SIZE_MAX : least;
}

bool CacheManager::fits_from_scratch(size_t length) const {
    for (size_t g = 0; g < groups_.size(); ++g) {
        const size_t bs = static_cast<size_t>(groups_[g].block_size);
        if ((length + bs - 1) / bs > pools_[g].available()) return false;
    }
    return true;
}

bool CacheManager::fits_in_total(size_t length, size_t budget) const {
    for (size_t g = 0; g < groups_.size(); ++g) {
        const size_t bs = static_cast<size_t>(groups_[g].block_size);
        size_t pages = (length + bs - 1) / bs;
        if (groups_[g].window > 0) {
            // A windowed group holds at most the window plus one step's tokens at a time.
            const size_t live = (static_cast<size_t>(groups_[g].window) + budget + bs - 1) / bs + 1;
            pages = std::min(pages, live);
        }
        if (pages > pools_[g].total()) return false;
    }
    return true;
}

}  // namespace pl
