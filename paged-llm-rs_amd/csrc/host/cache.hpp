// The cache manager's bookkeeping.  Nothing here touches a device: it hands out
// fixed-size pages (blocks) from pools, keeps for each request the table that
// says which page holds which stretch of its tokens, lets requests that begin
// alike share full pages by a chained content hash, and hands out fixed-size
// state slots.  (Reference: crates/pagedllm/src/blocks.rs.)
//
// Beyond the reference there are groups: layers with different needs (all keys,
// or a window of them) have pools and tables of their own, and a windowed group
// gives pages back as soon as the window has passed them.
#pragma once

#include <cstddef>
#include <cstdint>
#include <map>
#include <stdexcept>
#include <string>
#include <unordered_map>
#include <vector>

namespace pl {

using BlockId = int32_t;
using BlockHash = uint64_t;
constexpr BlockId kNoBlock = -1;

// FNV-1a over the little-endian bytes of (parent or 0, count, each token as a
// 64-bit value), finished with the splitmix64 mixer (blocks.rs:53-72).
BlockHash block_hash(bool has_parent, BlockHash parent, const uint32_t* tokens, size_t count);

struct Error : std::runtime_error {
    using std::runtime_error::runtime_error;
};

// One pool of pages: free list, holder counts, names and least-recently-released
// eviction of named pages (blocks.rs:76-293).
class BlockPool {
public:
    explicit BlockPool(size_t total);

    // A page for a request's own use, or kNoBlock.  A page without a name goes
    // first; only when every free page is named does the one released longest
    // ago lose its name.
    BlockId allocate();
    // The page that already holds this prefix, or kNoBlock.
    BlockId acquire_cached(BlockHash hash);
    void record_miss() { ++misses_; }
    // Name a page that has just been filled.  The first page under a name keeps it.
    void publish(BlockId block, BlockHash hash);
    // Give a page back.  It keeps its name and contents until the space is needed.
    void release(BlockId block);
    void clear_cache();

    size_t available() const { return free_anonymous_.size() + free_named_.size(); }
    size_t total() const { return total_; }
    size_t in_use() const { return total_ - available(); }
    size_t cached_blocks() const { return cached_.size(); }
    uint64_t handed_out() const { return handed_out_; }
    uint64_t hits() const { return hits_; }
    uint64_t misses() const { return misses_; }
    uint64_t evictions() const { return evictions_; }
    uint32_t holders(BlockId block) const { return slots_.at(static_cast<size_t>(block)).holders; }

private:
    struct Slot {
        uint32_t holders = 0;
        bool named = false;
        BlockHash hash = 0;
        uint64_t released_at = 0;
    };
    void forget(BlockId block);

    std::vector<Slot> slots_;
    std::vector<BlockId> free_anonymous_;          // a stack: the last released is taken first
    std::map<uint64_t, BlockId> free_named_;       // by release time: the oldest gives way first
    std::unordered_map<BlockHash, BlockId> cached_;
    size_t total_;
    uint64_t clock_ = 0, handed_out_ = 0, hits_ = 0, misses_ = 0, evictions_ = 0;
};

struct GroupSpec {
    int block_size;  // tokens a page
    int num_blocks;  // pages in this group's pool
    int window;      // 0: every key is kept; w > 0: only the last w keys are read
};

// Where one request's tokens live: per group a list of pages in logical order
// (kNoBlock where the window has passed), the tokens written, and the names of
// the full pages (blocks.rs:297-430).
struct SequenceTable {
    std::vector<std::vector<BlockId>> blocks;  // [group][logical block]
    size_t tokens = 0;
    std::vector<BlockHash> hashes;
    int state_slot = -1;
};

class CacheManager {
public:
    CacheManager(std::vector<GroupSpec> groups, int state_slots);

    size_t num_groups() const { return groups_.size(); }
    const GroupSpec& group(size_t g) const { return groups_.at(g); }
    BlockPool& pool(size_t g) { return pools_.at(g); }
    const BlockPool& pool(size_t g) const { return pools_.at(g); }

    // Whether full pages may be shared between requests: every group keeps all
    // keys, all pages are the same size, and there is no per-request state that
    // a shared page could not bring back.
    bool sharing_possible() const;
    void set_prefix_cache(bool enabled);
    bool prefix_cache() const { return prefix_cache_; }

    bool has(uint64_t id) const { return tables_.count(id) != 0; }
    // Registers a request.  Returns its state slot, -1 when no slots are
    // configured; throws when the id is known or no slot is free.
    int add_sequence(uint64_t id);
    bool state_slot_available() const { return state_slots_ == 0 || !free_state_slots_.empty(); }
    // Releases every page and the state slot.  Unknown ids are ignored.
    void free_sequence(uint64_t id);

    size_t tokens(uint64_t id) const { return table(id).tokens; }
    // Tokens the pages already held could take (the least over the groups).
    size_t capacity(uint64_t id) const;
    // Pages still needed, in the hungriest group, to hold `count` more tokens.
    size_t blocks_needed(uint64_t id, size_t count) const;
    // The same in one group.
    size_t blocks_needed_in(uint64_t id, size_t group, size_t count) const { return needed_in_group(table(id), group, count); }
    // Take pages until `count` more tokens fit; nothing is taken when any pool
    // cannot supply its share.
    bool reserve(uint64_t id, size_t count);
    // Take pages for as many of `count` more tokens as the pools allow; returns
    // how many tokens now fit (at most count).
    size_t reserve_up_to(uint64_t id, size_t count);
    // Record that `count` tokens were written.  Refused past the capacity.  A
    // windowed group then gives back the pages the window has passed.
    void advance(uint64_t id, size_t count);
    // Slot of a position in a group's pool, or -1 (blocks.rs:411-414).
    long slot_of(uint64_t id, size_t group, size_t position) const;

    // Take the pages that already hold this prompt's leading tokens; the
    // prompt's last page is always left alone (scheduler.rs:596-621).  Returns
    // how many tokens the request does not have to compute.
    size_t claim_prefix(uint64_t id, const uint32_t* prompt, size_t length);
    // Name the pages this request has just filled (blocks.rs:390-404).
    void publish_full(uint64_t id, const uint32_t* history, size_t length);

    const SequenceTable& table(uint64_t id) const;
    // Tokens in pages that are held and not yet written (blocks.rs:427-429), group 0.
    size_t wasted_tokens(uint64_t id) const;
    // Smallest number of free pages over the groups, and whether a new request of
    // `length` tokens fits (pages from scratch in every group).
    size_t min_available() const;
    bool fits_from_scratch(size_t length) const;
    bool fits_in_total(size_t length, size_t budget) const;
    size_t live_sequences() const { return tables_.size(); }
    int state_slots() const { return state_slots_; }
    int free_state_slots() const { return static_cast<int>(free_state_slots_.size()); }

private:
    SequenceTable& table_mut(uint64_t id);
    size_t needed_in_group(const SequenceTable& t, size_t g, size_t count) const;
    void release_passed(SequenceTable& t);

    std::vector<GroupSpec> groups_;
    std::vector<BlockPool> pools_;
    std::unordered_map<uint64_t, SequenceTable> tables_;
    int state_slots_;
    std::vector<int> free_state_slots_;
    bool prefix_cache_ = true;
};

}  // namespace pl
