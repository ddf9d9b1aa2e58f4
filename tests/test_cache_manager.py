"""The cache manager without a GPU: pools, tables, names, groups, windows, state slots.
Scenarios follow the reference's own unit tests (blocks.rs:432-675, batch.rs:439-453)."""

from __future__ import annotations

import random

import pytest

import plain_qwen3 as plain
from paged_llm_rs_amd.cache import (BlockPool, CacheLayout, CacheManager, GroupGeometry, KVCacheSpec,
                                    block_hash)
from paged_llm_rs_amd.cache.layout import CacheGroupLayout
from paged_llm_rs_amd.errors import ConfigError


def one_group(blocks, block_size, window=0, state_slots=0):
    return CacheManager([GroupGeometry(block_size, blocks, window)], state_slots)


# --- one pool ----------------------------------------------------------------------------------

def test_blocks_are_handed_out_in_order_and_come_back():
    """blocks.rs:436-448"""
    pool = BlockPool(4)
    assert pool.available == 4
    assert [pool.allocate() for _ in range(4)] == [0, 1, 2, 3]
    assert pool.allocate() is None, "an empty pool hands out nothing"
    assert pool.in_use == 4
    pool.release(2)
    assert pool.allocate() == 2
    assert pool.handed_out == 5


def test_releasing_twice_is_refused():
    pool = BlockPool(2)
    b = pool.allocate()
    pool.release(b)
    with pytest.raises(ConfigError):
        pool.release(b)
    with pytest.raises(ConfigError):
        pool.release(7)


def test_a_named_block_is_handed_to_a_second_request():
    """blocks.rs:552-569"""
    pool = BlockPool(4)
    block = pool.allocate()
    h = block_hash(None, [1, 2, 3, 4])
    pool.publish(block, h)
    assert pool.cached_blocks == 1
    assert pool.acquire_cached(h) == block
    assert pool.in_use == 1, "one block, two holders"
    pool.release(block)
    assert pool.in_use == 1
    pool.release(block)
    assert pool.in_use == 0


def test_an_unheld_block_keeps_its_name_until_the_space_is_needed():
    """blocks.rs:571-586"""
    pool = BlockPool(2)
    first = pool.allocate()
    h = block_hash(None, [7, 7, 7, 7])
    pool.publish(first, h)
    pool.release(first)
    assert pool.available == 2
    assert pool.acquire_cached(h) == first
    assert pool.hits == 1


def test_the_block_unheld_longest_gives_way_first():
    """blocks.rs:588-610"""
    pool = BlockPool(2)
    a, b = pool.allocate(), pool.allocate()
    ha, hb = block_hash(None, [1]), block_hash(None, [2])
    pool.publish(a, ha)
    pool.publish(b, hb)
    pool.release(a)
    pool.release(b)
    assert pool.allocate() == a, "a was unheld longest"
    assert pool.evictions == 1
    assert pool.acquire_cached(ha) is None, "its name went with its contents"
    assert pool.acquire_cached(hb) == b


def test_a_nameless_block_is_taken_before_a_cached_one_loses_its_name():
    """blocks.rs:612-627"""
    pool = BlockPool(3)
    cached = pool.allocate()
    h = block_hash(None, [5])
    pool.publish(cached, h)
    pool.release(cached)
    for _ in range(2):
        assert pool.allocate() != cached
    assert pool.evictions == 0
    assert pool.acquire_cached(h) == cached


def test_the_first_publisher_keeps_the_name():
    """blocks.rs:191-203"""
    pool = BlockPool(4)
    a, b = pool.allocate(), pool.allocate()
    h = block_hash(None, [9, 9])
    pool.publish(a, h)
    pool.publish(b, h)
    assert pool.cached_blocks == 1
    pool.release(a)
    pool.release(b)
    assert pool.acquire_cached(h) == a


def test_clearing_the_cache_leaves_the_pool_working():
    """blocks.rs:657-674"""
    pool = BlockPool(2)
    block = pool.allocate()
    h = block_hash(None, [1, 2])
    pool.publish(block, h)
    pool.release(block)
    pool.clear_cache()
    assert pool.cached_blocks == 0
    assert pool.acquire_cached(h) is None
    assert pool.available == 2
    assert pool.allocate() is not None


# --- names -----------------------------------------------------------------------------------------

def test_a_block_name_depends_on_everything_before_it():
    """blocks.rs:531-550, and the values against the independent implementation."""
    tokens = [1, 2, 3, 4]
    root = block_hash(None, tokens)
    assert root == block_hash(None, tokens)
    assert root != block_hash(99, tokens)
    assert block_hash(None, [1, 2, 3, 4]) != block_hash(None, [4, 3, 2, 1])
    assert block_hash(None, [1, 2]) != block_hash(None, [1, 2, 0, 0])
    rng = random.Random(3)
    for _ in range(50):
        toks = [rng.randrange(2 ** 32) for _ in range(rng.randrange(0, 20))]
        parent = rng.choice([None, rng.randrange(1, 2 ** 64)])
        assert block_hash(parent, toks) == plain.block_hash(parent, toks)


# --- tables ----------------------------------------------------------------------------------------

def test_a_table_asks_for_a_block_only_when_the_last_one_is_full():
    """blocks.rs:450-462"""
    m = one_group(16, 4)
    m.add_sequence(1)
    assert m.blocks_needed(1, 1) == 1
    assert m.blocks_needed(1, 4) == 1
    assert m.blocks_needed(1, 5) == 2
    assert m.reserve(1, 1)
    assert m.capacity(1) == 4
    m.advance(1, 3)
    assert m.blocks_needed(1, 1) == 0
    assert m.blocks_needed(1, 2) == 1


def test_a_position_past_a_block_boundary_lands_in_the_next_block():
    """blocks.rs:464-477, with blocks [7, 2, 5] of four tokens."""
    m = one_group(8, 4)
    # take blocks so that the request gets 7, 2, 5 in this order
    for other in range(8):
        m.add_sequence(100 + other)
        m.reserve(100 + other, 1)
    for owner in (107, 102, 105):
        m.free_sequence(owner)
    m.add_sequence(1)
    for want in (5, 2, 7):      # the stack hands back the last released first
        pass
    assert m.reserve(1, 12)
    assert m.table(1) == [5, 2, 7]
    m.advance(1, 10)
    t = m.table(1)
    assert m.slot_of(1, 0, 0) == t[0] * 4
    assert m.slot_of(1, 0, 3) == t[0] * 4 + 3
    assert m.slot_of(1, 0, 4) == t[1] * 4, "the boundary moves it"
    assert m.slot_of(1, 0, 9) == t[2] * 4 + 1
    assert m.slot_of(1, 0, 12) is None, "past the blocks it holds"


def test_writing_past_the_capacity_is_refused():
    """blocks.rs:479-486"""
    m = one_group(4, 4)
    m.add_sequence(1)
    m.reserve(1, 4)
    m.advance(1, 4)
    with pytest.raises(ConfigError):
        m.advance(1, 1)
    assert m.tokens(1) == 4


def test_what_paging_wastes_is_one_partial_block():
    """blocks.rs:488-498"""
    m = one_group(16, 16)
    m.add_sequence(1)
    m.reserve(1, 97)
    m.advance(1, 97)
    assert m.capacity(1) == 112
    assert m.wasted_tokens(1) == 15


def test_freeing_returns_every_block():
    """blocks.rs:500-515"""
    m = one_group(8, 4)
    m.add_sequence(1)
    m.reserve(1, 9)
    m.advance(1, 9)
    assert m.available() == 5
    m.free_sequence(1)
    assert m.available() == 8
    assert not m.has(1)


def test_cache_arithmetic_of_the_published_model():
    """batch.rs:439-453 and blocks.rs:517-528: Qwen3-0.6B in bfloat16."""
    layout = CacheLayout([CacheGroupLayout(KVCacheSpec(8, 128, None), list(range(28)))], {}, {})
    assert layout.bytes_per_token(2) == 114_688
    assert layout.blocks_within(3_758_096_384, 16, 2) == 2048
    assert layout.blocks_within(1, 16, 2) == 1, "a budget under one block still gives one"
    reserved = 3_758_096_384 // (1024 * 114_688)
    assert reserved == 32
    assert 2048 // -(-140 // 16) == 227


# --- sharing ------------------------------------------------------------------------------------------

def test_claim_takes_full_blocks_but_never_the_prompts_last():
    """scheduler.rs:596-621, blocks.rs:629-655"""
    m = one_group(16, 4)
    prompt = list(range(12))
    m.add_sequence(1)
    assert m.claim_prefix(1, prompt) == 0
    m.reserve(1, 12)
    m.advance(1, 3)
    m.publish_full(1, prompt)
    assert m.counter("cached_blocks") == 0, "three of four is not full"
    m.advance(1, 9)
    m.publish_full(1, prompt)
    assert m.counter("cached_blocks") == 3
    m.add_sequence(2)
    assert m.claim_prefix(2, prompt) == 8, "three blocks are full, the last is left alone"
    assert m.tokens(2) == 8 and m.table(2) == m.table(1)[:2]
    assert m.holders(0, m.table(1)[0]) == 2
    # a different prefix shares nothing, and the same tokens after it are another block
    m.add_sequence(3)
    assert m.claim_prefix(3, [50, 51, 52, 53] + prompt[4:]) == 0
    m.free_sequence(1)
    m.free_sequence(2)
    m.free_sequence(3)
    assert m.available() == 16


def test_sharing_is_off_with_a_window_or_state_slots():
    assert one_group(4, 4).sharing_possible()
    assert not one_group(4, 4, window=8).sharing_possible()
    assert not one_group(4, 4, state_slots=2).sharing_possible()
    assert not CacheManager([GroupGeometry(4, 4), GroupGeometry(8, 4)]).sharing_possible()


# --- groups and windows ----------------------------------------------------------------------------------

def test_groups_have_pages_of_their_own_and_a_window_gives_them_back():
    m = CacheManager([GroupGeometry(4, 32, 0), GroupGeometry(4, 8, 6)])
    m.add_sequence(1)
    assert m.reserve(1, 10)
    assert len(m.table(1, 0)) == 3 and len(m.table(1, 1)) == 3
    m.advance(1, 10)
    # next query at position 10 reads keys 5..10 in the windowed group: block 0 (0..3) is done
    assert m.table(1, 1)[0] == -1 and m.table(1, 1)[1] >= 0
    assert all(b >= 0 for b in m.table(1, 0)), "the full group keeps everything"
    assert m.available(1) == 8 - 2
    assert m.slot_of(1, 1, 2) is None and m.slot_of(1, 1, 5) is not None
    for _ in range(30):
        assert m.reserve(1, 1)
        m.advance(1, 1)
    assert m.in_use(1) <= 3, "a windowed group holds the window and no more"
    assert m.in_use(0) == 10
    m.free_sequence(1)
    assert m.available(0) == 32 and m.available(1) == 8


def test_reserve_takes_nothing_when_one_group_is_dry():
    m = CacheManager([GroupGeometry(4, 8, 0), GroupGeometry(4, 2, 0)])
    m.add_sequence(1)
    assert not m.reserve(1, 12), "the second group has two pages"
    assert m.available(0) == 8 and m.available(1) == 2
    assert m.reserve_up_to(1, 12) == 8
    assert m.capacity(1) == 8


def test_state_slots_are_handed_out_and_come_back():
    m = one_group(8, 4, state_slots=2)
    assert m.add_sequence(1) == 0
    assert m.add_sequence(2) == 1
    with pytest.raises(ConfigError):
        m.add_sequence(3)
    m.free_sequence(1)
    assert m.add_sequence(3) == 0
    assert m.state_slot(2) == 1 and m.free_state_slots == 0
    with pytest.raises(ConfigError):
        m.add_sequence(2)


# --- invariants under random orders of requests -------------------------------------------------------

@pytest.mark.parametrize("seed", range(6))
def test_no_page_is_lost_held_twice_or_freed_twice(seed):
    rng = random.Random(seed)
    window = rng.choice([0, 0, 7, 20])
    bs = rng.choice([1, 4, 16])
    total = rng.randrange(6, 40)
    m = CacheManager([GroupGeometry(bs, total, 0), GroupGeometry(bs, total, window)])
    m.set_prefix_cache(False)
    live: dict = {}
    next_id = 1
    for _ in range(600):
        action = rng.random()
        if action < 0.25 and len(live) < 6:
            m.add_sequence(next_id)
            live[next_id] = 0
            next_id += 1
        elif action < 0.8 and live:
            sid = rng.choice(list(live))
            n = rng.randrange(1, 3 * bs + 2)
            before = [m.available(g) for g in range(2)]
            if m.reserve(sid, n):
                m.advance(sid, n)
                live[sid] += n
            else:
                assert [m.available(g) for g in range(2)] == before, "a refused reservation takes nothing"
        elif live:
            sid = rng.choice(list(live))
            m.free_sequence(sid)
            del live[sid]
        # every held page is held once; held + free = total, in both groups
        for g in range(2):
            held = [b for sid in live for b in m.table(sid, g) if b >= 0]
            assert len(held) == len(set(held)), "a page is held twice"
            assert len(held) == m.in_use(g)
            assert m.in_use(g) + m.available(g) == total
            for b in held:
                assert m.holders(g, b) == 1
        for sid, n in live.items():
            assert m.tokens(sid) == n
            # the next query sits at position n and reads the keys n-window+1 .. n
            for p in range(max(0, n - window + 1) if window else 0, n):
                assert m.slot_of(sid, 1, p) is not None, "a position inside the window lost its page"
    for sid in list(live):
        m.free_sequence(sid)
    assert m.available(0) == total and m.available(1) == total


@pytest.mark.parametrize("seed", range(4))
def test_shared_pages_are_counted_right_under_random_orders(seed):
    rng = random.Random(100 + seed)
    bs, total = 4, 24
    m = one_group(total, bs)
    prompts = [[rng.randrange(3) for _ in range(rng.randrange(1, 30))] for _ in range(5)]
    live: dict = {}
    next_id = 1
    for _ in range(300):
        if rng.random() < 0.5 and len(live) < 4:
            prompt = rng.choice(prompts)
            sid = next_id
            next_id += 1
            m.add_sequence(sid)
            shared = m.claim_prefix(sid, prompt)
            assert shared % bs == 0 and shared < len(prompt)
            if m.reserve(sid, len(prompt) - shared):
                m.advance(sid, len(prompt) - shared)
                m.publish_full(sid, prompt)
                live[sid] = prompt
            else:
                m.free_sequence(sid)
        elif live:
            sid = rng.choice(list(live))
            m.free_sequence(sid)
            del live[sid]
        holders: dict = {}
        for sid in live:
            for b in m.table(sid):
                holders[b] = holders.get(b, 0) + 1
        for b, n in holders.items():
            assert m.holders(0, b) == n
        assert len(holders) == m.in_use()
        assert m.in_use() + m.available() == total
        # requests with the same prompt read the same pages for its shared part
        for a in live:
            for b in live:
                if a < b and live[a] == live[b]:
                    full = (len(live[a]) - 1) // bs
                    assert m.table(a)[:full] == m.table(b)[:full] or m.counter("evictions") > 0
    for sid in list(live):
        m.free_sequence(sid)
    assert m.available() == total


# --- the order of layers and whose cache a run uses ---------------------------------------------------------

def test_schedules_that_would_write_a_cache_twice_or_read_an_unwritten_one_are_refused():
    import types

    from paged_llm_rs_amd.cache import CacheLayout
    from paged_llm_rs_amd.cache.layout import KVCacheSpec
    from paged_llm_rs_amd.config import ScheduleEntry
    from paged_llm_rs_amd.errors import ConfigError

    def block(kv_heads, head_dim, window=None):
        mixer = types.SimpleNamespace(cache_spec=lambda: KVCacheSpec(kv_heads, head_dim, window), state_spec=lambda: None)
        return types.SimpleNamespace(mixer=mixer)

    blocks = [block(2, 16), block(2, 16), block(1, 16), block(2, 16, 8)]
    ok = CacheLayout.from_blocks(blocks, [ScheduleEntry(0), ScheduleEntry(1), ScheduleEntry(1, cache_from=1),
                                          ScheduleEntry(0, cache_from=1)])
    assert len(ok.groups) == 1 and ok.groups[0].layers == [0, 1]
    with pytest.raises(ConfigError, match="twice"):
        CacheLayout.from_blocks(blocks, [ScheduleEntry(0), ScheduleEntry(0)])
    with pytest.raises(ConfigError, match="no earlier run"):
        CacheLayout.from_blocks(blocks, [ScheduleEntry(0, cache_from=1), ScheduleEntry(1)])
    with pytest.raises(ConfigError, match="another shape"):
        CacheLayout.from_blocks(blocks, [ScheduleEntry(0), ScheduleEntry(2, cache_from=0)])
    with pytest.raises(ConfigError, match="another shape"):
        CacheLayout.from_blocks(blocks, [ScheduleEntry(0), ScheduleEntry(3, cache_from=0)])
