"""The cache manager: which pages each request holds, in every group, and which
state slot.  The bookkeeping is native (csrc/host/cache.cpp); this class is its
Python face.  Nothing here touches the device.
(Reference: crates/pagedllm/src/blocks.rs; groups and state slots go beyond it.)
"""

from __future__ import annotations

import ctypes
from dataclasses import dataclass

from .. import native
from ..errors import ConfigError

_COUNTERS = {"available": 0, "total": 1, "in_use": 2, "cached_blocks": 3, "handed_out": 4, "hits": 5,
             "misses": 6, "evictions": 7}


def block_hash(parent, tokens) -> int:
    """The name of a full page: its tokens chained onto the name of the page before it."""
    arr, n = native.u32_array(tokens)
    return native.library().plh_block_hash(0 if parent is None else 1, parent or 0, arr, n)


class BlockPool:
    """One pool of pages on its own (free list, holders, names, eviction)."""

    def __init__(self, total: int):
        self._lib = native.library()
        self._h = self._lib.plh_pool_create(total)

    def __del__(self):
        if getattr(self, "_h", None):
            self._lib.plh_pool_destroy(self._h)
            self._h = None

    def allocate(self):
        b = self._lib.plh_pool_allocate(self._h)
        return None if b < 0 else b

    def acquire_cached(self, hash_: int):
        b = self._lib.plh_pool_acquire_cached(self._h, hash_)
        return None if b < 0 else b

    def publish(self, block: int, hash_: int) -> None:
        self._lib.plh_pool_publish(self._h, block, hash_)

    def release(self, block: int) -> None:
        native.check(self._lib.plh_pool_release(self._h, block))

    def clear_cache(self) -> None:
        self._lib.plh_pool_clear_cache(self._h)

    def __getattr__(self, name):
        if name in _COUNTERS:
            return self._lib.plh_pool_counter(self._h, _COUNTERS[name])
        raise AttributeError(name)


@dataclass(frozen=True)
class GroupGeometry:
    block_size: int
    num_blocks: int
    window: int = 0   # 0: all keys


class CacheManager:
    def __init__(self, groups, state_slots: int = 0):
        groups = list(groups)
        self.groups = groups
        self.state_slots = state_slots
        self._lib = native.library()
        n = len(groups)
        arr = ctypes.c_int * max(n, 1)
        self._h = self._lib.plh_cache_create(
            n, arr(*[g.block_size for g in groups]), arr(*[g.num_blocks for g in groups]),
            arr(*[g.window for g in groups]), state_slots)
        if not self._h:
            raise ConfigError(native.last_error())

    def __del__(self):
        if getattr(self, "_h", None):
            self._lib.plh_cache_destroy(self._h)
            self._h = None

    @property
    def handle(self):
        return self._h

    # -- requests -------------------------------------------------------------------
    def add_sequence(self, seq_id: int) -> int:
        slot = self._lib.plh_cache_add_sequence(self._h, seq_id)
        if slot < -1:
            raise ConfigError(native.last_error())
        return slot

    def free_sequence(self, seq_id: int) -> None:
        self._lib.plh_cache_free_sequence(self._h, seq_id)

    def has(self, seq_id: int) -> bool:
        return bool(self._lib.plh_cache_has(self._h, seq_id))

    def tokens(self, seq_id: int) -> int:
        return native.check(self._lib.plh_cache_tokens(self._h, seq_id))

    def capacity(self, seq_id: int) -> int:
        return native.check(self._lib.plh_cache_capacity(self._h, seq_id))

    def blocks_needed(self, seq_id: int, count: int) -> int:
        return native.check(self._lib.plh_cache_blocks_needed(self._h, seq_id, count))

    def reserve(self, seq_id: int, count: int) -> bool:
        return bool(native.check(self._lib.plh_cache_reserve(self._h, seq_id, count)))

    def reserve_up_to(self, seq_id: int, count: int) -> int:
        return native.check(self._lib.plh_cache_reserve_up_to(self._h, seq_id, count))

    def advance(self, seq_id: int, count: int) -> None:
        native.check(self._lib.plh_cache_advance(self._h, seq_id, count))

    def slot_of(self, seq_id: int, group: int, position: int):
        slot = self._lib.plh_cache_slot_of(self._h, seq_id, group, position)
        if slot < -1:
            raise ConfigError(native.last_error())
        return None if slot < 0 else slot

    def claim_prefix(self, seq_id: int, prompt) -> int:
        arr, n = native.u32_array(prompt)
        return native.check(self._lib.plh_cache_claim_prefix(self._h, seq_id, arr, n))

    def publish_full(self, seq_id: int, history) -> None:
        arr, n = native.u32_array(history)
        native.check(self._lib.plh_cache_publish_full(self._h, seq_id, arr, n))

    def set_prefix_cache(self, enabled: bool) -> None:
        self._lib.plh_cache_set_prefix_cache(self._h, 1 if enabled else 0)

    def sharing_possible(self) -> bool:
        return bool(self._lib.plh_cache_sharing_possible(self._h))

    def table(self, seq_id: int, group: int = 0) -> list:
        n = native.check(self._lib.plh_cache_table_len(self._h, seq_id, group))
        buf = (ctypes.c_int * max(n, 1))()
        native.check(self._lib.plh_cache_table(self._h, seq_id, group, buf, n))
        return list(buf[:n])

    def table_into(self, seq_id: int, group: int, address: int, capacity: int) -> int:
        """Write the page list of one group at a raw address (a row of a pinned
        host buffer); returns its length."""
        return native.check(self._lib.plh_cache_table(self._h, seq_id, group, address, capacity))

    def fill_step(self, ids_address: int, count: int, positions_address: int, group: int, tables_address: int,
                  width: int) -> int:
        """For ``count`` requests (64-bit ids at a raw address): where each one's next token goes, and
        the rows of one group's block table (-1 beyond a request's pages), written at raw addresses
        of 32-bit buffers.  An address of 0 leaves that output out.  Returns 0, or, when a request has
        more pages than ``width``, that number of pages (the rows are then not written)."""
        return native.check(self._lib.plh_cache_fill_step(self._h, count, ids_address, positions_address, group,
                                                          tables_address, width))

    def state_slot(self, seq_id: int) -> int:
        slot = self._lib.plh_cache_state_slot(self._h, seq_id)
        if slot < -1:
            raise ConfigError(native.last_error())
        return slot

    def wasted_tokens(self, seq_id: int) -> int:
        return native.check(self._lib.plh_cache_wasted_tokens(self._h, seq_id))

    # -- counters ---------------------------------------------------------------------
    def counter(self, name: str, group: int = 0) -> int:
        return self._lib.plh_cache_counter(self._h, group, _COUNTERS[name])

    def available(self, group: int = 0) -> int:
        return self.counter("available", group)

    def in_use(self, group: int = 0) -> int:
        return self.counter("in_use", group)

    def total(self, group: int = 0) -> int:
        return self.counter("total", group)

    def holders(self, group: int, block: int) -> int:
        return native.check(self._lib.plh_cache_holders(self._h, group, block))

    @property
    def live_sequences(self) -> int:
        return self._lib.plh_cache_live_sequences(self._h)

    @property
    def free_state_slots(self) -> int:
        return self._lib.plh_cache_free_state_slots(self._h)
