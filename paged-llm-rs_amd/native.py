"""The host runtime library (cache manager, scheduler, sampler) behind ctypes."""

from __future__ import annotations

import ctypes
from ctypes import POINTER, c_char_p, c_double, c_float, c_int, c_long, c_size_t, c_uint32, c_uint64, c_void_p

from . import build
from .errors import ConfigError

_lib = None

u64, u32, sz, vp, i32, lg, f32 = c_uint64, c_uint32, c_size_t, c_void_p, c_int, c_long, c_float
P = POINTER


def _signatures(lib) -> None:
    table = {
        "plh_last_error": ([], c_char_p),
        "plh_block_hash": ([i32, u64, P(u32), sz], u64),
        "plh_pool_create": ([sz], vp), "plh_pool_destroy": ([vp], None),
        "plh_pool_allocate": ([vp], i32), "plh_pool_acquire_cached": ([vp, u64], i32),
        "plh_pool_publish": ([vp, i32, u64], None), "plh_pool_release": ([vp, i32], lg),
        "plh_pool_clear_cache": ([vp], None), "plh_pool_counter": ([vp, i32], u64),
        "plh_cache_create": ([i32, P(i32), P(i32), P(i32), i32], vp), "plh_cache_destroy": ([vp], None),
        "plh_cache_add_sequence": ([vp, u64], lg), "plh_cache_free_sequence": ([vp, u64], None),
        "plh_cache_has": ([vp, u64], i32), "plh_cache_tokens": ([vp, u64], lg),
        "plh_cache_capacity": ([vp, u64], lg), "plh_cache_blocks_needed": ([vp, u64, sz], lg),
        "plh_cache_reserve": ([vp, u64, sz], lg), "plh_cache_reserve_up_to": ([vp, u64, sz], lg),
        "plh_cache_advance": ([vp, u64, sz], lg), "plh_cache_slot_of": ([vp, u64, sz, sz], lg),
        "plh_cache_claim_prefix": ([vp, u64, P(u32), sz], lg),
        "plh_cache_publish_full": ([vp, u64, P(u32), sz], lg),
        "plh_cache_set_prefix_cache": ([vp, i32], None), "plh_cache_sharing_possible": ([vp], i32),
        "plh_cache_table": ([vp, u64, sz, vp, sz], lg), "plh_cache_table_len": ([vp, u64, sz], lg),
        "plh_cache_fill_step": ([vp, sz, vp, vp, sz, vp, sz], lg),
        "plh_cache_state_slot": ([vp, u64], lg), "plh_cache_wasted_tokens": ([vp, u64], lg),
        "plh_cache_counter": ([vp, sz, i32], u64), "plh_cache_live_sequences": ([vp], lg),
        "plh_cache_free_state_slots": ([vp], i32), "plh_cache_holders": ([vp, sz, i32], lg),
        "plh_rng_next_u64": ([P(u64)], u64), "plh_rng_next_f32": ([P(u64)], f32),
        "plh_sampling_problem": ([f32, i32, lg, i32, f32], c_char_p),
        "plh_sample": ([f32, i32, f32, vp, sz, P(u64)], lg),
        "plh_sched_create": ([vp, sz, sz, sz], vp), "plh_sched_destroy": ([vp], None),
        "plh_sched_set_chunk": ([vp, sz], None), "plh_sched_set_prefix_cache": ([vp, i32], None),
        "plh_sched_submit": ([vp, u64, P(u32), sz, f32, i32, lg, i32, f32, sz, P(u32), sz, u64], lg),
        "plh_sched_plan": ([vp, P(sz)], lg),
        "plh_sched_plan_read": ([vp, i32, P(u64), P(i32), P(i32), P(i32), P(i32), P(i32), P(i32), P(u32), P(u64),
                                 P(u64), P(i32), P(u64)], None),
        "plh_sched_launched": ([vp], lg), "plh_sched_plan_ahead": ([vp, P(sz)], lg),
        "plh_sched_drop_ahead": ([vp], None), "plh_sched_abandon": ([vp], None),
        "plh_sched_commit": ([vp, P(u32), sz, P(sz)], lg),
        "plh_sched_drain_finished": ([vp, P(sz)], lg),
        "plh_sched_outcome_read": ([vp, P(u64), P(u32), P(u64), P(i32), P(u64), P(u64), P(u32)], None),
        "plh_sched_cancel": ([vp, u64], lg),
        "plh_sched_waiting": ([vp], sz), "plh_sched_running": ([vp], sz),
        "plh_sched_running_ids": ([vp, P(u64), sz], sz), "plh_sched_wasted_tokens": ([vp], sz),
        "plh_sched_metrics": ([vp, P(u64)], None),
        "plh_sched_sample": ([vp, u64, vp, sz], lg),
        "plh_sched_sampling_of": ([vp, u64, P(f32), P(i32), P(f32), P(f32)], lg),
        "plh_oracle_rms_norm": ([vp, vp, c_double, lg, lg, vp], None),
        "plh_oracle_rotate": ([vp, vp, lg, lg, lg, lg, c_double, i32], None),
        "plh_oracle_product": ([vp, vp, lg, lg, lg, vp], None),
        "plh_oracle_swiglu": ([vp, lg, lg, vp], None),
        "plh_oracle_paged_attention": ([vp, vp, vp, vp, vp, vp, lg, lg, lg, lg, lg, lg, c_double, lg, vp], None),
        "plh_oracle_argmax": ([vp, lg, lg, vp], None),
    }
    for name, (argtypes, restype) in table.items():
        fn = getattr(lib, name)
        fn.argtypes = argtypes
        fn.restype = restype


def library():
    global _lib
    if _lib is None:
        lib = build.load("host")
        _signatures(lib)
        _lib = lib
    return _lib


def last_error() -> str:
    return library().plh_last_error().decode()


def check(value: int) -> int:
    """A count from a call that reports failure as a negative number."""
    if value < 0:
        raise ConfigError(last_error())
    return value


def u32_array(values):
    values = list(values)
    return (u32 * len(values))(*values), len(values)
