"""The scheduler's Python face.  The policy is native (csrc/host/scheduler.cpp):
it admits requests, cuts prompts into portions under a token budget, decodes,
finishes, frees, and evicts the newest request when pages run out.
(Reference: crates/pagedllm/src/scheduler.rs.)"""

from __future__ import annotations

import ctypes
from dataclasses import dataclass, field

from .. import native
from ..errors import ConfigError
from .batch import StepEntry

IDLE, PREFILL, MIXED, DECODE, REFUSED = range(5)
KIND_NAMES = ["idle", "prefill", "mixed", "decode", "refused"]
FINISH_NAMES = {1: "stop", 2: "length"}
_METRICS = ["steps", "prefills", "tokens", "decode_rows", "admission_stalls", "preemptions", "mixed_steps",
            "decode_steps", "recomputed_tokens", "cached_tokens", "prefilled_tokens"]


@dataclass
class Plan:
    kind: int
    ids: list = field(default_factory=list)           # requests a token comes back for, in row order
    advanced: list = field(default_factory=list)      # (id, tokens written)
    entries: list = field(default_factory=list)       # StepEntry, in batch order
    refused: int = 0

    @property
    def kind_name(self) -> str:
        return KIND_NAMES[self.kind]

    @property
    def num_tokens(self) -> int:
        return sum(len(e.tokens) for e in self.entries)


@dataclass
class Finished:
    id: int
    finish: str
    prompt_tokens: int
    generated: int
    preemptions: int


@dataclass
class Outcome:
    tokens: list = field(default_factory=list)        # (id, token)
    finished: list = field(default_factory=list)      # Finished


class Scheduler:
    def __init__(self, manager, max_batch: int = 16, chunk=128, max_positions: int = 0,
                 prefix_cache: bool = True):
        """``chunk`` None runs a prompt whole; a number is the most tokens one step carries."""
        if chunk is not None and chunk < 1:
            raise ConfigError("a chunk of 0 would carry nothing")
        self._lib = native.library()
        self.manager = manager            # keeps the native cache manager alive
        self._h = self._lib.plh_sched_create(manager.handle, max_batch, chunk or 0, max_positions)
        self.set_prefix_cache(prefix_cache)

    def __del__(self):
        if getattr(self, "_h", None):
            self._lib.plh_sched_destroy(self._h)
            self._h = None

    def set_chunk(self, chunk) -> None:
        self._lib.plh_sched_set_chunk(self._h, chunk or 0)

    def set_prefix_cache(self, enabled: bool) -> None:
        self._lib.plh_sched_set_prefix_cache(self._h, 1 if enabled else 0)

    def submit(self, seq_id: int, prompt, temperature: float = 0.0, top_k=None, top_p=None,
               max_tokens: int = 16, stop_tokens=(), seed: int = 0) -> None:
        prompt_arr, n = native.u32_array(prompt)
        stop_arr, stops = native.u32_array(stop_tokens)
        native.check(self._lib.plh_sched_submit(
            self._h, seq_id, prompt_arr, n, float(temperature), 0 if top_k is None else 1, int(top_k or 0),
            0 if top_p is None else 1, float(top_p if top_p is not None else 1.0), int(max_tokens),
            stop_arr, stops, seed & (2 ** 64 - 1)))

    def plan(self) -> Plan:
        sizes = (ctypes.c_size_t * 4)()
        kind = native.check(self._lib.plh_sched_plan(self._h, sizes))
        return self._read_plan(kind, sizes, 0)

    def _read_plan(self, kind: int, sizes, which: int) -> Plan:
        n_entries, n_tokens, n_ids, n_adv = (int(x) for x in sizes)
        u64, i32, u32 = ctypes.c_uint64, ctypes.c_int, ctypes.c_uint32
        e_id, e_start, e_len = (u64 * max(n_entries, 1))(), (i32 * max(n_entries, 1))(), (i32 * max(n_entries, 1))()
        e_want, e_slot, e_fresh = (i32 * max(n_entries, 1))(), (i32 * max(n_entries, 1))(), (i32 * max(n_entries, 1))()
        e_fed = (i32 * max(n_entries, 1))()
        tokens = (u32 * max(n_tokens, 1))()
        ids = (u64 * max(n_ids, 1))()
        a_id, a_n = (u64 * max(n_adv, 1))(), (i32 * max(n_adv, 1))()
        refused = u64(0)
        self._lib.plh_sched_plan_read(self._h, which, e_id, e_start, e_len, e_want, e_slot, e_fresh, e_fed, tokens,
                                      ids, a_id, a_n, ctypes.byref(refused))
        entries, at = [], 0
        for i in range(n_entries):
            count = e_len[i]
            entries.append(StepEntry(int(e_id[i]), list(tokens[at:at + count]), e_start[i],
                                     [count - 1] if e_want[i] else [], e_slot[i], bool(e_fresh[i]), e_fed[i]))
            at += count
        return Plan(kind, [int(x) for x in ids[:n_ids]], [(int(a_id[i]), a_n[i]) for i in range(n_adv)],
                    entries, int(refused.value))

    def launched(self) -> None:
        """The planned step is queued on the device: what it writes is there for everything queued behind
        it, so the lengths in the cache move now.  (``commit`` does this itself where nobody has.)"""
        native.check(self._lib.plh_sched_launched(self._h))

    def plan_ahead(self):
        """The step behind a launched decoding step, before that step's tokens are known: rows for the
        residents as the planner would seat them.  A request with a row in the launched step, which that
        step can only end by a stop token, is fed the token of its row there on the device
        (``StepEntry.fed_row``); one without (there were more residents than rows) brings the token it
        holds.  None when the next step is not known yet: the front of the queue can come in or is to be
        turned away, a prompt is part-way in, or pages have run out.  Once the step before is committed,
        the step planned ahead is the planned step: it is committed next, and ``plan`` may not be asked
        before."""
        sizes = (ctypes.c_size_t * 4)()
        if not native.check(self._lib.plh_sched_plan_ahead(self._h, sizes)):
            return None
        return self._read_plan(DECODE, sizes, 1)

    def drop_ahead(self) -> None:
        """Forget the step planned ahead: it was not launched after all."""
        self._lib.plh_sched_drop_ahead(self._h)

    def abandon(self) -> None:
        """The planned step failed and will not be committed: forget it and any step planned ahead of it
        (the caller cancels its requests)."""
        self._lib.plh_sched_abandon(self._h)

    def _read_outcome(self, sizes) -> Outcome:
        n_tok, n_fin = int(sizes[0]), int(sizes[1])
        u64, i32, u32 = ctypes.c_uint64, ctypes.c_int, ctypes.c_uint32
        t_id, t_tok = (u64 * max(n_tok, 1))(), (u32 * max(n_tok, 1))()
        f_id, f_fin = (u64 * max(n_fin, 1))(), (i32 * max(n_fin, 1))()
        f_prompt, f_gen, f_pre = (u64 * max(n_fin, 1))(), (u64 * max(n_fin, 1))(), (u32 * max(n_fin, 1))()
        self._lib.plh_sched_outcome_read(self._h, t_id, t_tok, f_id, f_fin, f_prompt, f_gen, f_pre)
        return Outcome(
            [(int(t_id[i]), int(t_tok[i])) for i in range(n_tok)],
            [Finished(int(f_id[i]), FINISH_NAMES[f_fin[i]], int(f_prompt[i]), int(f_gen[i]), int(f_pre[i]))
             for i in range(n_fin)])

    def commit(self, sampled) -> Outcome:
        """Record that the planned step ran.  ``sampled`` is one token per id of the plan."""
        arr, n = native.u32_array(sampled)
        sizes = (ctypes.c_size_t * 2)()
        native.check(self._lib.plh_sched_commit(self._h, arr, n, sizes))
        return self._read_outcome(sizes)

    def drain_finished(self) -> Outcome:
        sizes = (ctypes.c_size_t * 2)()
        native.check(self._lib.plh_sched_drain_finished(self._h, sizes))
        return self._read_outcome(sizes)

    def cancel(self, seq_id: int) -> None:
        native.check(self._lib.plh_sched_cancel(self._h, seq_id))

    def sample_on_host(self, seq_id: int, logits_row) -> int:
        """One token from a row of 32-bit logits (a numpy array), with the
        request's own parameters and generator."""
        return native.check(self._lib.plh_sched_sample(self._h, seq_id, logits_row.ctypes.data, logits_row.size))

    def sampling_of(self, seq_id: int):
        """(temperature, top_k, top_p, uniform): what a device sampler needs.  For a
        request that draws, ``uniform`` is the next number of its generator."""
        t, k, p, u = ctypes.c_float(), ctypes.c_int(), ctypes.c_float(), ctypes.c_float()
        native.check(self._lib.plh_sched_sampling_of(self._h, seq_id, ctypes.byref(t), ctypes.byref(k),
                                                     ctypes.byref(p), ctypes.byref(u)))
        return t.value, k.value, p.value, u.value

    @property
    def waiting(self) -> int:
        return self._lib.plh_sched_waiting(self._h)

    @property
    def running(self) -> int:
        return self._lib.plh_sched_running(self._h)

    def running_ids(self) -> list:
        buf = (ctypes.c_uint64 * 4096)()
        n = self._lib.plh_sched_running_ids(self._h, buf, 4096)
        return [int(x) for x in buf[:min(n, 4096)]]

    def wasted_tokens(self) -> int:
        return self._lib.plh_sched_wasted_tokens(self._h)

    def metrics(self) -> dict:
        out = (ctypes.c_uint64 * len(_METRICS))()
        self._lib.plh_sched_metrics(self._h, out)
        m = {name: int(out[i]) for i, name in enumerate(_METRICS)}
        asked = m["cached_tokens"] + m["prefilled_tokens"]
        m["prefix_hit_rate"] = m["cached_tokens"] / asked if asked else 0.0
        m["mean_batch"] = m["decode_rows"] / m["decode_steps"] if m["decode_steps"] else 0.0
        return m
