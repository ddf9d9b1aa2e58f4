"""Replay of given tokens through the engine's own model, step function, cache
and kernels.  It samples nothing and has no forward pass, cache or loader of its
own.  (The reference's nearest things are the test helpers that feed tokens
through forward_batch: tests/batching.rs:48-64, 265-297.)"""

from __future__ import annotations

import numpy as np
import torch

from ..cache import PagedCache
from ..errors import ConfigError
from ..parts.model import DTYPES, load_model
from .batch import StepEntry
from .step import StepRunner, commit_step, require_gpu, run_step


class Replayer:
    LIVE_AT_MOST = 4        # requests that a trace holds at a time

    def __init__(self, model_dir, dtype: str, max_tokens: int, block_size: int = 16, device="cuda:0",
                 max_live: int = 64, graphs: bool = True, pages: int | None = None, strips: bool = True):
        """``pages`` sets the pool's size by hand instead of deriving it from ``max_tokens``.  ``strips``: as
        in ``load_model``."""
        device = require_gpu(device)
        self.config, self.model = load_model(model_dir, dtype, device, strips=strips)
        if max_tokens < 1:
            raise ConfigError(f"--max-tokens {max_tokens}")
        # Each live request's tokens are counted rounded up to 64, so a pool of max_tokens/block_size pages
        # holds them when the page size divides 64.  With any other page size a request's last page may
        # reach past its multiple of 64: one page more for each of the requests that a trace may hold.
        tokens = (max_tokens + 63) // 64 * 64
        pages_given, pages = pages, -(-tokens // block_size)
        if 64 % block_size:
            pages += self.LIVE_AT_MOST
        if pages_given is not None:
            pages = pages_given
        self.cache = PagedCache(self.model.cache_layout, block_size, max(pages, 1), DTYPES[dtype], device,
                                max_seqs=max_live)
        self.runner = StepRunner(self.model, self.cache, graphs=graphs)
        self.ids: dict = {}
        self.next_id = 1

    def step(self, entries, end=(), trace: dict | None = None):
        """Run one step.  Returns the logits at the wanted places as a numpy
        array [wanted, vocabulary] of 32-bit floats, or None when nothing is wanted.
        ``trace`` (32-bit models) receives the step's named activations, rows in the order of the
        entries' tokens; such a step runs kernel by kernel."""
        manager = self.cache.manager
        step_entries = []
        for e in entries:
            name = e["id"]
            tokens = list(e["tokens"])
            fresh = name not in self.ids
            if fresh:
                self.ids[name] = self.next_id
                self.next_id += 1
                slot = manager.add_sequence(self.ids[name])
            else:
                slot = manager.state_slot(self.ids[name])
            seq_id = self.ids[name]
            if not manager.reserve(seq_id, len(tokens)):
                raise ConfigError(
                    f"request {name!r} needs {manager.blocks_needed(seq_id, len(tokens))} more pages and the pool "
                    f"has {manager.available()} free: --max-tokens is too small for this trace")
            step_entries.append(StepEntry(seq_id, tokens, manager.tokens(seq_id), list(e.get("want", [])),
                                          state_slot=slot, fresh_state=fresh and slot >= 0))
        logits = None
        if step_entries:
            if trace is not None:
                out = run_step(self.model, self.cache, step_entries, trace=trace)
            else:
                out = self.runner.run(step_entries).logits
            commit_step(self.cache, step_entries)
            if out.shape[0] > 0:
                logits = out.to(torch.float32).cpu().numpy().astype("<f4", copy=False)
        for name in end:
            if name in self.ids:
                manager.free_sequence(self.ids.pop(name))
        return logits
