"""The engine loop and the Python entry point.

One iteration (reference: crates/pagedllm-server/src/engine.rs:180-250): ask the
scheduler for a plan, run the step function, choose a token for every request a
token comes back for, commit.  A failed step fails the requests in it and
commits nothing; lengths only move once a step is on the device.  While only
decoding goes on, the step after is queued before this one's tokens are read
(``Engine._launch_ahead``).
"""

from __future__ import annotations

import itertools
import time
from dataclasses import dataclass, field
from pathlib import Path
from typing import Optional

import numpy as np
import torch

from .. import kernels
from ..cache import PagedCache
from ..config import GenerationConfig
from ..errors import ConfigError, PagedLLMError
from ..parts.model import DTYPES, load_model
from ..sampling.sampler import Sampling
from ..weights.loader import CheckpointFiles
from . import scheduler as sched
from .batch import CannotFeed
from .step import StepRunner, require_gpu

_seed_counter = itertools.count()


def default_seed() -> int:
    """A seed for a request that names none: the clock mixed with a counter, so two
    requests in the same second do not draw the same tokens (reference: routes.rs:69-80)."""
    n = next(_seed_counter)
    return (int(time.time()) * 0x9E3779B97F4A7C15 + n * 0xBF58476D1CE4E5B9) & (2 ** 64 - 1)


def checkpoint_dtype(model_dir) -> str:
    """``auto``: whatever the checkpoint stores its embedding in (reference: model/mod.rs:175)."""
    f = CheckpointFiles(model_dir)
    try:
        for name in f.names():
            if name.endswith("embed_tokens.weight"):
                return "float32" if f.dtype(name) in (torch.float32, torch.float64) else "bfloat16"
    finally:
        f.close()
    return "bfloat16"


@dataclass
class Completion:
    """What a finished request returns."""
    tokens: list = field(default_factory=list)
    finish: str = ""
    prompt_tokens: int = 0
    preemptions: int = 0


class Engine:
    """A model, its cache and its scheduler on one GPU.

    The options carry the names and meanings of the reference's command line
    (crates/pagedllm-server/src/main.rs:20-71): ``dtype`` auto|f32|bf16,
    ``block_size`` (16), ``cache_mib`` (3584), ``max_batch`` (16), ``prefix_cache``
    (on), ``chunk`` (128; None or "off" runs a prompt whole), ``max_tokens`` (512,
    the budget of a request that names none).  ``num_blocks`` sets the pool
    directly instead of ``cache_mib``.

    ``strips``: the weights are kept a second time in the order the products of a decoding step read them
    fastest (``kernels.weights_in_strips``), which costs their memory again.

    ``ahead``: while nothing but decoding is going on (and the tokens are chosen on the device: not with
    ``sampler="host"``), the next step is queued on the device before the tokens of the one before have been read (they are fed to it on the device), so the
    device does not wait for the host between steps.  The tokens a request gets do not depend on it;
    a request that arrives meanwhile is admitted one step later, and the row of a request that a
    stop token has just ended runs once more for nothing.
    """

    def __init__(self, model, dtype: str = "auto", block_size: int = 16, cache_mib: int = 3584,
                 num_blocks: Optional[int] = None, max_batch: int = 16, chunk=128, prefix_cache: bool = True,
                 max_tokens: int = 512, device="cuda:0", sampler: str = "device", graphs: bool = True,
                 ahead: bool = True, strips: bool = True):
        self.device = require_gpu(device)
        dtype = {"auto": None, "f32": "float32", "bf16": "bfloat16"}.get(dtype, dtype)
        if dtype is None:
            dtype = checkpoint_dtype(model)
        if dtype not in ("float32", "bfloat16"):
            raise ConfigError(f"dtype {dtype!r}, which is none of auto, f32, bf16")
        if chunk == "off":
            chunk = None
        if chunk is not None and int(chunk) < 1:
            raise ConfigError("--chunk 0 would carry nothing")
        if sampler not in ("device", "host"):
            raise ConfigError(f"sampler {sampler!r}, which is neither device nor host")
        self.dtype = dtype
        self.model_dir = Path(model)
        self.config, self.model = load_model(model, dtype, self.device, strips=strips)
        self.generation = GenerationConfig.from_dir(model)
        element = 4 if dtype == "float32" else 2
        layout = self.model.cache_layout
        if num_blocks is None:
            # The page count follows from the byte budget, so changing the page
            # size compares two layouts at the same memory (reference: main.rs:89-120).
            num_blocks = layout.blocks_within(int(cache_mib) << 20, block_size, element)
        self.block_size, self.num_blocks = block_size, num_blocks
        self.bytes_per_token = layout.bytes_per_token(element)
        self.cache = PagedCache(layout, block_size, num_blocks, DTYPES[dtype], self.device,
                                max_seqs=max(max_batch * 2, 8))
        self.scheduler = sched.Scheduler(self.cache.manager, max_batch=max_batch,
                                         chunk=None if chunk is None else int(chunk),
                                         max_positions=self.model.spec.max_positions, prefix_cache=prefix_cache)
        self.runner = StepRunner(self.model, self.cache, graphs=graphs)
        # Pages are shared between requests only where every layer keeps all its keys in pages of one size and
        # no layer keeps state of its own beside them (a window's pages are given back, a state is not in pages):
        # asked for and not possible is said, in the banner and in the metrics, not passed over.
        self.prefix_cache = "on" if prefix_cache else "off"
        if prefix_cache and not self.cache.manager.sharing_possible():
            self.prefix_cache = "off (asked for; this model's layers keep a window of their keys or state of their own)"
        self.default_max_tokens = max_tokens
        self.sampler = sampler
        # (a model class whose embedding does not take ids from the device is never fed a step ahead)
        self.ahead = bool(ahead) and bool(getattr(self.model, "takes_fed_tokens", False))
        self._flight = None      # (plan, output) of a step that is on the device and not yet committed
        self.steps_ahead = 0     # steps that were launched before the tokens of the one before were read
        self._next_id = 1
        self._results: dict = {}
        self._open: dict = {}
        self._greedy: dict = {}
        self._chunk = None if chunk is None else int(chunk)

    # -- requests -------------------------------------------------------------------------

    def resolve_sampling(self, temperature=None, top_k=None, top_p=None) -> Sampling:
        """The request's value, else the model's generation config, else temperature 1;
        an explicit temperature of zero drops top-k and top-p (reference: routes.rs:106-126)."""
        if temperature is None:
            temperature = self.generation.temperature if self.generation.temperature is not None else 1.0
        if temperature <= 0.0:
            return Sampling(float(temperature), None, None)
        return Sampling(float(temperature), top_k if top_k is not None else self.generation.top_k,
                        top_p if top_p is not None else self.generation.top_p)

    def submit(self, prompt, max_tokens: Optional[int] = None, temperature=0.0, top_k=None, top_p=None,
               seed: Optional[int] = None, stop_tokens=None) -> int:
        prompt = [int(t) for t in prompt]
        if not prompt:
            raise ConfigError("cannot generate from an empty prompt")
        vocab = self.model.spec.vocab_size
        if min(prompt) < 0 or max(prompt) >= vocab:
            raise ConfigError(f"a prompt token outside the vocabulary of {vocab}")
        how = self.resolve_sampling(temperature, top_k, top_p)
        stops = list(self.generation.eos_token_ids) if stop_tokens is None else [int(t) for t in stop_tokens]
        seq_id = self._next_id
        self._next_id += 1
        self.scheduler.submit(seq_id, prompt, how.temperature, how.top_k, how.top_p,
                              self.default_max_tokens if max_tokens is None else int(max_tokens), stops,
                              default_seed() if seed is None else int(seed))
        self._open[seq_id] = Completion(prompt_tokens=len(prompt))
        self._greedy[seq_id] = how.is_greedy
        return seq_id

    def cancel(self, seq_id: int) -> None:
        self.scheduler.cancel(seq_id)
        self._open.pop(seq_id, None)

    # -- the loop ---------------------------------------------------------------------------

    def _draw_on_device(self, ids, logits, out=None, out_holds_largest: bool = False) -> torch.Tensor:
        """One token per row of ``logits`` by the sampling kernel, each with its request's parameters and the
        next number of the request's generator (a greedy row takes its largest logit and draws nothing).
        ``out_holds_largest``: ``out`` already holds the rows' largest logits' places (``kernels.sample``)."""
        how = [self.scheduler.sampling_of(i) for i in ids]     # (draws the number of every request that samples)
        # one transfer: temperatures, top-k, top-p and the drawn numbers as the four rows of one 32-bit array
        # (the 32-bit floats as their bits), of which the kernel's arguments are views
        packed = np.empty((4, len(how)), dtype=np.int32)
        as_float = packed.view(np.float32)
        for col, (t, k, p, u) in enumerate(how):
            as_float[0, col], packed[1, col], as_float[2, col], as_float[3, col] = t, k, p, u
        params = torch.from_numpy(packed).pin_memory().to(logits.device, non_blocking=True)
        return kernels.sample(logits, params[0].view(torch.float32), params[1], params[2].view(torch.float32),
                              params[3].view(torch.float32), out=out, out_holds_largest=out_holds_largest)

    def _chooser(self, plan):
        """What a decoding step of ``plan`` is run with (``StepRunner.run``): nothing where every request
        takes its largest logit or the host samples; else the sampling kernel, behind the step."""
        if self.sampler != "device" or all(self._greedy.get(i, True) for i in plan.ids):
            return None
        # (behind a decoding step the tokens are the largest logits' when the chooser is called)
        return lambda logits, out: self._draw_on_device(plan.ids, logits, out, out_holds_largest=True)

    def _choose(self, plan, output) -> list:
        """One token per id of the plan.  On the device (the default) greedy rows are an argmax and
        the others are drawn by the sampling kernel with the next number of the request's generator;
        with ``sampler="host"`` the logits go to the host sampler instead."""
        if not plan.ids:
            return []      # a portion in the middle of a prompt: the logits have no rows and are not touched
        logits = output.logits
        if logits.shape[0] != len(plan.ids):
            raise PagedLLMError(f"{logits.shape[0]} rows of logits for {len(plan.ids)} requests")
        if self.sampler == "device":
            if output.sent is not None or all(self._greedy.get(i, True) for i in plan.ids):
                return output.greedy_on_host()     # chosen behind the step already, or largest logits
            return self._draw_on_device(plan.ids, logits).cpu().tolist()
        host = logits.cpu().numpy()
        return [self.scheduler.sample_on_host(i, host[row]) for row, i in enumerate(plan.ids)]

    def step(self):
        """One iteration.  Returns the outcome, or None when there is nothing to run."""
        if self._flight is not None:
            plan, output = self._flight       # launched during the step before; by now the planned step
            self._flight = None
        else:
            plan = self.scheduler.plan()
            if plan.kind == sched.IDLE:
                outcome = self.scheduler.drain_finished()
                self._record(outcome)
                return outcome if outcome.finished else None
            output = None
        sampled = []
        if plan.entries:
            try:
                if output is None:
                    output = self.runner.run(plan.entries, self._chooser(plan))
                self._launch_ahead(plan)
                sampled = self._choose(plan, output)
            except PagedLLMError:
                # A failed step fails every request in it; nothing was committed
                # (reference: engine.rs:340-348).
                self.scheduler.abandon()
                self._flight = None
                for e in plan.entries:
                    self.scheduler.cancel(e.seq_id)
                    done = self._open.pop(e.seq_id, None)
                    if done is not None:
                        done.finish = "failed"
                        self._results[e.seq_id] = done
                raise
        outcome = self.scheduler.commit(sampled)
        self._record(outcome)
        return outcome

    def _launch_ahead(self, plan) -> None:
        """With the step of ``plan`` queued on the device: queue the one behind it as well, if it is known
        without this one's tokens (see ``Scheduler.plan_ahead``) and the tokens are chosen on the device."""
        if not (self.ahead and self.sampler == "device" and plan.kind == sched.DECODE):
            return
        self.scheduler.launched()
        following = self.scheduler.plan_ahead()
        if following is None:
            return
        try:
            self._flight = (following, self.runner.run(following.entries, self._chooser(following)))
            self.steps_ahead += 1
        except CannotFeed:
            self.scheduler.drop_ahead()      # (a graph has to be captured first: the step runs the ordinary way)

    def _record(self, outcome) -> None:
        for seq_id, token in outcome.tokens:
            if seq_id in self._open:
                self._open[seq_id].tokens.append(token)
        for f in outcome.finished:
            done = self._open.pop(f.id, None)
            if done is None:
                continue
            done.finish, done.prompt_tokens, done.preemptions = f.finish, f.prompt_tokens, f.preemptions
            self._greedy.pop(f.id, None)
            self._results[f.id] = done

    @property
    def open_requests(self) -> int:
        """Requests that were submitted and have not finished."""
        return len(self._open)

    def run(self) -> None:
        """Run until every submitted request has finished."""
        while self._open:
            if self.step() is None and self._open:
                raise PagedLLMError("the scheduler idles while requests are open")
        if self._flight is not None:
            self.step()        # a step queued ahead whose requests have all ended: its tokens are dropped

    def take_result(self, seq_id: int) -> Completion:
        return self._results.pop(seq_id)

    def generate(self, prompts, max_tokens: Optional[int] = None, temperature=0.0, top_k=None, top_p=None,
                 seed: int = 0, stop_tokens=None) -> list:
        """Generate for a list of prompts (lists of token ids).  Returns, in order,
        dicts of ``tokens``, ``finish`` ("stop" or "length"), ``prompt_tokens`` and
        ``preemptions``.  Request i draws from seed + i."""
        ids = [self.submit(p, max_tokens, temperature, top_k, top_p, seed + i, stop_tokens)
               for i, p in enumerate(prompts)]
        self.run()
        out = []
        for i in ids:
            c = self.take_result(i)
            out.append({"tokens": c.tokens, "finish": c.finish, "prompt_tokens": c.prompt_tokens,
                        "preemptions": c.preemptions})
        return out

    def metrics(self) -> dict:
        m = self.scheduler.metrics()
        manager = self.cache.manager
        m.update({k: manager.counter(k) for k in
                  ("available", "total", "in_use", "cached_blocks", "handed_out", "hits", "misses", "evictions")})
        m["wasted_tokens"] = self.scheduler.wasted_tokens()
        m["prefix_cache"] = self.prefix_cache
        m["steps_ahead"] = self.steps_ahead
        return m

    def describe(self) -> str:
        """The start-up banner (reference: main.rs:133-158)."""
        chunk = self.scheduler_chunk
        stored, strips = self.model.matrix_bytes() if hasattr(self.model, "matrix_bytes") else (0, 0)
        return (
            f"paged-llm-rs_amd\n  model    {self.model_dir}\n"
            f"  backend  MI355X (gfx950), dtype {self.dtype}, chunk {chunk if chunk else 'off'}\n"
            f"  weights  {stored / 2 ** 30:.2f} GiB of matrices"
            + (f", and {strips / 2 ** 30:.2f} GiB more for their copies in strips (decoding reads those)\n" if strips else "\n") +
            f"  sampling temperature {self.generation.temperature}, top_p {self.generation.top_p}, "
            f"top_k {self.generation.top_k}, from the model's generation config\n"
            f"  stop     {self.generation.eos_token_ids}\n"
            f"  cache    {self.num_blocks} blocks of {self.block_size} tokens, "
            f"{self.cache.bytes / 2 ** 30:.2f} GiB, {self.bytes_per_token} bytes a token, "
            f"{self.num_blocks * self.block_size} tokens held at once, prefix cache {self.prefix_cache}")

    @property
    def scheduler_chunk(self):
        return self._chunk


def generate(model, prompts, max_tokens: int = 16, temperature=0.0, top_k=None, top_p=None, seed: int = 0,
             stop_tokens=None, **engine_options) -> list:
    """Load ``model`` (a folder), generate for ``prompts`` and return the completions."""
    return Engine(model, **engine_options).generate(prompts, max_tokens, temperature, top_k, top_p, seed,
                                                    stop_tokens)
