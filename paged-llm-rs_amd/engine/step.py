"""The step function: run the tokens a step brings, as one batch, from the
cache, and return the logits at the wanted places (reference:
model/mod.rs:305-352).  Pages are written; the lengths in the cache manager do
not move: whoever asked for the step records it once it has succeeded.

A step in which every request brings exactly one token (plain decoding) is
launch-bound: some two hundred small kernels.  Such steps are captured once as a
HIP graph over static buffers, per (requests, pages a request) bucket, and
replayed; the descriptor of the step is written into a pinned host buffer by the
native cache manager and copied in with one transfer.

A plain decoding step may be launched before the host has read the tokens of
the one before: an entry then names the row of that step whose chosen token it
feeds (``StepEntry.fed_row``), and the embedding takes the id from the buffer
that every decoding step's argmax writes.  The chosen tokens also travel to
pinned memory behind every decoding step, so that reading those of one step does
not wait for the next, which is already queued behind it.

Any other step costs the host some five milliseconds to launch, which is more
than the GPU needs for a portion of a few hundred tokens.  Such steps are
padded with rows that belong to no request up to a bucket of tokens, so that
steps of many lengths have few shapes (rows, requests, wanted places); a shape
that comes a second time is captured too and replayed from then on, and a few
such graphs are kept.  A shape seen once runs eagerly, padded alike.  All ways
run the same model code and the same kernels.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Optional

import numpy as np
import torch

from .. import kernels
from ..errors import ConfigError, PagedLLMError, TensorError
from .batch import CannotFeed, CaptureOutgrown, StepBatch, TableTooWide, build_batch, context_bound, token_bucket

GRAPH_MAX_REQUESTS = 256     # requests a captured step may have (steps of more run kernel by kernel)
SHAPE_GRAPH_ROWS_KEPT = 32768    # rows over all captured shapes of steps other than plain decoding (the
                                 # least recently used go first): their buffers stay allocated
SHAPE_GRAPH_MAX_TOKENS = 8192


def require_gpu(device) -> torch.device:
    device = torch.device(device)
    if device.type != "cuda" or not torch.cuda.is_available():
        raise TensorError("the engine runs on the GPU only; no GPU is visible to this process")
    return device


def run_step(model, cache, entries, check_start: bool = True, pad_to: int | None = None,
             short_bounds: dict | None = None, trace: dict | None = None) -> torch.Tensor:
    """32-bit logits [wanted places, vocabulary], in the order of the entries and of their ``want``.
    ``trace`` receives the named activations of the step (32-bit models; see ``DecoderModel.forward``)."""
    batch = build_batch(entries, cache.manager, len(cache.layout.groups), model.spec.vocab_size,
                        model.spec.max_positions, model.device, check_start=check_start, pad_to=pad_to,
                        short_bounds=short_bounds)
    for e in entries:
        if e.fresh_state and e.state_slot >= 0:
            cache.clear_state_slot(e.state_slot)
    if trace is not None:
        return model.forward(batch, cache, trace=trace)
    return model.forward(batch, cache)


def commit_step(cache, entries) -> None:
    """Record that the step ran: every request has its tokens written."""
    for e in entries:
        cache.manager.advance(e.seq_id, len(e.tokens))


@dataclass
class StepOutput:
    """What a step left on the device.  The tensors of a captured step are the graph's own: the next step
    of the same kind overwrites them."""
    logits: torch.Tensor                      # [wanted, vocabulary], 32-bit, on the device
    # [wanted] int32 on the device, when already computed: the largest logit's index of every row, or what
    # the ``choose`` that the step was run with put in its place
    greedy: Optional[torch.Tensor] = None
    sent: Optional[torch.Tensor] = None       # the same in pinned memory, once ``arrived`` has passed
    arrived: Optional[torch.cuda.Event] = None

    def greedy_tokens(self) -> torch.Tensor:
        if self.greedy is None:
            self.greedy = kernels.argmax(self.logits)
        return self.greedy

    def greedy_on_host(self) -> list:
        """The chosen token of every wanted row (see ``greedy``), as a list.  Waits for this step only,
        where the step sent its tokens to the host itself."""
        if self.sent is not None:
            self.arrived.synchronize()
            return self.sent.tolist()
        return self.greedy_tokens().cpu().tolist()


def _bucket(n: int, least: int = 1) -> int:
    b = least
    while b < n:
        b *= 2
    return b


def _all_idle(host: torch.Tensor, layout: dict) -> torch.Tensor:
    """A copy of a step's descriptor in which every row is padding: position -1, no context, no state slot, no
    pages.  The rows, the requests they belong to and the wanted places stay, so the step has the same shape;
    a step of such rows reads and writes nothing that belongs to a request."""
    idle = host.clone()
    for name, (begin, count) in layout.items():
        if name == "token_ids":
            idle[begin:begin + count] = 0
        elif name == "ctx_len":
            idle[begin:begin + count] = 0
        elif name in ("positions", "state_slots") or name.startswith("block_table_"):
            idle[begin:begin + count] = -1
    return idle


class _DescriptorRing:
    """Pinned buffers for a graph's step descriptor, used in turn.  A descriptor travels to the device without
    the host waiting, so the copy of one step has to have left its buffer before that buffer is written again.
    A caller that reads every step's result has waited already; one that does not (a portion in the middle of
    a prompt gives nothing to read) would overwrite a descriptor that the device has not yet fetched.  An
    event after every copy would guard that, at some microseconds a step; here an event is recorded after the
    copy from the last buffer of a lap and waited for before the first buffer is written again: copies run
    in the order of the stream, so all of the lap's copies are done by then."""

    LAP = 8

    def __init__(self, size: int):
        self.buffers = [torch.zeros(size, dtype=torch.int32).pin_memory() for _ in range(self.LAP)]
        self.views = [b.numpy() for b in self.buffers]
        self.at = 0
        self.event = None

    def advance(self) -> None:
        """Go on to the buffer that the next step is written into."""
        self.at = (self.at + 1) % self.LAP
        if self.at == 0 and self.event is not None:
            self.event.synchronize()

    @property
    def host(self) -> torch.Tensor:
        return self.buffers[self.at]

    @property
    def view(self):
        return self.views[self.at]

    def sent(self) -> None:
        """After the copy of the current buffer has been put on the stream."""
        if self.at == self.LAP - 1:
            if self.event is None:
                self.event = torch.cuda.Event()
            self.event.record()


class DecodeGraph:
    """One decode step for up to ``cap`` requests with up to ``widths[g]`` pages each, captured; or, with
    ``captured=False``, launched kernel by kernel over the same buffers with the same idle rows, so that a
    runner without graphs computes what one with graphs replays.  The chosen tokens go into the first
    ``cap`` places of ``chosen``, the runner's buffer, where the next decoding step (of this graph or of
    another of the runner's) finds the tokens that are fed to it on the device."""

    def __init__(self, model, cache, cap: int, widths: list, chosen: torch.Tensor, captured: bool = True):
        self.model, self.cache, self.cap, self.widths = model, cache, cap, list(widths)
        self.captured = captured
        self.feeds = bool(getattr(model, "takes_fed_tokens", False))
        pieces = [("token_ids", cap), ("positions", cap), ("seq_of", cap), ("q_start", cap), ("q_len", cap),
                  ("ctx_len", cap), ("state_slots", cap), ("logit_rows", cap)]
        if self.feeds:
            pieces.append(("token_src", cap))
        pieces += [(f"block_table_{g}", cap * w) for g, w in enumerate(widths)]
        self.layout, offset = {}, 0
        for name, count in pieces:
            self.layout[name] = (offset, count)
            offset += (count + 3) // 4 * 4
        self.ring = _DescriptorRing(offset)
        self.sent = [torch.zeros(cap, dtype=torch.int32).pin_memory() for _ in range(self.ring.LAP)]
        self.arrived = [torch.cuda.Event() for _ in range(self.ring.LAP)]
        self.ids = np.zeros(cap, dtype=np.uint64)
        self.device_buf = torch.zeros(offset, dtype=torch.int32, device=model.device)
        block_size = cache.block_size
        self.batch = StepBatch(self.device_buf, self.layout, cap, cap, list(widths), cap, 1,
                               context_bound(max(widths or [1]) * block_size), [])
        self.all_chosen = chosen
        self.tokens = chosen[:cap]
        if self.feeds:
            self.batch.fed_tokens = chosen
        for _ in range(self.ring.LAP):         # what no step changes, in every buffer
            h = self.ring.view
            for name in ("seq_of", "q_start", "logit_rows"):
                b, c = self.layout[name]
                h[b:b + c] = np.arange(cap, dtype=np.int32)
            b, c = self.layout["q_len"]
            h[b:b + c] = 1
            self._idle_rows(0)
            self.ring.advance()
        self.graph = None
        self.logits = None

    def _view(self, name):
        b, c = self.layout[name]
        return self.ring.view[b:b + c]

    def _idle_rows(self, live: int) -> None:
        """Rows past the live requests are padding: position -1, no pages."""
        self._view("token_ids")[live:] = 0
        if self.feeds:
            self._view("token_src")[live:] = -1
        self._view("positions")[live:] = -1
        self._view("ctx_len")[live:] = 0
        self._view("state_slots")[live:] = -1
        for g, w in enumerate(self.widths):
            self._view(f"block_table_{g}").reshape(self.cap, w)[live:] = -1

    def _forward(self):
        logits = self.model.forward(self.batch, self.cache)
        kernels.argmax(logits, out=self.tokens)
        return logits

    def capture(self) -> None:
        # The run before the capture (everything that initialises lazily does so there, outside the capture)
        # and the capture itself see a step of idle rows only: they write no page and touch no request's
        # state, so the one replay that follows is the only time the real step runs.  (A mixer that keeps
        # state of its own would otherwise advance it twice on the step that brings a capture about.)
        # Both overwrite the chosen tokens of the step before, which is why a step that is fed from them
        # is never the one that brings a capture about.
        self.device_buf.copy_(_all_idle(self.ring.host, self.layout))
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            self._forward()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        self.graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(self.graph):
            self.logits = self._forward()

    def fill(self, entries) -> None:
        """Write the step's descriptor into the pinned buffer.  Raises TableTooWide when a request has
        outgrown the rows of this graph's block table."""
        live = len(entries)
        manager = self.cache.manager
        self.ids[:live] = [e.seq_id for e in entries]
        positions = self._view("positions")
        manager.fill_step(self.ids.ctypes.data, live, positions.ctypes.data, 0, 0, 0)
        for g, w in enumerate(self.widths):
            pages = manager.fill_step(self.ids.ctypes.data, live, 0, g, self._view(f"block_table_{g}").ctypes.data, w)
            if pages:
                raise TableTooWide(g, pages)
        tokens = self._view("token_ids")
        tokens[:live] = [e.tokens[0] for e in entries]
        if self.feeds:
            self._view("token_src")[:live] = [e.fed_row for e in entries]
        vocab, limit = self.model.spec.vocab_size, self.model.spec.max_positions
        if tokens[:live].min() < 0 or tokens[:live].max() >= vocab:
            raise ConfigError(f"a token id outside the vocabulary of {vocab}")
        if limit and positions[:live].max() >= limit:
            raise ConfigError(f"position {int(positions[:live].max())} is past the model's {limit}")
        self._view("ctx_len")[:live] = positions[:live] + 1
        self._view("state_slots")[:live] = [e.state_slot for e in entries]
        self._idle_rows(live)

    def run(self, entries, fed: bool = False, choose=None) -> StepOutput:
        """``fed``: some entry takes its token from the chosen tokens of the step before.  Raises
        CannotFeed, before anything is launched, where this step would overwrite them first.
        ``choose(logits, out)``: called behind the step to put other tokens than the largest logits'
        into ``out`` ([live] int32), which is what travels to the host and what a step behind is fed."""
        live = len(entries)
        if fed and (not self.feeds or (self.captured and self.graph is None)):
            raise CannotFeed("this step has to be captured first, which overwrites the chosen tokens")
        self.ring.advance()
        self.fill(entries)
        if self.captured and self.graph is None:
            self.capture()
        self.device_buf.copy_(self.ring.host, non_blocking=True)
        self.ring.sent()
        if self.captured:
            self.graph.replay()
            logits = self.logits
        else:
            logits = self._forward()
        if choose is not None:
            choose(logits[:live], self.tokens[:live])
        sent, arrived = self.sent[self.ring.at], self.arrived[self.ring.at]
        sent.copy_(self.tokens, non_blocking=True)
        arrived.record()
        return StepOutput(logits[:live], self.tokens[:live], sent[:live], arrived)


class ShapeGraph:
    """A step of one shape (rows after padding, requests, wanted places), with block tables of
    ``widths`` pages a row and contexts up to ``ctx_bound``, captured."""

    def __init__(self, model, cache, entries, widths: list, ctx_bound: int, rows: int, short_bounds: dict):
        self.model, self.cache, self.widths, self.ctx_bound, self.rows = model, cache, list(widths), ctx_bound, rows
        self.short_bounds = dict(short_bounds)
        first = self._lay_out(entries)
        self.size = first.packed.numel()
        self.ring = _DescriptorRing(self.size)
        self.device_buf = torch.zeros(self.size, dtype=torch.int32, device=model.device)
        self.ring.host.copy_(first.packed)
        self.layout = first.layout
        self.batch = StepBatch(self.device_buf, first.layout, first.num_tokens, first.num_seqs, list(widths),
                               first.num_logit_rows, first.max_q_len, ctx_bound, [],
                               tokens_each=first.tokens_each, padded=True, short_bounds=first.short_bounds)
        self.batch.live_seqs = first.live_seqs
        self.graph = None
        self.logits = None

    def _lay_out(self, entries):
        return build_batch(entries, self.cache.manager, len(self.cache.layout.groups), self.model.spec.vocab_size,
                           self.model.spec.max_positions, "cpu", widths=self.widths, ctx_bound=self.ctx_bound,
                           pad_to=self.rows, short_bounds=self.short_bounds)

    def capture(self) -> None:
        # (over a step of idle rows, as in DecodeGraph.capture: the real step runs once, in the replay)
        self.device_buf.copy_(_all_idle(self.ring.host, self.layout))
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            self.model.forward(self.batch, self.cache)     # lazy initialisation happens outside the capture
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        self.graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(self.graph):
            self.logits = self.model.forward(self.batch, self.cache)

    def run(self, entries) -> StepOutput:
        """Raises CaptureOutgrown when the step no longer fits what was captured."""
        if self.graph is not None:
            batch = self._lay_out(entries)
            if batch.packed.numel() != self.size:
                raise ConfigError("a step of another shape than the captured one")
            self.ring.advance()
            self.ring.host.copy_(batch.packed)
        else:
            self.capture()
        self.device_buf.copy_(self.ring.host, non_blocking=True)
        self.ring.sent()
        self.graph.replay()
        return StepOutput(self.logits)


class StepRunner:
    """Runs steps for one model and cache, keeping the captured graphs."""

    def __init__(self, model, cache, graphs: bool = True):
        self.model, self.cache = model, cache
        self.use_graphs = graphs and getattr(model, "graph_safe", True)
        # A model whose parts all take padding rows gets its steps padded whether graphs are on or not,
        # so that a step launches the same kernels either way.
        self.pads = getattr(model, "graph_safe", True)
        self._graphs: dict = {}
        self._shapes: dict = {}          # shape of a step -> ShapeGraph, or None after its first (eager) run
        self.graph_steps = 0
        self.eager_steps = 0
        # Every decoding step leaves its chosen tokens here, row by row, for a step launched behind it to
        # take its ids from; ``_feedable`` is how many of them the last step left (0: it was no such step).
        self._chosen = torch.zeros(GRAPH_MAX_REQUESTS, dtype=torch.int32, device=model.device)
        self._feedable = 0

    def _is_plain_decode(self, entries) -> bool:
        return ((self.use_graphs or self.pads) and 0 < len(entries) <= GRAPH_MAX_REQUESTS
                and all(len(e.tokens) == 1 and e.want == [0] for e in entries))

    def _run_shaped(self, entries) -> StepOutput:
        """A step other than plain decoding: eagerly the first time its shape comes, from a captured
        graph from the second time on (while the requests' tables and contexts fit the capture)."""
        tokens = sum(len(e.tokens) for e in entries)
        rows = token_bucket(tokens) if self.pads and tokens <= SHAPE_GRAPH_MAX_TOKENS else None
        # For every limit below which a mixer of the model runs a request through a kernel of its own: the
        # tokens of such requests, rounded up (that kernel gets so many workgroups).  Part of the shape.
        short_bounds = None
        if rows is not None:
            short_bounds = {}
            for limit in getattr(self.model, "portion_limits", ()):
                short = sum(len(e.tokens) for e in entries if len(e.tokens) < limit)
                short_bounds[limit] = min(rows, _bucket(short, 16)) if short else 0
        if not self.use_graphs or rows is None or len(entries) > GRAPH_MAX_REQUESTS:
            self.eager_steps += 1
            return StepOutput(run_step(self.model, self.cache, entries, pad_to=rows, short_bounds=short_bounds))
        shape = (rows, len(entries), sum(len(e.want) for e in entries), tuple(sorted(short_bounds.items())))
        known = shape in self._shapes
        graph = self._shapes.pop(shape, None)
        if not known:
            self._shapes[shape] = None          # seen once
            while len(self._shapes) > 256:
                self._shapes.pop(next(iter(self._shapes)))
            self.eager_steps += 1
            return StepOutput(run_step(self.model, self.cache, entries, pad_to=rows, short_bounds=short_bounds))
        for e in entries:
            if e.fresh_state and e.state_slot >= 0:
                self.cache.clear_state_slot(e.state_slot)
        if graph is not None:
            try:
                out = graph.run(entries)
                self._shapes[shape] = graph     # most recently used last
                self.graph_steps += 1
                return out
            except CaptureOutgrown:
                pass                            # a request has outgrown the capture: a new one below
        widths = [_bucket(w + 1, 32) for w in self._widths_needed(entries)]
        longest = max(e.start + len(e.tokens) for e in entries)
        graph = ShapeGraph(self.model, self.cache, entries, widths, context_bound(longest), rows, short_bounds)
        out = graph.run(entries)
        self._shapes[shape] = graph
        live = [k for k, g in self._shapes.items() if g is not None]
        held = sum(k[0] for k in live)
        for k in live[:-1]:
            if held <= SHAPE_GRAPH_ROWS_KEPT:
                break
            held -= k[0]
            del self._shapes[k]
        self.graph_steps += 1
        return out

    def _widths_needed(self, entries) -> list:
        manager = self.cache.manager
        return [max(len(manager.table(e.seq_id, g)) for e in entries) for g in range(len(self.cache.layout.groups))]

    def run(self, entries, choose=None) -> StepOutput:
        """Raises CannotFeed, with nothing launched, when an entry is to be fed on the device
        (``fed_row``) and this step cannot take it so: it is no plain decoding step, the step before was
        none or had no such row, or its graph has to be captured (again) first.

        ``choose(logits, out)``: for a plain decoding step, what picks the tokens instead of the largest
        logit (``DecodeGraph.run``); it is called only once the step is on the device, and not at all for
        any other step, whose output then has no chosen tokens."""
        entries = list(entries)
        if not entries:
            raise ConfigError("an empty batch")
        fed = any(e.fed_row >= 0 for e in entries)
        if not self._is_plain_decode(entries):
            if fed:
                raise CannotFeed("only a step of single tokens takes them from the step before")
            self._feedable = 0
            return self._run_shaped(entries)
        if len({e.seq_id for e in entries}) != len(entries):
            raise ConfigError("a request appears twice in one step")
        if fed and max(e.fed_row for e in entries) >= self._feedable:
            raise CannotFeed(f"the step before chose {self._feedable} tokens")
        for e in entries:
            if e.fresh_state and e.state_slot >= 0:
                self.cache.clear_state_slot(e.state_slot)
        cap = _bucket(len(entries))
        graph = self._graphs.get(cap)
        if graph is not None:
            try:
                out = graph.run(entries, fed, choose)
                self._count(graph)
                self._feedable = len(entries)
                return out
            except TableTooWide:
                pass
        if fed:
            raise CannotFeed("a step of this many requests and pages has to be captured first")
        # no graph for this many requests yet, or a request has outgrown the bucket's table
        widths = [_bucket(w + 1, 32) for w in self._widths_needed(entries)]
        graph = DecodeGraph(self.model, self.cache, cap, widths, self._chosen, captured=self.use_graphs)
        self._graphs[cap] = graph
        out = graph.run(entries, False, choose)
        self._count(graph)
        self._feedable = len(entries)
        return out

    def _count(self, graph) -> None:
        if graph.captured:
            self.graph_steps += 1
        else:
            self.eager_steps += 1
