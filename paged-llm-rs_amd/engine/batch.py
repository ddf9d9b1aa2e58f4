"""The descriptor of one step: a ragged batch of (request, its next tokens).

Portions of prompts stand beside single decoded tokens, cut anywhere.  Per token
the batch carries its id, its position and the index of its request; per request
the first row, the number of rows, the context length after the step, the state
slot and, for every cache group, the row of the block table.  Everything goes to
the device in one copy.  (Reference: batch.rs:67-275, which pads a rectangle and
builds a mask on the host instead.)
"""

from __future__ import annotations

from dataclasses import dataclass, field

import numpy as np
import torch

from ..errors import ConfigError


@dataclass
class StepEntry:
    """The next tokens of one request.  ``start`` is the position of the first;
    ``want`` lists the places among these tokens whose logits are asked for."""
    seq_id: int
    tokens: list
    start: int
    want: list = field(default_factory=list)
    state_slot: int = -1
    fresh_state: bool = False
    # For a single token that the host does not know yet: the row of the decoding step launched just before
    # whose chosen token this is (``tokens`` then holds a placeholder).  -1: ``tokens`` is what is fed.
    fed_row: int = -1


class StepBatch:
    """Device tensors of one step (all int32)."""

    def __init__(self, packed: torch.Tensor, layout: dict, num_tokens: int, num_seqs: int, max_blocks: list,
                 num_logit_rows: int, max_q_len: int, max_ctx_len: int, seq_ids: list,
                 tokens_each=None, padded: bool = False, short_bounds: dict | None = None):
        self.packed = packed
        self.layout = layout
        self.num_tokens = num_tokens
        self.num_seqs = num_seqs
        self.live_seqs = num_seqs        # without the request of padding rows at the end, if there is one
        self.num_logit_rows = num_logit_rows
        self.max_q_len = max_q_len
        self.max_ctx_len = max_ctx_len
        self.seq_ids = seq_ids
        # On the host: the tokens every live request brings; whether the step reports bounds instead of
        # counts (a padded step does); and, for such a step, {limit: the most tokens that requests of fewer
        # than ``limit`` tokens bring together}.
        self.tokens_each = (np.ones(num_seqs, np.int64) if tokens_each is None
                            else np.asarray(tokens_each, dtype=np.int64))
        self.padded = padded
        self.short_bounds = dict(short_bounds or {})

        def view(name, *shape):
            begin, count = layout[name]
            return packed[begin:begin + count].view(*shape)

        self.token_ids = view("token_ids", num_tokens)
        # Rows whose id is a token that the step before left on the device: for each row the row of
        # ``fed_tokens`` it takes, or -1 for its own ``token_ids``.  Both None where no step feeds another.
        self.token_src = view("token_src", num_tokens) if "token_src" in layout else None
        self.fed_tokens = None
        self.positions = view("positions", num_tokens)
        self.seq_of = view("seq_of", num_tokens)
        self.q_start = view("q_start", num_seqs)
        self.q_len = view("q_len", num_seqs)
        self.ctx_len = view("ctx_len", num_seqs)
        self.state_slots = view("state_slots", num_seqs)
        self.logit_rows = view("logit_rows", num_logit_rows)
        self.block_tables = [view(f"block_table_{g}", num_seqs, mb) for g, mb in enumerate(max_blocks)]

    def tokens_of_short_requests(self, limit: int) -> int:
        """How many tokens the requests that bring fewer than ``limit`` tokens bring together: what a
        mixer that runs such requests through a kernel of their own sizes that launch by.  A padded step
        gives a bound (the one it was laid out with for this limit, else all its rows), or 0 when there
        is no such request."""
        short = int(self.tokens_each[self.tokens_each < limit].sum())
        if not self.padded or short == 0:
            return short
        return min(self.num_tokens, self.short_bounds.get(limit, self.num_tokens))


def context_bound(longest: int) -> int:
    """What a step reports as its longest context: the power of two (1024 at least), or one and a half
    times a power of two, that holds it.  The kernels size their launches and choose how to split the keys
    by it, so steps of one shape whose contexts share a bound run the same launches, captured in a graph or
    not.  (Powers of two alone overstate a context by up to a factor of two, and the keys were then dealt
    to more workgroups than paid.)"""
    bound = 1024
    while bound < longest:
        if bound + bound // 2 >= longest:
            return bound + bound // 2
        bound *= 2
    return bound


class CannotFeed(Exception):
    """A step that was to take tokens from the step before on the device cannot: nothing was launched, and
    the caller reads those tokens and runs the step with them instead."""


class CaptureOutgrown(Exception):
    """A step no longer fits the fixed sizes it was to be laid out with."""


class TableTooWide(CaptureOutgrown):
    """A request has more pages than the rows of a fixed-width block table have room for."""

    def __init__(self, group: int, pages: int):
        super().__init__(f"group {group}: a table of {pages} pages")
        self.group, self.pages = group, pages


class ContextTooLong(CaptureOutgrown):
    """A request's context is longer than the bound the step was to report."""


class ShortTokensOutgrown(CaptureOutgrown):
    """The requests of few tokens bring more tokens together than the bound the step was to report."""


def token_bucket(tokens: int) -> int:
    """The number of rows a step of so many tokens is padded to: steps of many lengths then have few
    shapes, and a shape that comes again replays from a graph."""
    for small in (16, 32, 64):
        if tokens <= small:
            return small
    step = 64 if tokens <= 1024 else 256
    return (tokens + step - 1) // step * step


def build_batch(entries, manager, num_groups: int, vocab_size: int, max_positions: int, device,
                check_start: bool = True, widths: list | None = None, ctx_bound: int | None = None,
                pad_to: int | None = None, short_bounds: dict | None = None) -> StepBatch:
    """Validate the entries against the cache manager and lay the step out for the device.

    ``widths`` fixes the pages a row of each group's block table has (TableTooWide if a request
    has more) and ``ctx_bound`` what the batch reports as its longest context (ContextTooLong): a step laid out
    so has the same layout, and gives the kernels the same launch sizes, as any other step with
    the same tokens a request, whatever the requests' positions.

    ``pad_to`` adds one more request after the others that holds the rows up to that many: padding
    (token 0, position -1, no pages, no context, state slot -1; it has no rows when none are
    missing).  The batch then reports bounds instead of counts (every row might belong to one
    request, or to short ones), so that steps with the same rows, requests and wanted places give
    the kernels the same launch sizes.  ``short_bounds`` maps a limit to how many tokens the requests
    with fewer than ``limit`` tokens bring together at most (ShortTokensOutgrown if they bring more);
    for a limit it does not name every row might be one of theirs.

    Refused with ConfigError: an empty step, an entry without tokens, a token id
    outside the vocabulary, a position with no page or past the longest position
    the model knows, a wanted place outside the entry, a request that appears
    twice, and (with ``check_start``) an entry that does not start where the
    cache says the request has got to."""
    entries = list(entries)
    if not entries:
        raise ConfigError("an empty batch")
    seen = set()
    live = sum(len(e.tokens) for e in entries)
    if pad_to is not None and pad_to < live:
        raise ConfigError(f"{live} tokens in a step padded to {pad_to}")
    n = live if pad_to is None else pad_to
    S = len(entries) + (0 if pad_to is None else 1)
    token_ids = np.zeros(n, np.int32)
    positions = np.full(n, -1, np.int32)
    seq_of = np.full(n, S - 1, np.int32)
    q_start = np.empty(S, np.int32)
    q_len = np.empty(S, np.int32)
    ctx_len = np.empty(S, np.int32)
    state_slots = np.empty(S, np.int32)
    logit_rows: list = []
    tables = [[] for _ in range(num_groups)]
    at = 0
    for s, e in enumerate(entries):
        count = len(e.tokens)
        if count == 0:
            raise ConfigError(f"request {e.seq_id} brings no tokens to the step")
        if e.seq_id in seen:
            raise ConfigError(f"request {e.seq_id} appears twice in one step")
        seen.add(e.seq_id)
        toks = np.asarray(e.tokens, dtype=np.int64)
        if toks.min() < 0 or toks.max() >= vocab_size:
            raise ConfigError(f"request {e.seq_id}: token id outside the vocabulary of {vocab_size}")
        written = manager.tokens(e.seq_id)
        if check_start and e.start != written:
            raise ConfigError(f"request {e.seq_id}: tokens start at position {e.start}, the cache holds {written}")
        if e.start + count > manager.capacity(e.seq_id):
            raise ConfigError(f"request {e.seq_id} has no block for position {e.start + count - 1}")
        if max_positions and e.start + count > max_positions:
            raise ConfigError(f"request {e.seq_id}: position {e.start + count - 1} is past the model's {max_positions}")
        for w in e.want:
            if not 0 <= w < count:
                raise ConfigError(f"request {e.seq_id}: logits wanted at place {w} of {count} tokens")
            logit_rows.append(at + w)
        token_ids[at:at + count] = toks
        positions[at:at + count] = np.arange(e.start, e.start + count, dtype=np.int32)
        seq_of[at:at + count] = s
        q_start[s], q_len[s], ctx_len[s], state_slots[s] = at, count, e.start + count, e.state_slot
        for g in range(num_groups):
            tables[g].append(manager.table(e.seq_id, g))
        at += count
    if pad_to is not None:
        q_start[S - 1], q_len[S - 1], ctx_len[S - 1], state_slots[S - 1] = live, n - live, 0, -1
        for g in range(num_groups):
            tables[g].append([])

    max_blocks = [max(1, max(len(t) for t in tables[g])) for g in range(num_groups)]
    if widths is not None:
        for g in range(num_groups):
            if max_blocks[g] > widths[g]:
                raise TableTooWide(g, max_blocks[g])
        max_blocks = list(widths)
    pieces = [("token_ids", token_ids), ("positions", positions), ("seq_of", seq_of), ("q_start", q_start),
              ("q_len", q_len), ("ctx_len", ctx_len), ("state_slots", state_slots),
              ("logit_rows", np.asarray(logit_rows, dtype=np.int32))]
    for g in range(num_groups):
        bt = np.full((S, max_blocks[g]), -1, np.int32)
        for s, t in enumerate(tables[g]):
            bt[s, :len(t)] = t
        pieces.append((f"block_table_{g}", bt.reshape(-1)))
    layout = {}
    offset = 0
    for name, arr in pieces:
        layout[name] = (offset, arr.size)
        offset += (arr.size + 3) // 4 * 4      # keep every piece 16-byte aligned
    host = np.zeros(max(offset, 4), np.int32)
    for name, arr in pieces:
        begin, count = layout[name]
        host[begin:begin + count] = arr
    packed = torch.from_numpy(host).to(device)
    longest = int(ctx_len.max())
    if ctx_bound is None:
        ctx_bound = context_bound(longest)
    if longest > ctx_bound:
        raise ContextTooLong(f"a context of {longest} tokens in a step laid out for {ctx_bound}")
    longest = ctx_bound
    each = q_len[:len(entries)]
    if pad_to is not None:
        # every row might belong to one request
        for limit, bound in (short_bounds or {}).items():
            short = int(each[each < limit].sum())
            if short > bound:
                raise ShortTokensOutgrown(f"{short} tokens of requests that bring fewer than {limit} "
                                          f"in a step laid out for {bound}")
        batch = StepBatch(packed, layout, n, S, max_blocks, len(logit_rows), n, longest,
                          [e.seq_id for e in entries], tokens_each=each, padded=True, short_bounds=short_bounds)
        batch.live_seqs = S - 1
        return batch
    return StepBatch(packed, layout, n, S, max_blocks, len(logit_rows), int(q_len.max()), longest,
                     [e.seq_id for e in entries], tokens_each=each)
