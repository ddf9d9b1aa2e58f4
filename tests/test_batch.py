"""The descriptor of a step on the host: layout, bounds, padding and refusals (no GPU)."""

import numpy as np
import pytest

from paged_llm_rs_amd.cache import CacheManager, GroupGeometry
from paged_llm_rs_amd.engine.batch import (ContextTooLong, ShortTokensOutgrown, StepEntry, TableTooWide, build_batch, context_bound,
                                            token_bucket)
from paged_llm_rs_amd.errors import ConfigError


def manager(blocks=64, block_size=4):
    return CacheManager([GroupGeometry(block_size, blocks, 0)])


def requests(m, lengths, written=None):
    entries = []
    for i, n in enumerate(lengths):
        m.add_sequence(i + 1)
        have = (written or [0] * len(lengths))[i]
        if have:
            assert m.reserve(i + 1, have)
            m.advance(i + 1, have)
        assert m.reserve(i + 1, n)
        entries.append(StepEntry(i + 1, list(range(10, 10 + n)), have, [n - 1]))
    return entries


def piece(batch, name):
    begin, count = batch.layout[name]
    return batch.packed[begin:begin + count].numpy()


def test_buckets():
    assert [token_bucket(n) for n in (1, 16, 17, 33, 64, 65, 128, 1000, 1024, 1025, 2048, 2049)] == \
        [16, 16, 32, 64, 64, 128, 128, 1024, 1024, 1280, 2048, 2304]
    assert [context_bound(n) for n in (1, 1024, 1025, 1537, 5000, 6145)] == [1024, 1024, 1536, 2048, 6144, 8192]


def test_a_step_without_padding_reports_what_it_holds():
    m = manager()
    batch = build_batch(requests(m, [5, 1, 20], written=[0, 9, 3]), m, 1, 100, 0, "cpu")
    assert (batch.num_tokens, batch.num_seqs, batch.live_seqs, batch.num_logit_rows) == (26, 3, 3, 3)
    assert batch.max_q_len == 20 and batch.max_ctx_len == 1024 and batch.tokens_of_short_requests(16) == 6
    assert piece(batch, "positions").tolist() == list(range(5)) + [9] + list(range(3, 23))
    assert piece(batch, "q_start").tolist() == [0, 5, 6] and piece(batch, "ctx_len").tolist() == [5, 10, 23]
    assert piece(batch, "logit_rows").tolist() == [4, 5, 25]


def test_padding_adds_a_request_that_holds_nothing_and_bounds_instead_of_counts():
    m = manager()
    entries = requests(m, [5, 20], written=[0, 3])
    batch = build_batch(entries, m, 1, 100, 0, "cpu", pad_to=32)
    assert (batch.num_tokens, batch.num_seqs, batch.live_seqs) == (32, 3, 2)
    assert batch.max_q_len == 32 and batch.tokens_of_short_requests(16) == 32          # a short request is there: every row might be short
    assert piece(batch, "positions")[25:].tolist() == [-1] * 7 and piece(batch, "seq_of")[25:].tolist() == [2] * 7
    assert piece(batch, "q_start").tolist() == [0, 5, 25] and piece(batch, "q_len").tolist() == [5, 20, 7]
    assert piece(batch, "ctx_len").tolist() == [5, 23, 0] and piece(batch, "state_slots")[2] == -1
    table = piece(batch, "block_table_0").reshape(3, -1)
    assert (table[2] == -1).all() and table[1, 0] >= 0
    # told how many tokens the short requests bring at most, the batch reports that bound; more of them are refused
    bounded = build_batch(entries, m, 1, 100, 0, "cpu", pad_to=32, short_bounds={16: 16})
    assert bounded.tokens_of_short_requests(16) == 16 and bounded.max_q_len == 32
    with pytest.raises(ShortTokensOutgrown):
        build_batch(entries, m, 1, 100, 0, "cpu", pad_to=32, short_bounds={16: 4})
    # the same step without short requests reports no short rows; a full bucket has a request of no rows
    m2 = manager()
    full = build_batch(requests(m2, [16, 16]), m2, 1, 100, 0, "cpu", pad_to=32)
    assert full.tokens_of_short_requests(16) == 0 and piece(full, "q_len").tolist() == [16, 16, 0]
    with pytest.raises(ConfigError):
        build_batch(requests(manager(), [40]), manager(), 1, 100, 0, "cpu", pad_to=32)


def test_fixed_widths_and_bounds_are_kept_or_refused():
    m = manager(block_size=4)
    entries = requests(m, [30])
    batch = build_batch(entries, m, 1, 100, 0, "cpu", widths=[16], ctx_bound=64)
    assert piece(batch, "block_table_0").size == 16 and batch.max_ctx_len == 64
    with pytest.raises(TableTooWide):
        build_batch(entries, m, 1, 100, 0, "cpu", widths=[4])
    with pytest.raises(ContextTooLong):
        build_batch(entries, m, 1, 100, 0, "cpu", ctx_bound=16)


def test_steps_of_one_shape_have_one_layout():
    a, b = manager(), manager()
    one = build_batch(requests(a, [40, 1], written=[0, 7]), a, 1, 100, 0, "cpu", widths=[32], ctx_bound=1024, pad_to=64)
    two = build_batch(requests(b, [13, 30], written=[50, 0]), b, 1, 100, 0, "cpu", widths=[32], ctx_bound=1024, pad_to=64)
    assert one.layout == two.layout and one.packed.numel() == two.packed.numel()
    assert (one.max_q_len, one.tokens_of_short_requests(16), one.num_seqs) == (two.max_q_len, two.tokens_of_short_requests(16), two.num_seqs)
