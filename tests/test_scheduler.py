"""The scheduler's decisions without a model: every step is answered with a constant
token.  The scenarios are the reference's own (scheduler.rs:832-1369)."""

from __future__ import annotations

import random

import pytest

from paged_llm_rs_amd.cache import CacheManager, GroupGeometry
from paged_llm_rs_amd.engine import scheduler as sched
from paged_llm_rs_amd.errors import ConfigError


def scheduler(blocks, block_size, max_batch, chunk=128, window=0, state_slots=0, max_positions=0):
    manager = CacheManager([GroupGeometry(block_size, blocks, window)], state_slots)
    return sched.Scheduler(manager, max_batch=max_batch, chunk=chunk, max_positions=max_positions)


def submit(s, seq_id, prompt_len, max_tokens, prompt=None):
    s.submit(seq_id, prompt if prompt is not None else [1] * prompt_len, 0.0, None, None, max_tokens, [99], seq_id)


def step(s, token=7):
    plan = s.plan()
    outcome = s.commit([token] * len(plan.ids))
    return plan, outcome


def test_a_prompt_is_admitted_before_anything_decodes():
    """scheduler.rs:832-845"""
    s = scheduler(64, 4, 4, chunk=None)
    submit(s, 1, 3, 10)
    submit(s, 2, 5, 10)
    assert step(s)[0].kind == sched.PREFILL
    assert step(s)[0].kind == sched.PREFILL
    assert step(s)[0].kind == sched.DECODE
    assert s.running == 2


def test_a_sequence_takes_only_the_blocks_its_tokens_need():
    """scheduler.rs:847-856"""
    s = scheduler(64, 16, 4)
    submit(s, 1, 20, 100)
    step(s)
    assert s.manager.in_use() == 2 and s.manager.available() == 62


def test_a_block_is_taken_only_when_the_last_one_fills():
    """scheduler.rs:858-871"""
    s = scheduler(64, 4, 4)
    submit(s, 1, 3, 20)
    step(s)
    assert s.manager.in_use() == 1
    step(s)
    assert s.manager.in_use() == 1
    step(s)
    assert s.manager.in_use() == 2


def test_late_arrivals_join_the_running_batch():
    """scheduler.rs:873-893"""
    s = scheduler(64, 8, 4, chunk=None)
    submit(s, 1, 3, 20)
    for _ in range(4):
        step(s)
    submit(s, 2, 3, 20)
    assert step(s)[0].kind == sched.PREFILL
    plan, _ = step(s)
    assert plan.kind == sched.DECODE and plan.ids == [1, 2]
    assert len(plan.entries) == 2
    assert plan.entries[0].start != plan.entries[1].start


def test_a_stop_token_ends_a_sequence_and_gives_its_blocks_back():
    """scheduler.rs:895-906"""
    s = scheduler(64, 4, 4)
    submit(s, 1, 6, 10)
    step(s)
    assert s.manager.in_use() == 2
    _, outcome = step(s, 99)
    assert outcome.tokens == [], "the stop token is not output"
    assert [(f.id, f.finish) for f in outcome.finished] == [(1, "stop")]
    assert s.manager.available() == 64


def test_the_pool_running_dry_evicts_the_newest_and_recomputes_it():
    """scheduler.rs:908-932"""
    s = scheduler(4, 4, 50, chunk=None)
    submit(s, 1, 4, 50)
    submit(s, 2, 4, 50)
    step(s)
    step(s)
    assert s.manager.available() == 2
    for _ in range(10):
        step(s)
    m = s.metrics()
    assert m["preemptions"] > 0 and m["recomputed_tokens"] > 0
    assert s.waiting + s.running == 2, "what was evicted went back to the queue"


def test_the_sequence_that_arrived_first_is_never_the_one_evicted():
    """scheduler.rs:934-954"""
    s = scheduler(4, 4, 50)
    submit(s, 1, 4, 50)
    submit(s, 2, 4, 50)
    step(s)
    step(s)
    for _ in range(12):
        step(s)
        assert 1 in s.running_ids() or s.waiting > 0
    assert s.metrics()["preemptions"] > 0


def test_a_prompt_longer_than_the_whole_pool_is_refused():
    """scheduler.rs:956-966"""
    s = scheduler(2, 4, 4)
    submit(s, 1, 20, 10)
    plan = s.plan()
    assert plan.kind == sched.REFUSED and plan.refused == 1
    outcome = s.commit([])
    assert [(f.id, f.finish) for f in outcome.finished] == [(1, "length")]
    assert s.waiting == 0 and s.manager.available() == 2


def test_cancelling_gives_the_blocks_back_at_once():
    """scheduler.rs:968-977"""
    s = scheduler(8, 4, 4)
    submit(s, 1, 8, 100)
    step(s)
    assert s.manager.in_use() == 2
    s.cancel(1)
    assert s.manager.available() == 8 and s.running == 0
    submit(s, 2, 8, 100)
    s.cancel(2)
    assert s.waiting == 0


def test_an_idle_scheduler_plans_nothing():
    """scheduler.rs:979-983"""
    assert scheduler(8, 4, 4).plan().kind == sched.IDLE


def test_a_second_request_with_the_same_prompt_reuses_the_blocks_of_the_first():
    """scheduler.rs:985-1005"""
    s = scheduler(64, 4, 4)
    submit(s, 1, 12, 4)
    for _ in range(5):
        step(s)
    assert s.running == 0
    first = s.metrics()
    assert first["cached_tokens"] == 0 and first["prefilled_tokens"] >= 12
    submit(s, 2, 12, 4)
    step(s)
    second = s.metrics()
    assert second["cached_tokens"] == 8
    assert second["prefilled_tokens"] - first["prefilled_tokens"] == 4


def test_sharing_stops_where_the_prompts_stop_agreeing():
    """scheduler.rs:1007-1032"""
    s = scheduler(64, 4, 4)
    common = list(range(12))
    submit(s, 1, 0, 2, prompt=common + [100, 101, 102, 103])
    for _ in range(4):
        step(s)
    before = s.metrics()["cached_tokens"]
    submit(s, 2, 0, 2, prompt=common + [200, 201, 202, 203])
    step(s)
    assert s.metrics()["cached_tokens"] - before == 12


def test_a_prefix_can_be_shared_while_its_first_owner_is_still_generating():
    """scheduler.rs:1034-1052"""
    s = scheduler(64, 4, 100)
    submit(s, 1, 12, 50)
    for _ in range(3):
        step(s)
    assert s.running == 1
    submit(s, 2, 12, 50)
    step(s)
    assert s.metrics()["cached_tokens"] == 8
    assert s.running == 2


def test_nothing_is_shared_when_the_cache_is_off():
    """scheduler.rs:1054-1068"""
    s = scheduler(64, 4, 4)
    s.set_prefix_cache(False)
    for seq_id in (1, 2):
        submit(s, seq_id, 12, 4)
        for _ in range(5):
            step(s)
    assert s.metrics()["cached_tokens"] == 0 and s.metrics()["prefix_hit_rate"] == 0.0


def test_cached_blocks_give_way_before_a_sequence_is_refused():
    """scheduler.rs:1070-1096"""
    s = scheduler(5, 4, 4)
    for seq_id in (1, 2, 3):
        submit(s, seq_id, 0, 2, prompt=[t + seq_id * 1000 for t in range(12)])
        for _ in range(4):
            step(s)
    assert s.waiting == 0 and s.running == 0
    assert s.manager.counter("evictions") > 0


def test_what_paging_wastes_is_bounded_by_one_block_a_sequence():
    """scheduler.rs:1098-1113"""
    s = scheduler(64, 16, 8)
    for seq_id in range(1, 5):
        submit(s, seq_id, 20, 50)
    for _ in range(4):
        step(s)
    assert s.running == 4
    assert s.wasted_tokens() < 4 * 16


def test_the_average_batch_counts_only_decode_passes():
    """scheduler.rs:1115-1130"""
    s = scheduler(64, 8, 4, chunk=None)
    submit(s, 1, 2, 10)
    submit(s, 2, 2, 10)
    for _ in range(5):
        step(s)
    m = s.metrics()
    assert m["prefills"] == 2 and m["steps"] == 5
    assert abs(m["mean_batch"] - 2.0) < 1e-9


def test_a_long_prompt_is_fed_a_slice_at_a_time_within_the_budget():
    """scheduler.rs:1132-1163"""
    s = scheduler(64, 8, 8, chunk=16)
    submit(s, 1, 100, 4)
    slices = fed = 0
    while True:
        plan, outcome = step(s)
        if plan.kind == sched.DECODE:
            break
        assert plan.kind == sched.MIXED
        assert plan.num_tokens <= 16
        slices += 1
        fed += plan.num_tokens
        assert slices < 20
        if not outcome.tokens:
            assert fed < 100, "the prompt ran out without producing a token"
    assert slices >= 6 and fed == 100


def test_a_prompt_arriving_mid_flight_does_not_stop_the_sequences_already_decoding():
    """scheduler.rs:1165-1194"""
    s = scheduler(64, 8, 8, chunk=16)
    submit(s, 1, 4, 40)
    submit(s, 2, 4, 40)
    for _ in range(6):
        step(s)
    assert s.running == 2
    submit(s, 3, 90, 40)
    for _ in range(5):
        plan, outcome = step(s)
        assert plan.kind == sched.MIXED
        produced = [i for i, _ in outcome.tokens]
        assert 1 in produced and 2 in produced and 3 not in produced


def test_a_prompts_last_slice_is_the_one_that_produces_its_first_token():
    """scheduler.rs:1196-1210"""
    s = scheduler(64, 8, 8, chunk=16)
    submit(s, 1, 40, 4)
    answered = [bool(step(s)[1].tokens) for _ in range(4)]
    assert answered == [False, False, True, True]


def test_the_budget_covers_the_decodes_and_the_slice_together():
    """scheduler.rs:1212-1237"""
    s = scheduler(64, 8, 8, chunk=8)
    for seq_id in (1, 2, 3):
        submit(s, seq_id, 2, 40)
    for _ in range(6):
        step(s)
    assert s.running == 3
    submit(s, 9, 60, 40)
    plan, _ = step(s)
    assert plan.kind == sched.MIXED and plan.num_tokens == 8
    assert dict(plan.advanced)[9] == 5
    # decodes come first, then the slice
    assert [len(e.tokens) for e in plan.entries] == [1, 1, 1, 5]


def test_chunking_off_gives_a_prompt_its_own_pass_and_on_does_not():
    """scheduler.rs:1239-1256"""
    for chunk, alone in ((None, True), (16, False)):
        s = scheduler(64, 8, 8, chunk=chunk)
        submit(s, 1, 4, 40)
        for _ in range(3):
            step(s)
        submit(s, 2, 20, 40)
        _, outcome = step(s)
        assert any(i == 1 for i, _ in outcome.tokens) == (not alone)


def test_a_dry_pool_evicts_under_chunking_too():
    """scheduler.rs:1258-1280"""
    s = scheduler(6, 4, 50, chunk=8)
    for seq_id in (1, 2, 3):
        submit(s, seq_id, 4, 50)
    for _ in range(20):
        step(s)
    m = s.metrics()
    assert m["preemptions"] > 0 and m["tokens"] > 20
    assert s.running + s.waiting == 3


def test_a_slices_tokens_carry_the_positions_they_hold_in_the_prompt():
    """scheduler.rs:1282-1330"""
    s = scheduler(64, 8, 8, chunk=16)
    submit(s, 1, 4, 40)
    for _ in range(3):
        step(s)
    assert s.running == 1
    submit(s, 2, 0, 4, prompt=list(range(100, 140)))
    expected = 0
    for _ in range(3):
        plan = s.plan()
        assert plan.kind == sched.MIXED
        entry = [e for e in plan.entries if e.seq_id == 2][0]
        assert plan.entries[-1] is entry, "the resident's rows come first"
        assert entry.start == expected
        assert entry.tokens == list(range(100 + expected, 100 + expected + len(entry.tokens)))
        assert dict(plan.advanced)[2] == len(entry.tokens)
        expected += len(entry.tokens)
        assert entry.want == ([len(entry.tokens) - 1] if expected == 40 else [])
        s.commit([7] * len(plan.ids))
    assert expected == 40


def test_a_prompt_that_is_admitted_gets_a_slice_in_the_pass_that_admitted_it():
    """scheduler.rs:1332-1369"""
    s = scheduler(9, 4, 8, chunk=64)
    for seq_id in range(1, 5):
        submit(s, seq_id, 4, 30)
    before = s.metrics()["prefills"]
    for _ in range(60):
        plan = s.plan()
        after = s.metrics()["prefills"]
        if after > before:
            assert plan.kind in (sched.MIXED, sched.PREFILL)
            assert plan.advanced, "a sequence was admitted and the pass ran nothing for it"
        before = after
        s.commit([7] * len(plan.ids))
    assert s.metrics()["prefills"] >= 4


# --- beyond the reference's scenarios ---------------------------------------------------------------

def test_short_prompts_share_a_step_while_the_budget_lasts():
    """Not in the reference, whose step carries a slice of one prompt: here the tokens that the first prompt
    leaves of the budget go to the next waiting ones, and at most one prompt is left part-way."""
    s = scheduler(256, 4, 8, chunk=32)
    for i, n in enumerate([10, 10, 10, 10, 50], start=1):
        submit(s, i, n, 4, prompt=[i] * n)        # nothing in common: no pages are shared
    plan, _ = step(s)
    # 32 tokens: three prompts whole and two tokens of the fourth
    assert [(e.seq_id, len(e.tokens), e.want) for e in plan.entries] == [(1, 10, [9]), (2, 10, [9]), (3, 10, [9]), (4, 2, [])]
    assert plan.ids == [1, 2, 3] and plan.kind == sched.MIXED
    plan, _ = step(s)
    # three decodes first, then the prompt in flight, then the next one with what is left: 3 + 8 + 21
    assert [(e.seq_id, len(e.tokens), e.start) for e in plan.entries] == [(1, 1, 10), (2, 1, 10), (3, 1, 10), (4, 8, 2), (5, 21, 0)]
    assert plan.ids == [1, 2, 3, 4]
    plan, _ = step(s)
    assert [(e.seq_id, len(e.tokens), e.start) for e in plan.entries] == [(1, 1, 11), (2, 1, 11), (3, 1, 11), (4, 1, 10), (5, 28, 21)]
    # the rows of a step are bounded by max_batch (a step always has room for one prompt)
    t = scheduler(256, 4, 3, chunk=32)
    for i in range(1, 7):
        submit(t, i, 2, 4, prompt=[i, i])
    assert [e.seq_id for e in step(t)[0].entries] == [1, 2, 3]
    assert [e.seq_id for e in step(t)[0].entries] == [1, 2, 3, 4]
    while t.running or t.waiting:
        step(t)
    assert t.manager.available() == t.manager.total()


def test_bad_requests_are_refused_at_submission():
    """session/sampler refusals: scheduler.rs:68-70, sampler.rs:72-95"""
    s = scheduler(8, 4, 4)
    with pytest.raises(ConfigError):
        s.submit(1, [], 0.0, None, None, 4, [], 0)
    with pytest.raises(ConfigError):
        s.submit(1, [1], -0.5, None, None, 4, [], 0)
    with pytest.raises(ConfigError):
        s.submit(1, [1], 1.0, 0, None, 4, [], 0)
    with pytest.raises(ConfigError):
        s.submit(1, [1], 1.0, None, 1.5, 4, [], 0)
    with pytest.raises(ConfigError):
        sched.Scheduler(CacheManager([GroupGeometry(4, 4)]), chunk=0)


def test_a_request_stops_at_the_models_longest_position():
    s = scheduler(64, 4, 4, max_positions=10)
    submit(s, 1, 8, 100)
    produced = 0
    for _ in range(10):
        _, outcome = step(s)
        produced += len(outcome.tokens)
        if outcome.finished:
            assert outcome.finished[0].finish == "length"
            break
    # positions 0..9 exist: 8 prompt tokens, then tokens fed at 8 and 9, and the last one sampled is never fed
    assert produced == 3 and s.running == 0
    submit(s, 2, 11, 5)
    assert s.plan().kind == sched.REFUSED


def test_a_request_alone_that_outgrows_the_pool_ends_instead_of_idling_forever():
    s = scheduler(2, 4, 4)
    submit(s, 1, 6, 100)
    finished = None
    for _ in range(8):
        plan = s.plan()
        if plan.kind == sched.IDLE:
            finished = s.drain_finished().finished
            break
        s.commit([7] * len(plan.ids))
    assert finished and finished[0].finish == "length" and finished[0].generated == 3
    assert s.manager.available() == 2


def test_state_slots_limit_admission_and_are_marked_fresh_once():
    s = scheduler(64, 4, 8, chunk=16, state_slots=2)
    for seq_id in (1, 2, 3):
        submit(s, seq_id, 20, 3)
    plan = s.plan()
    assert plan.entries[0].state_slot == 0 and plan.entries[0].fresh_state
    s.commit([7] * len(plan.ids))
    plan = s.plan()
    assert not plan.entries[0].fresh_state, "a slot is cleared once, before its first use"
    s.commit([7] * len(plan.ids))
    seen = set()
    for _ in range(40):
        plan = s.plan()
        if plan.kind == sched.IDLE:
            break
        assert s.running <= 2
        for e in plan.entries:
            seen.add(e.seq_id)
            assert e.state_slot in (0, 1)
        s.commit([7] * len(plan.ids))
    assert seen == {1, 2, 3}
    assert s.manager.free_state_slots == 2


def test_a_windowed_group_serves_a_prompt_longer_than_its_pool():
    s = scheduler(8, 4, 4, chunk=8, window=8)
    submit(s, 1, 100, 5)
    produced = 0
    for _ in range(40):
        plan = s.plan()
        if plan.kind == sched.IDLE:
            break
        assert plan.kind != sched.REFUSED
        produced += len(s.commit([7] * len(plan.ids)).tokens)
        assert s.manager.in_use() <= 5
    assert produced == 5


@pytest.mark.parametrize("seed", range(5))
def test_every_request_finishes_and_every_page_returns_under_random_load(seed):
    rng = random.Random(seed)
    bs = rng.choice([2, 4, 16])
    blocks = rng.randrange(8, 30)
    chunk = rng.choice([None, 8, 32])
    s = scheduler(blocks, bs, rng.randrange(1, 6), chunk=chunk)
    submitted = {}
    finished = {}
    next_id = 1
    for it in range(3000):
        if next_id <= 25 and rng.random() < 0.15:
            n = rng.randrange(1, bs * blocks // 2)
            submit(s, next_id, 0, rng.randrange(1, 12), prompt=[rng.randrange(5) for _ in range(n)])
            submitted[next_id] = n
            next_id += 1
        plan = s.plan()
        if plan.kind == sched.IDLE:
            for f in s.drain_finished().finished:
                finished[f.id] = f
            if next_id > 25 and not s.running and not s.waiting:
                break
            continue
        if chunk:
            assert plan.num_tokens <= chunk
        starts = {e.seq_id: e.start for e in plan.entries}
        for e in plan.entries:
            assert e.start == s.manager.tokens(e.seq_id), "a portion starts where the cache has got to"
            assert e.start + len(e.tokens) <= s.manager.capacity(e.seq_id)
        token = 99 if rng.random() < 0.05 else 7
        for f in s.commit([token] * len(plan.ids)).finished:
            finished[f.id] = f
        assert s.manager.in_use() + s.manager.available() == blocks
    assert set(finished) == set(submitted), "a request was lost"
    assert s.manager.available() == blocks and s.manager.live_sequences == 0
    assert all(f.finish in ("stop", "length") for f in finished.values())


# ---------------------------------------------------------------------------
# Decoding a step ahead: the step behind a decoding step is planned, and would be
# launched, before that step's tokens are known.  (No counterpart in the reference,
# whose engine reads every step's tokens before it plans the next.)
# ---------------------------------------------------------------------------

def drive(s, arrivals, token_of, ahead: bool, steps: int = 4000, log=None):
    """Run the scheduler to the end.  ``arrivals``: {iteration: [(id, prompt, max_tokens)]};
    ``token_of(id, n)`` is the n-th token request id samples.  With ``ahead`` every step that can be is
    planned before the tokens of the one before are committed, the way the engine does it.  Returns
    ({id: tokens}, {id: finish}, (steps planned ahead, steps of single tokens))."""
    out, finish, count, planned_ahead, decoding = {}, {}, {}, 0, 0
    flight = None
    for it in range(steps):
        for seq_id, prompt, most in arrivals.get(it, []):
            s.submit(seq_id, prompt, 0.0, None, None, most, [99], seq_id)
            out[seq_id], count[seq_id] = [], 0
        if flight is not None:
            plan, flight = flight, None
        else:
            plan = s.plan()
            if plan.kind == sched.IDLE:
                for f in s.drain_finished().finished:
                    finish[f.id] = f.finish
                if it > max(arrivals) and not s.running and not s.waiting:
                    break
                continue
        decoding += plan.kind == sched.DECODE
        if log is not None:
            log.append((plan.kind, tuple(plan.ids), tuple((e.seq_id, e.start, len(e.tokens)) for e in plan.entries)))
        if ahead and plan.kind == sched.DECODE:
            s.launched()
            before = {i: s.manager.tokens(i) for i in s.running_ids()}
            flight = s.plan_ahead()
            if flight is not None:
                planned_ahead += 1
                for e in flight.entries:
                    if e.fed_row >= 0:
                        assert plan.ids[e.fed_row] == e.seq_id, "a row is fed the token of its own request"
                    else:
                        assert e.seq_id not in plan.ids and e.tokens == out[e.seq_id][-1:], \
                            "a request without a row in the step before brings its last token itself"
                    assert e.start == before[e.seq_id] == s.manager.tokens(e.seq_id)
                    assert e.start + 1 <= s.manager.capacity(e.seq_id)
        sampled = []
        for i in plan.ids:
            sampled.append(token_of(i, count.get(i, 0)))
            count[i] = count.get(i, 0) + 1
        outcome = s.commit(sampled)
        for i, token in outcome.tokens:
            out[i].append(token)
        for f in outcome.finished:
            finish[f.id] = f.finish
    else:
        raise AssertionError("the scheduler did not come to an end")
    return out, finish, (planned_ahead, decoding)


def test_a_step_planned_ahead_has_a_row_for_everyone_the_step_before_cannot_end():
    s = scheduler(64, 4, 4)
    submit(s, 1, 3, 2)         # its second token is its last
    submit(s, 2, 5, 10)
    submit(s, 3, 2, 10)
    assert step(s)[0].kind == sched.MIXED and not s.waiting     # the prompts: everyone has one token out
    plan = s.plan()
    assert plan.kind == sched.DECODE and plan.ids == [1, 2, 3]
    assert s.plan_ahead() is None, "not before the step is on the device"
    s.launched()
    following = s.plan_ahead()
    assert [e.seq_id for e in following.entries] == [2, 3] and [e.fed_row for e in following.entries] == [1, 2]
    assert all(e.want == [0] and len(e.tokens) == 1 for e in following.entries)
    assert [e.start for e in following.entries] == [s.manager.tokens(2), s.manager.tokens(3)]
    with pytest.raises(Exception, match="planned ahead"):
        s.plan()
    outcome = s.commit([7, 7, 7])
    assert [f.id for f in outcome.finished] == [1]
    with pytest.raises(Exception, match="planned ahead"):
        s.plan()               # the step planned ahead is the planned step now
    outcome = s.commit([8, 8])
    assert outcome.tokens == [(2, 8), (3, 8)]
    assert s.plan().ids == [2, 3]


def test_a_stop_token_ends_a_request_whose_row_ahead_then_counts_for_nothing():
    s = scheduler(64, 4, 4)
    submit(s, 1, 3, 10)
    submit(s, 2, 3, 10)
    assert step(s)[0].kind == sched.MIXED and not s.waiting
    plan = s.plan()
    s.launched()
    following = s.plan_ahead()
    assert [e.seq_id for e in following.entries] == [1, 2]
    in_use = s.manager.in_use()
    outcome = s.commit([99, 7])                      # request 1 stops
    assert [(f.id, f.finish) for f in outcome.finished] == [(1, "stop")]
    assert s.manager.in_use() < in_use, "its pages are back although its row ahead is still running"
    outcome = s.commit([5, 6])                       # the step planned ahead: the token of request 1 is dropped
    assert outcome.tokens == [(2, 6)] and not outcome.finished
    assert s.plan().ids == [2]


def test_nothing_is_planned_ahead_while_a_request_waits_or_pages_are_short():
    s = scheduler(64, 4, 4)
    submit(s, 1, 3, 10)
    assert step(s)[0].kind == sched.MIXED and not s.waiting
    s.plan()
    s.launched()
    submit(s, 2, 3, 10)                              # arrives while the step runs
    assert s.plan_ahead() is None
    s.commit([7])
    assert s.plan().kind == sched.MIXED              # and is admitted by the ordinary planner

    s = scheduler(2, 4, 4)                           # two pages of four tokens
    submit(s, 1, 3, 100)
    step(s)                                          # the prompt: 3 tokens
    for _ in range(3):                               # tokens 4, 5, 6: the second page is taken
        assert step(s)[0].kind == sched.DECODE
    s.plan()                                         # token 7
    s.launched()
    assert s.plan_ahead() is not None                # token 8 still has a place
    s.commit([7])
    s.commit([7])
    s.plan()                                         # nothing left: alone and out of pages, the request ends
    s.launched()
    assert s.plan_ahead() is None
    s.commit([])
    assert s.manager.available() == 2


def test_a_step_ahead_that_cannot_stand_takes_no_page():
    """Two of three residents need a new page for the step ahead and one page is free: the step is the planner's
    (someone gives way), and the resident that could have had the page does not hold it a step early, where it
    would stand between the planner and the queue's front."""
    s = scheduler(7, 2, 4)                           # seven pages of two tokens
    submit(s, 1, 1, 100, prompt=[1])
    submit(s, 2, 2, 100, prompt=[2, 2])
    submit(s, 3, 2, 100, prompt=[3, 3])
    assert step(s)[0].kind == sched.MIXED            # the prompts: a page each
    assert step(s)[0].kind == sched.DECODE           # positions 1, 2, 2: requests 2 and 3 take their second page
    plan = s.plan()                                  # positions 2, 3, 3: request 1 takes its second page
    assert plan.kind == sched.DECODE and s.manager.available() == 1
    s.launched()
    assert s.plan_ahead() is None                    # positions 3, 4, 4 would take two pages
    assert s.manager.available() == 1
    s.commit([7, 7, 7])
    plan = s.plan()                                  # the planner's step: one of the two gives way
    assert plan.kind == sched.DECODE and len(plan.ids) == 2 and plan.ids[0] == 1 and s.metrics()["preemptions"] == 1


def test_steps_are_planned_ahead_while_the_queue_cannot_move():
    """Serving at its limit: more residents than rows, and a front of the queue that no page or slot can
    take yet.  The planner would decode, so the step is planned ahead; when the front can come in, it is not."""
    s = scheduler(64, 4, 2, chunk=16)                # two rows
    for seq_id in (1, 2, 3):
        submit(s, seq_id, 3, 10)
    step(s)
    assert step(s)[0].kind == sched.MIXED and s.running == 3 and not s.waiting   # the third prompt beside two rows
    plan = s.plan()
    assert plan.kind == sched.DECODE and plan.ids == [1, 2]
    s.launched()
    following = s.plan_ahead()
    assert [(e.seq_id, e.fed_row) for e in following.entries] == [(1, 0), (2, 1)], "the rows the planner would give"
    s.commit([7, 7])
    s.commit([7, 7])
    # request 1 has one token left: the step behind its last has a row for request 3, which brings its own token
    s = scheduler(64, 4, 2, chunk=16)
    submit(s, 1, 3, 3)
    submit(s, 2, 3, 10)
    submit(s, 3, 3, 10)
    step(s)
    step(s)
    assert s.plan().ids == [1, 2]
    s.launched()
    following = s.plan_ahead()
    assert [(e.seq_id, e.fed_row, e.tokens) for e in following.entries] == [(2, 1, [0]), (3, -1, [7])]
    assert following.entries[1].start == s.manager.tokens(3)
    outcome = s.commit([8, 8])
    assert [f.id for f in outcome.finished] == [1]
    assert s.commit([5, 6]).tokens == [(2, 5), (3, 6)]

    # a queue that waits for a state slot, and one that waits for pages
    s = scheduler(64, 4, 4, chunk=16, state_slots=1)
    submit(s, 1, 3, 10)
    submit(s, 2, 3, 10)
    step(s)
    assert s.running == 1 and s.waiting == 1
    assert s.plan().kind == sched.DECODE
    stalls = s.metrics()["admission_stalls"]
    s.launched()
    assert s.plan_ahead() is not None
    assert s.metrics()["admission_stalls"] == stalls + 1, "the stall is counted as the planner counts it"
    s.drop_ahead()
    assert s.metrics()["admission_stalls"] == stalls
    s.commit([7])

    s = scheduler(4, 4, 4, chunk=None)               # prompts run whole: the front needs all its pages at once
    submit(s, 1, 9, 10)                              # three of the four pages
    step(s)
    submit(s, 2, 0, 10, prompt=[2] * 6)              # two pages: waits
    assert s.plan().kind == sched.DECODE
    s.launched()
    following = s.plan_ahead()
    assert following is not None and following.ids == [1]
    s.commit([7])
    s.commit([7])
    s.cancel(1)
    assert s.plan().kind == sched.PREFILL            # and comes in by the planner once the pages are back

    s = scheduler(4, 4, 4, chunk=None)               # a front that can never be served is the planner's to turn away
    submit(s, 1, 9, 10)
    step(s)
    assert s.plan().kind == sched.DECODE
    s.launched()
    submit(s, 2, 1000, 1)
    assert s.plan_ahead() is None
    s.commit([7])
    assert s.plan().kind == sched.REFUSED


@pytest.mark.parametrize("seed", range(4))
def test_a_crowded_scheduler_plans_most_decoding_steps_ahead(seed):
    """Many more requests than rows and pages, all at once: the same tokens and endings as without planning
    ahead, and most decoding steps are planned ahead although the queue is never empty."""
    rng = random.Random(900 + seed)
    bs, blocks, max_batch = 4, 24, 3
    chunk = [None, 16][seed % 2]
    arrivals = {0: [(i, [rng.randrange(5) for _ in range(rng.randrange(2, 14))], rng.randrange(8, 30))
                    for i in range(1, 13)]}

    def token_of(seq_id, n):
        return 99 if (seq_id * 13 + n * 7) % 41 == 0 else (seq_id + n) % 50

    results = []
    for ahead in (False, True):
        s = scheduler(blocks, bs, max_batch, chunk=chunk)
        results.append(drive(s, arrivals, token_of, ahead))
        assert s.manager.available() == blocks and s.manager.live_sequences == 0
    (plain_out, plain_finish, _), (ahead_out, ahead_finish, (planned_ahead, decoding)) = results
    assert ahead_out == plain_out and ahead_finish == plain_finish
    # (the steps of single tokens that are not planned ahead: the first behind a prompt, and those behind which
    # the front of the queue comes in)
    assert planned_ahead > 0.6 * decoding, (planned_ahead, decoding)


def test_a_step_ahead_that_was_not_launched_is_forgotten():
    s = scheduler(64, 4, 4)
    submit(s, 1, 3, 10)
    assert step(s)[0].kind == sched.MIXED and not s.waiting
    steps = s.metrics()["steps"]
    s.plan()
    s.launched()
    assert s.plan_ahead() is not None
    s.drop_ahead()
    assert s.metrics()["steps"] == steps + 1
    s.commit([7])
    assert s.plan().ids == [1]                       # the ordinary planner goes on


def test_a_failed_step_is_abandoned_with_what_was_planned_ahead_of_it():
    s = scheduler(64, 4, 4)
    submit(s, 1, 3, 10)
    submit(s, 2, 3, 10)
    assert step(s)[0].kind == sched.MIXED and not s.waiting
    s.plan()
    s.launched()
    assert s.plan_ahead() is not None
    s.commit([7, 7])                                 # the step planned ahead is the planned step now ...
    s.abandon()                                      # ... and fails: whoever saw that cancels its requests
    s.cancel(1)
    assert s.plan().ids == [2]
    s.launched()
    assert s.plan_ahead() is not None
    s.abandon()                                      # a step and the one planned ahead of it
    s.cancel(2)
    assert s.plan().kind == sched.IDLE and s.manager.available() == 64


@pytest.mark.parametrize("seed", range(6))
def test_requests_get_the_same_tokens_with_and_without_steps_planned_ahead(seed):
    rng = random.Random(100 + seed)
    bs = rng.choice([2, 4, 16])
    blocks = rng.randrange(10, 40)
    chunk = rng.choice([None, 8, 32])
    max_batch = rng.randrange(1, 6)
    window = rng.choice([0, 0, 3 * bs])
    arrivals, next_id = {}, 1
    for it in range(0, 120):
        if next_id <= 20 and rng.random() < 0.25:
            n = rng.randrange(1, bs * blocks // 3)
            arrivals.setdefault(it, []).append((next_id, [rng.randrange(5) for _ in range(n)], rng.randrange(1, 25)))
            next_id += 1
    arrivals.setdefault(0, []).append((next_id, [1, 2, 3], 7))

    def token_of(seq_id, n):
        return 99 if (seq_id * 31 + n * 17) % 23 == 0 else (seq_id + n) % 50

    results = []
    for ahead in (False, True):
        s = scheduler(blocks, bs, max_batch, chunk=chunk, window=window)
        results.append(drive(s, arrivals, token_of, ahead))
        assert s.manager.available() == blocks and s.manager.live_sequences == 0
    (plain_out, plain_finish, (none, _)), (ahead_out, ahead_finish, (some, _)) = results
    assert none == 0 and some > 0
    assert ahead_out == plain_out and ahead_finish == plain_finish


@pytest.mark.parametrize("seed", list(range(10)) + [1051, 1052, 1102, 1148, 1173])
def test_without_stop_tokens_planning_ahead_changes_no_step(seed):
    """Where no stop token ends a request, nothing a step's tokens say changes the step behind it: with steps planned
    ahead the scheduler runs the very same steps, row for row, as without (a queue that stalls, requests that give
    way and come back, more residents than rows).  Where the step's own end changes what the planner would do (a
    request at its budget leaves, and the front of the queue may come in) nothing is planned ahead."""
    rng = random.Random(300 + seed)
    bs = rng.choice([2, 4, 16])
    blocks = rng.randrange(8, 30)
    chunk = rng.choice([None, 4, 8, 32])
    max_batch = rng.randrange(1, 6)
    window = rng.choice([0, 0, 3 * bs])
    # (all requests are there from the start: one that arrives while a step planned ahead is queued comes in a step
    # later than it would otherwise, which is the one difference that planning ahead makes by design)
    arrivals = {0: [(i, [rng.randrange(5) for _ in range(rng.randrange(1, bs * blocks // 3))], rng.randrange(1, 25))
                    for i in range(1, rng.randrange(3, 26))]}

    def token_of(seq_id, n):
        return (seq_id + n) % 50          # never the stop token (99)

    logs = []
    for ahead in (False, True):
        s = scheduler(blocks, bs, max_batch, chunk=chunk, window=window)
        # (no shared prefixes: a page that holds a token fed on the device gets its name a commit later, so a
        # newcomer may find a page less to share than it would otherwise)
        s.manager.set_prefix_cache(False)
        log = []
        drive(s, arrivals, token_of, ahead, log=log)
        logs.append(log)
    assert logs[0] == logs[1]


@pytest.mark.parametrize("seed", range(8))
def test_no_page_is_lost_when_steps_ahead_are_dropped_abandoned_and_cancelled_at_random(seed):
    """The engine's moves in a random order: plan, launch, plan ahead, and then commit, or drop what was planned
    ahead, or abandon the step as failed (cancelling its requests), with requests arriving and being cancelled in
    between.  Pages in use and free always add up, every request ends once, and at the end every page is free."""
    rng = random.Random(500 + seed)
    bs = rng.choice([2, 4, 16])
    blocks = rng.randrange(12, 40)
    chunk = rng.choice([None, 8, 32])
    s = scheduler(blocks, bs, rng.randrange(1, 6), chunk=chunk, window=rng.choice([0, 0, 2 * bs]))
    submitted, ended, cancelled = set(), {}, set()
    next_id, flight, idle = 1, None, 0
    for it in range(6000):
        if next_id <= 40 and rng.random() < 0.2:
            n = rng.randrange(1, bs * blocks // 3)
            s.submit(next_id, [rng.randrange(5) for _ in range(n)], 0.0, None, None, rng.randrange(1, 20), [99], next_id)
            submitted.add(next_id)
            next_id += 1
        if submitted - set(ended) - cancelled and rng.random() < 0.03:
            victim = rng.choice(sorted(submitted - set(ended) - cancelled))
            s.cancel(victim)
            cancelled.add(victim)
        if flight is not None:
            plan, flight = flight, None
        else:
            plan = s.plan()
            if plan.kind == sched.IDLE:
                for f in s.drain_finished().finished:
                    ended[f.id] = ended.get(f.id, 0) + 1
                idle += 1
                if next_id > 40 and not s.running and not s.waiting:
                    break
                continue
        move = rng.random()
        if plan.kind == sched.DECODE and move < 0.8:
            s.launched()
            flight = s.plan_ahead()
            if flight is not None and rng.random() < 0.15:
                s.drop_ahead()
                flight = None
        if move > 0.95:
            s.abandon()                      # the step failed: whoever saw it cancels its requests
            flight = None
            for e in plan.entries:
                if e.seq_id not in cancelled and e.seq_id not in ended:
                    s.cancel(e.seq_id)
                    cancelled.add(e.seq_id)
        else:
            tokens = [99 if rng.random() < 0.05 else 7 for _ in plan.ids]
            for f in s.commit(tokens).finished:
                ended[f.id] = ended.get(f.id, 0) + 1
        assert s.manager.in_use() + s.manager.available() == blocks
    else:
        raise AssertionError("the scheduler did not come to an end")
    assert all(count == 1 for count in ended.values()), "a request ended twice"
    assert set(ended) | cancelled == submitted, "a request was lost"
    assert s.manager.available() == blocks and s.manager.live_sequences == 0
