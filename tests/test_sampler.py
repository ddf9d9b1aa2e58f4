"""The host sampler (reference: sampler.rs:196-331) and its agreement with the plain one."""

from __future__ import annotations

import math
import random

import numpy as np
import pytest

import plain_qwen3 as plain
from paged_llm_rs_amd.errors import ConfigError
from paged_llm_rs_amd.sampling import Rng, Sampling, sample_host

SPREAD = [1.0, 0.0, -1.0, -2.0]     # softmax close to 0.64, 0.24, 0.09, 0.03


def test_greedy_takes_the_largest_and_never_draws():
    rng = Rng(1)
    assert sample_host(Sampling.greedy(), SPREAD, rng) == 0
    assert rng.state == 1, "the generator has not moved"
    assert sample_host(Sampling.greedy(), [0.5, 2.0, 2.0, -1.0], rng) == 1, "the first maximum wins"


def test_top_k_of_one_is_greedy_whatever_the_temperature():
    rng = Rng(7)
    s = Sampling(5.0, 1, None)
    assert all(sample_host(s, SPREAD, rng) == 0 for _ in range(50))


def test_the_same_seed_gives_the_same_tokens():
    s = Sampling(1.0, None, None)

    def draw(seed):
        rng = Rng(seed)
        return [sample_host(s, SPREAD, rng) for _ in range(40)]

    assert draw(42) == draw(42)
    assert draw(42) != draw(43)


def test_the_draw_follows_the_distribution_it_claims():
    s = Sampling(1.0, None, None)
    rng = Rng(20260726)
    draws = 200_000
    counts = [0] * 4
    for _ in range(draws):
        counts[sample_host(s, SPREAD, rng)] += 1
    total = sum(math.exp(l) for l in SPREAD)
    for i, l in enumerate(SPREAD):
        assert abs(counts[i] / draws - math.exp(l) / total) < 0.005


def test_top_p_keeps_the_token_that_crosses_the_threshold():
    rng = Rng(3)
    s = Sampling(1.0, None, 0.5)
    assert all(sample_host(s, SPREAD, rng) == 0 for _ in range(50))
    s = Sampling(1.0, None, 0.8)
    assert {sample_host(s, SPREAD, rng) for _ in range(200)} == {0, 1}


def test_parameters_out_of_range_are_refused():
    for args in ((-0.1, None, None), (float("nan"), None, None), (1.0, 0, None), (1.0, None, 0.0), (1.0, None, 1.5)):
        with pytest.raises(ConfigError):
            Sampling(*args)
    Sampling(1.0, 20, 0.95)


def test_empty_logits_are_an_error():
    with pytest.raises(ConfigError):
        sample_host(Sampling.greedy(), [], Rng(1))
    with pytest.raises(ConfigError):
        sample_host(Sampling(1.0, None, None), [], Rng(1))


def test_a_top_k_past_the_vocabulary_is_the_whole_vocabulary():
    rng = Rng(11)
    s = Sampling(1.0, 1000, None)
    assert {sample_host(s, SPREAD, rng) for _ in range(500)} == {0, 1, 2, 3}


def test_the_generator_spreads_over_the_unit_interval():
    rng = Rng(99)
    buckets = [0] * 10
    for _ in range(100_000):
        x = rng.next_f32()
        assert 0.0 <= x < 1.0
        buckets[int(x * 10)] += 1
    assert all(9_000 < b < 11_000 for b in buckets)
    a, b = Rng(5), plain.SplitMix64(5)
    assert [a.next_u64() for _ in range(10)] == [b.next_u64() for _ in range(10)]


@pytest.mark.parametrize("seed", range(4))
def test_native_and_plain_samplers_pick_the_same_tokens(seed):
    r = random.Random(seed)
    rs = np.random.RandomState(seed)
    for _ in range(60):
        V = r.choice([7, 50, 331])
        logits = (rs.randn(V) * r.choice([0.5, 2.0, 6.0])).astype(np.float32)
        if r.random() < 0.3:
            logits[r.randrange(V)] = logits[r.randrange(V)]     # a tie
        t = r.choice([0.0, 0.3, 0.8, 1.0, 2.5])
        k = r.choice([None, None, 1, 5, 40, 1000])
        p = r.choice([None, None, 0.1, 0.5, 0.9, 1.0])
        s0 = r.randrange(2 ** 63)
        a, b = Rng(s0), plain.SplitMix64(s0)
        how = Sampling(t, k, p)
        for _ in range(5):
            assert sample_host(how, logits, a) == plain.sample(logits, t, k, p, b)
        assert a.state == b.state
