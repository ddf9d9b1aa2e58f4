"""Generation through the entry point: greedy against the plain implementation,
what happens when pages run out, prefix sharing, sampling with a seed, the
command line."""

from __future__ import annotations

import json
import subprocess
import sys

import pytest
import torch

import plain_qwen3 as plain
import replay_util as ru
from conftest import ROOT, TINY_INIT, load_plain

pytestmark = pytest.mark.gpu


def plain_greedy_check(model_dir, prompt, produced, noise):
    """Every produced token is the plain implementation's argmax, or differs from it
    by less than the engine's rounding noise (the reference's rule for bfloat16:
    tests/reference_model.rs:260-297)."""
    cfg, weights = load_plain(model_dir)
    tokens = list(prompt)
    for token in produced:
        logits = plain.forward(weights, cfg, tokens)[-1]
        best = int(torch.argmax(logits))
        if token != best:
            gap = float(logits[best] - logits[token])
            assert gap <= noise * float(logits.abs().max()), f"token {token} against {best}: gap {gap:.3e}"
        tokens.append(token)


@pytest.mark.parametrize("name,dtype,chunk", [("A", "f32", 128), ("B", "f32", 7), ("B", "bf16", 7),
                                              ("A", "bf16", None), ("C", "f32", 5)])
def test_greedy_generation_matches_the_plain_implementation(model_dirs, name, dtype, chunk):
    from paged_llm_rs_amd import Engine

    long_name = "float32" if dtype == "f32" else "bfloat16"
    d = model_dirs(name, long_name)
    vocab = TINY_INIT[name]["config"]["vocab_size"]
    prompts = list(ru.make_prompts(vocab, [5, 17, 33, 1], seed=3).values())
    engine = Engine(d, dtype=dtype, block_size=8, num_blocks=64, max_batch=4, chunk=chunk)
    out = engine.generate(prompts, max_tokens=16, temperature=0.0, stop_tokens=[])
    for prompt, result in zip(prompts, out):
        assert result["finish"] == "length" and len(result["tokens"]) == 16
        assert result["prompt_tokens"] == len(prompt)
        plain_greedy_check(d, prompt, result["tokens"], 1e-5 if dtype == "f32" else 2e-2)
    m = engine.metrics()
    assert m["available"] == m["total"] and m["tokens"] == 64
    # (these sizes are whole strips: a bfloat16 model keeps its matrices a second time, and says so)
    assert ("GiB more for their copies in strips" in engine.describe()) == (dtype == "bf16" and name in "AB")
    stored, strips = engine.model.matrix_bytes()
    assert strips == (stored if dtype == "bf16" and name in "AB" else 0)


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_greedy_generation_that_does_not_repeat_the_prompts_last_token(tmp_path, dtype):
    """With small weights and a tied head a random model's most likely next token is the one it was just
    given, and a model with every layer left out would pass a comparison of tokens.  Here the head is its
    own matrix and the weights are large: the tokens wander, and every one is the plain implementation's."""
    from paged_llm_rs_amd import Engine
    from paged_llm_rs_amd.weights import write_random_model

    config = TINY_INIT["B"]["config"]
    long_name = "float32" if dtype == "f32" else "bfloat16"
    d = write_random_model(tmp_path / "m", config, seed=21, std=0.3, gain_std=0.2, dtype=long_name)
    prompts = list(ru.make_prompts(config["vocab_size"], [5, 17, 33, 2], seed=4).values())
    engine = Engine(d, dtype=dtype, block_size=8, num_blocks=64, max_batch=4, chunk=9)
    out = engine.generate(prompts, max_tokens=16, temperature=0.0, stop_tokens=[])
    for prompt, result in zip(prompts, out):
        tokens = result["tokens"]
        assert len(tokens) == 16
        assert tokens[0] != prompt[-1] and len(set(tokens)) >= 4, f"{prompt[-1]} then {tokens}"
        plain_greedy_check(d, prompt, tokens, 1e-5 if dtype == "f32" else 2e-2)


def test_running_out_of_pages_changes_no_token(model_dirs):
    """Eviction recomputes a request from its history; the tokens it had already
    returned stay returned and the rest come out the same."""
    from paged_llm_rs_amd import Engine

    d = model_dirs("A", "float32")
    prompts = list(ru.make_prompts(256, [9, 12, 7, 10], seed=8).values())
    roomy = Engine(d, dtype="f32", block_size=4, num_blocks=64, max_batch=4, chunk=16, prefix_cache=False)
    want = roomy.generate(prompts, max_tokens=24, stop_tokens=[])
    tight = Engine(d, dtype="f32", block_size=4, num_blocks=18, max_batch=4, chunk=16, prefix_cache=False)
    got = tight.generate(prompts, max_tokens=24, stop_tokens=[])
    assert tight.metrics()["preemptions"] > 0, "the pool was meant to run dry"
    assert [g["tokens"] for g in got] == [w["tokens"] for w in want]
    assert sum(g["preemptions"] for g in got) == tight.metrics()["preemptions"]
    assert tight.metrics()["available"] == 18


def test_a_prompt_the_pool_cannot_hold_is_refused(model_dirs):
    from paged_llm_rs_amd import Engine

    engine = Engine(model_dirs("A", "float32"), dtype="f32", block_size=4, num_blocks=4, max_batch=2, chunk=8)
    out = engine.generate([[1] * 40, [2, 3]], max_tokens=3, stop_tokens=[])
    assert out[0]["finish"] == "length" and out[0]["tokens"] == []
    assert len(out[1]["tokens"]) == 3


def test_prefix_sharing_changes_no_token(model_dirs):
    """Two prompts with a common head of 16 tokens (two pages of 8): shared and
    unshared runs give the same tokens (reference: tests/prefix.rs:87-139)."""
    from paged_llm_rs_amd import Engine

    d = model_dirs("B", "float32")
    head = list(ru.make_prompts(384, [16], seed=5).values())[0]
    tails = list(ru.make_prompts(384, [9, 24, 3], seed=6).values())
    prompts = [head + t for t in tails] + [head + tails[0]]
    on = Engine(d, dtype="f32", block_size=8, num_blocks=64, max_batch=1, chunk=7, prefix_cache=True)
    off = Engine(d, dtype="f32", block_size=8, num_blocks=64, max_batch=1, chunk=7, prefix_cache=False)
    got = on.generate(prompts, max_tokens=8, stop_tokens=[])
    want = off.generate(prompts, max_tokens=8, stop_tokens=[])
    assert [g["tokens"] for g in got] == [w["tokens"] for w in want]
    assert on.metrics()["cached_tokens"] >= 3 * 16 and off.metrics()["cached_tokens"] == 0
    assert on.metrics()["prefix_cache"] == "on" and "prefix cache on" in on.describe()
    assert off.metrics()["prefix_cache"] == "off" and "prefix cache off" in off.describe()
    assert got[0]["tokens"] == got[3]["tokens"], "the same prompt gives the same tokens"


@pytest.mark.parametrize("sampler", ["device", "host"])
def test_sampling_with_a_seed_repeats_and_stop_tokens_end_a_request(model_dirs, sampler):
    from paged_llm_rs_amd import Engine

    d = model_dirs("B", "float32")
    prompts = list(ru.make_prompts(384, [1, 9, 24, 40], seed=1).values())
    engine = Engine(d, dtype="f32", block_size=8, num_blocks=64, max_batch=4, chunk=7, sampler=sampler)
    a = engine.generate(prompts, max_tokens=12, temperature=0.8, seed=1234, stop_tokens=[])
    b = engine.generate(prompts, max_tokens=12, temperature=0.8, seed=1234, stop_tokens=[])
    c = engine.generate(prompts, max_tokens=12, temperature=0.8, seed=99, stop_tokens=[])
    assert [x["tokens"] for x in a] == [x["tokens"] for x in b]
    assert [x["tokens"] for x in a] != [x["tokens"] for x in c]
    # the plain sampler on the plain logits, with the request's own generator, picks the same tokens
    cfg, weights = load_plain(d)
    rng = plain.SplitMix64(1234 + 1)
    tokens = list(prompts[1])
    for produced in a[1]["tokens"]:
        logits = plain.forward(weights, cfg, tokens)[-1].float().numpy()
        assert plain.sample(logits, 0.8, None, None, rng) == produced
        tokens.append(produced)
    # a stop token ends the request and is not part of the output
    stop = a[0]["tokens"][3]
    cut = engine.generate(prompts[:1], max_tokens=12, temperature=0.8, seed=1234, stop_tokens=[stop])
    assert cut[0]["finish"] == "stop" and cut[0]["tokens"] == a[0]["tokens"][:a[0]["tokens"].index(stop)]
    # top_k 1 is greedy whatever the temperature
    g = engine.generate(prompts[:2], max_tokens=6, temperature=0.0, stop_tokens=[])
    k = engine.generate(prompts[:2], max_tokens=6, temperature=3.0, top_k=1, seed=5, stop_tokens=[])
    assert [x["tokens"] for x in g] == [x["tokens"] for x in k]


@pytest.mark.parametrize("sampler", ["device", "host"])
def test_sampling_with_cuts_over_a_vocabulary_of_thousands(model_dirs, sampler):
    """Several requests at once, each with its own generator, temperature, top-k and top-p over 4,099 logits:
    the plain sampler on the plain model's logits picks the tokens the engine picked (sampler.rs:113-183)."""
    from paged_llm_rs_amd import Engine

    d = model_dirs("D", "float32")
    vocab = TINY_INIT["D"]["config"]["vocab_size"]
    prompts = list(ru.make_prompts(vocab, [5, 23, 12], seed=8).values())
    cfg, weights = load_plain(d)
    engine = Engine(d, dtype="f32", block_size=16, num_blocks=32, max_batch=4, chunk=16, sampler=sampler)
    for temperature, top_k, top_p in ((0.9, 40, 0.9), (1.3, None, 0.7), (0.7, 300, None)):
        out = engine.generate(prompts, max_tokens=8, temperature=temperature, top_k=top_k, top_p=top_p, seed=77,
                              stop_tokens=[])
        assert len({tuple(o["tokens"]) for o in out}) == 3
        for i, (prompt, result) in enumerate(zip(prompts, out)):
            rng = plain.SplitMix64(77 + i)
            tokens = list(prompt)
            for produced in result["tokens"]:
                logits = plain.forward(weights, cfg, tokens)[-1].float().numpy()
                assert plain.sample(logits, temperature, top_k, top_p, rng) == produced, (temperature, top_k, top_p, i)
                tokens.append(produced)


def test_the_command_line(model_dirs, tmp_path):
    d = model_dirs("A", "float32")
    proc = subprocess.run(
        [sys.executable, str(ROOT / "bin" / "pagedllm"), "--model", str(d), "--dtype", "f32", "--max-tokens", "5",
         "--block-size", "16", "--cache-mib", "1", "--max-batch", "2", "--chunk", "off", "--prefix-cache", "off",
         "--prompt-ids", "3,17,42,8", "--prompt-ids", "1 2 3", "--temperature", "0", "--stop-ids", ""],
        capture_output=True, text=True, timeout=600)
    assert proc.returncode == 0, proc.stderr[-2000:]
    lines = [json.loads(l) for l in proc.stdout.strip().splitlines()]
    assert len(lines) == 2 and all(len(l["tokens"]) == 5 and l["finish"] == "length" for l in lines)
    assert "blocks of 16 tokens" in proc.stderr
    plain_greedy_check(d, [3, 17, 42, 8], lines[0]["tokens"], 1e-5)
    bad = subprocess.run([sys.executable, str(ROOT / "bin" / "pagedllm"), "--model", str(d), "--chunk", "0"],
                         capture_output=True, text=True, timeout=600)
    assert bad.returncode == 1 and "--chunk 0" in bad.stderr
    # bfloat16 with and without the second copy of the matrices: the same tokens, and the banner says which
    b = model_dirs("A", "bfloat16")
    runs = {}
    for strips in ("on", "off"):
        proc = subprocess.run(
            [sys.executable, str(ROOT / "bin" / "pagedllm"), "--model", str(b), "--max-tokens", "6", "--strips", strips,
             "--prompt-ids", "3,17,42,8", "--temperature", "0", "--stop-ids", ""], capture_output=True, text=True, timeout=600)
        assert proc.returncode == 0, proc.stderr[-2000:]
        assert ("copies in strips" in proc.stderr) == (strips == "on")
        runs[strips] = json.loads(proc.stdout.strip().splitlines()[0])["tokens"]
    assert runs["on"] == runs["off"] and len(runs["on"]) == 6


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_captured_decode_step_replays_like_the_eager_one(model_dirs, dtype):
    """Every replay of the decode graph is checked against the eager step, with eager
    work and synchronisations in between, over requests that come and go, cross page
    edges and outgrow the graph's table."""
    from paged_llm_rs_amd.engine.replay import Replayer

    d = model_dirs("B", dtype)
    prompts = ru.make_prompts(384, [30, 3, 17, 9, 40], seed=21)
    steps = []
    live = {}
    order = list(prompts.items())
    rng = __import__("random").Random(4)
    fed = {}
    # a first step with whole prompt heads (eager), then single tokens (graph), requests ending at different times
    heads = {n: max(1, len(t) - rng.choice([3, 8, 14])) for n, t in order}
    steps.append({"step": 0, "entries": [{"id": n, "tokens": t[:heads[n]], "want": [heads[n] - 1]} for n, t in order[:4]],
                  "end": []})
    fed = {n: heads[n] for n, _ in order[:4]}
    k = 1
    while fed:
        entries, end = [], []
        for n in list(fed):
            t = prompts[n]
            entries.append({"id": n, "tokens": [t[fed[n]]], "want": [0]})
            fed[n] += 1
            if fed[n] == len(t):
                end.append(n)
                del fed[n]
        steps.append({"step": k, "entries": entries, "end": end})
        k += 1
        if k == 4:      # a late arrival: one eager step in the middle, then it joins the graph steps
            n, t = order[4]
            steps.append({"step": k, "entries": [{"id": n, "tokens": t[:heads[n]], "want": [heads[n] - 1]}], "end": []})
            fed[n] = heads[n]
            k += 1
    eager = Replayer(d, dtype, max_tokens=64 * 5, block_size=8, graphs=False)
    graph = Replayer(d, dtype, max_tokens=64 * 5, block_size=8, graphs=True)
    a = ru.collect(eager, steps)
    b = ru.collect(graph, steps)
    assert graph.runner.graph_steps > 10 and eager.runner.graph_steps == 0
    assert a.keys() == b.keys()
    for key in a:
        assert np.array_equal(a[key], b[key]), f"{key}: a replay differs from the eager step"


@pytest.mark.parametrize("name,dtype,block_size", [("B", "float32", 8), ("B", "bfloat16", 8), ("E", "bfloat16", 16)])
def test_a_shape_of_step_that_comes_again_is_captured_and_replays_like_the_eager_one(model_dirs, name, dtype, block_size):
    """A long prompt cut into equal portions beside a request that decodes: from its second coming on a
    shape of step is replayed from a graph.  Every replay is checked against the eager step, over
    growing contexts (the tables outgrow the capture once) and with other shapes in between.  (The wide
    model's captured steps hold the library's products and the grouped attention kernel.)"""
    from paged_llm_rs_amd.engine.replay import Replayer

    d = model_dirs(name, dtype)
    prompts = ru.make_prompts(TINY_INIT[name]["config"]["vocab_size"], [300, 60, 23], seed=33)
    long_one, other, third = prompts["r0"], prompts["r1"], prompts["r2"]
    steps, k = [], 0
    steps.append({"step": k, "entries": [{"id": "r1", "tokens": other[:20], "want": [19]}], "end": []})
    k += 1
    fed, at = 20, 0
    while at < 294:
        entries = [{"id": "r0", "tokens": long_one[at:at + 21], "want": [20] if at + 21 >= 294 else []}]
        if fed < len(other):
            entries.append({"id": "r1", "tokens": [other[fed]], "want": [0]})
            fed += 1
        steps.append({"step": k, "entries": entries, "end": []})
        at += 21
        k += 1
        if k == 6:      # another shape in between
            steps.append({"step": k, "entries": [{"id": "r2", "tokens": third, "want": [len(third) - 1]}], "end": ["r2"]})
            k += 1
    steps.append({"step": k, "entries": [{"id": "r0", "tokens": long_one[294:], "want": [5]}], "end": ["r0", "r1"]})
    eager = Replayer(d, dtype, max_tokens=64 * 8, block_size=block_size, graphs=False)
    graph = Replayer(d, dtype, max_tokens=64 * 8, block_size=block_size, graphs=True)
    a = ru.collect(eager, steps)
    b = ru.collect(graph, steps)
    assert graph.runner.graph_steps >= 10 and eager.runner.graph_steps == 0
    assert a.keys() == b.keys() and len(a) >= 12
    for key in a:
        assert np.array_equal(a[key], b[key]), f"{key}: a replay differs from the eager step"


@pytest.mark.parametrize("lap", [1, 8])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_portions_that_return_nothing_replay_like_eager_ones(model_dirs, dtype, lap, monkeypatch):
    """Equal portions in the middle of a prompt give nothing to read, so nothing makes the host wait for
    the device between them: each replay still has to run on its own step's descriptor, not on the next
    one's, which the host is already writing.  (The pinned descriptors are used in turn; with a lap of one
    buffer every step waits for the copy before it, with the usual lap only every eighth.)"""
    from paged_llm_rs_amd.engine import step
    from paged_llm_rs_amd.engine.replay import Replayer

    monkeypatch.setattr(step._DescriptorRing, "LAP", lap)

    d = model_dirs("C", dtype)
    prompt = ru.make_prompts(TINY_INIT["C"]["config"]["vocab_size"], [150], seed=41)["r0"]
    results = {}
    for portion in (7, 2):
        steps = []
        for k, at in enumerate(range(0, len(prompt), portion)):
            tokens = prompt[at:at + portion]
            last = at + portion >= len(prompt)
            steps.append({"step": k, "entries": [{"id": "r0", "tokens": tokens, "want": [len(tokens) - 1] if last else []}],
                          "end": ["r0"] if last else []})
        for graphs in (False, True):
            r = Replayer(d, dtype, max_tokens=256, block_size=4, graphs=graphs)
            results[(portion, graphs)] = ru.collect(r, steps)
            if graphs:
                assert r.runner.graph_steps >= 10
        a, b = results[(portion, False)], results[(portion, True)]
        assert a.keys() == b.keys() and len(a) == 1
        for key in a:
            assert np.array_equal(a[key], b[key]), f"portions of {portion}: a replay differs from the eager step"


def drawn_engine_case(case: int):
    import random

    rng = random.Random(case)
    name = rng.choice("ABC")
    vocab = TINY_INIT[name]["config"]["vocab_size"]
    head = [rng.randrange(vocab) for _ in range(rng.choice([0, 8, 16, 33]))]
    prompts = []
    for _ in range(rng.randint(2, 9)):
        body = [rng.randrange(vocab) for _ in range(rng.randint(1, 60))]
        prompts.append((head if rng.random() < 0.6 else []) + body)
    if rng.random() < 0.3:
        prompts.append(list(prompts[0]))
    max_tokens = rng.randint(1, 40)
    block_size = rng.choice([1, 2, 4, 8, 16])
    one = -(-(max(len(p) for p in prompts) + max_tokens) // block_size)      # pages of the longest request
    settings = dict(block_size=block_size, num_blocks=rng.choice([one + 1, one * 2, one * 4, 10 * one]),
                    max_batch=rng.choice([1, 2, 3, 4, 6, 8]), chunk=rng.choice([None, 2, 3, 7, 16, 64]),
                    prefix_cache=rng.random() < 0.5, sampler=rng.choice(["device", "host"]))
    sampling = rng.choice([dict(temperature=0.0), dict(temperature=0.8, seed=case),
                           dict(temperature=1.2, top_k=20, top_p=0.9, seed=case)])
    return name, prompts, max_tokens, settings, sampling


@pytest.mark.parametrize("case", range(16))
def test_the_engines_settings_change_no_token(model_dirs, case):
    """Page size, pool (down to one request's worth and a page), requests a step, portion size, prefix
    sharing and the sampler's place, all drawn: in 32-bit the tokens are those of an engine that runs the
    requests one by one, whole, with room to spare; greedy and drawn with a seed."""
    from paged_llm_rs_amd import Engine

    name, prompts, max_tokens, settings, sampling = drawn_engine_case(case)
    d = model_dirs(name, "float32")
    roomy = Engine(d, dtype="f32", block_size=16, num_blocks=64 * len(prompts), max_batch=1, chunk=None,
                   prefix_cache=False, sampler=settings["sampler"], ahead=False)
    want = roomy.generate(prompts, max_tokens=max_tokens, stop_tokens=[], **sampling)
    engine = Engine(d, dtype="f32", **settings)
    got = engine.generate(prompts, max_tokens=max_tokens, stop_tokens=[], **sampling)
    assert [g["tokens"] for g in got] == [w["tokens"] for w in want], f"{settings} {sampling}"
    m = engine.metrics()
    if not settings["prefix_cache"]:
        assert m["available"] == m["total"]


@pytest.mark.parametrize("case", range(8))
def test_requests_that_arrive_and_are_cancelled_while_others_run(model_dirs, case):
    """Requests are submitted at drawn steps, some are cancelled a few steps later, the pool is drawn from
    tight to roomy: every request that finishes has the tokens it has alone in an engine with room to
    spare, and without prefix sharing every page is free again at the end."""
    import random

    from paged_llm_rs_amd import Engine

    rng = random.Random(1000 + case)
    name = rng.choice("ABC")
    vocab = TINY_INIT[name]["config"]["vocab_size"]
    head = [rng.randrange(vocab) for _ in range(rng.choice([0, 8, 16, 33]))]
    requests = []
    for i in range(rng.randint(3, 14)):
        prompt = (head if rng.random() < 0.6 else []) + [rng.randrange(vocab) for _ in range(rng.randint(1, 60))]
        sampling = rng.choice([dict(temperature=0.0), dict(temperature=0.8, seed=case * 100 + i),
                               dict(temperature=1.2, top_k=20, top_p=0.9, seed=case * 100 + i)])
        requests.append(dict(prompt=prompt, max_tokens=rng.randint(1, 30), sampling=sampling, arrives=rng.randint(0, 40),
                             cancelled_after=rng.randint(1, 25) if rng.random() < 0.2 else None))
    block_size = rng.choice([1, 2, 4, 8, 16])
    one = -(-max(len(r["prompt"]) + r["max_tokens"] for r in requests) // block_size)
    settings = dict(block_size=block_size, num_blocks=rng.choice([one + 1, one * 2, one * 4, 10 * one]),
                    max_batch=rng.choice([1, 2, 3, 4, 6, 8]), chunk=rng.choice([None, 2, 3, 7, 16, 64]),
                    prefix_cache=rng.random() < 0.5, sampler=rng.choice(["device", "host"]))
    d = model_dirs(name, "float32")
    roomy = Engine(d, dtype="f32", block_size=16, num_blocks=64 * len(requests), max_batch=1, chunk=None,
                   prefix_cache=False, sampler=settings["sampler"], ahead=False)
    for r in requests:
        i = roomy.submit(r["prompt"], r["max_tokens"], stop_tokens=[], **r["sampling"])
        roomy.run()
        r["want"] = roomy.take_result(i).tokens
    engine = Engine(d, dtype="f32", **settings)
    step = 0
    while any("id" not in r for r in requests) or engine.open_requests:
        for r in requests:
            if "id" not in r and r["arrives"] <= step:
                r["id"] = engine.submit(r["prompt"], r["max_tokens"], stop_tokens=[], **r["sampling"])
                r["submitted"] = step
            if (r.get("cancelled_after") is not None and "id" in r and not r.get("gone")
                    and r["submitted"] + r["cancelled_after"] <= step):
                engine.cancel(r["id"])
                r["gone"] = True
        if engine.open_requests:
            assert engine.step() is not None or not engine.open_requests, "the scheduler idles while requests are open"
        step += 1
        assert step < 5000
    for r in requests:
        if not r.get("gone"):
            assert engine.take_result(r["id"]).tokens == r["want"], f"{settings}"
    m = engine.metrics()
    if not settings["prefix_cache"]:
        assert m["available"] == m["total"]


@pytest.mark.parametrize("name,seed", [("D", 0), ("E", 1)])
def test_a_long_run_of_arrivals_gives_the_same_tokens_from_graphs_as_kernel_by_kernel(model_dirs, name, seed, monkeypatch):
    """A hundred requests of drawn lengths arriving over some hundred steps, in bfloat16, greedy and drawn:
    steps of many shapes are captured, dropped again (few rows of captured shapes are kept here) and
    captured again, tables and contexts outgrow their captures; every token is the one that the same
    engine gives when it launches every step kernel by kernel."""
    import random

    from paged_llm_rs_amd import Engine
    from paged_llm_rs_amd.engine import step as step_module

    monkeypatch.setattr(step_module, "SHAPE_GRAPH_ROWS_KEPT", 2048)
    rng = random.Random(seed)
    vocab = TINY_INIT[name]["config"]["vocab_size"]
    head = [rng.randrange(vocab) for _ in range(48)]
    requests, at = [], 0
    for i in range(100):
        at += rng.choice([0, 0, 1, 2, 5, 20])
        body = [rng.randrange(vocab) for _ in range(rng.choice([rng.randint(1, 40), rng.randint(100, 400)]))]
        sampling = rng.choice([dict(temperature=0.0), dict(temperature=0.9, top_k=40, top_p=0.95, seed=i)])
        requests.append(((head if rng.random() < 0.3 else []) + body, rng.randint(1, 40), sampling, at))
    settings = dict(block_size=16, num_blocks=400, max_batch=rng.choice([8, 24, 64]), chunk=rng.choice([64, 128, 512]))
    d = model_dirs(name, "bfloat16")
    tokens = {}
    for graphs in (False, True):
        engine = Engine(d, dtype="bf16", graphs=graphs, **settings)
        ids, step = {}, 0
        while len(ids) < len(requests) or engine.open_requests:
            for r, (prompt, most, sampling, arrives) in enumerate(requests):
                if r not in ids and arrives <= step:
                    ids[r] = engine.submit(prompt, most, stop_tokens=[], **sampling)
            if engine.open_requests:
                engine.step()
            step += 1
            assert step < 5000
        tokens[graphs] = [engine.take_result(ids[r]).tokens for r in range(len(requests))]
        if graphs:
            assert engine.runner.graph_steps > 5 * engine.runner.eager_steps
    assert tokens[True] == tokens[False]


import numpy as np  # noqa: E402


# ---------------------------------------------------------------------------
# Steps queued ahead: the next decoding step is on the device before the tokens of
# the one before have been read.
# ---------------------------------------------------------------------------

def _generate_each(engine, prompts, budgets, stop, drawn=False):
    how = [dict(temperature=0.0)] * len(prompts)
    if drawn:        # some draw, some take the largest logit, in one step
        how = [dict(temperature=0.9, seed=40 + i) if i % 3 else dict(temperature=0.0) for i in range(len(prompts))]
        how[2] = dict(temperature=1.1, top_k=30, top_p=0.95, seed=7)
    ids = [engine.submit(p, m, stop_tokens=stop, **h) for p, m, h in zip(prompts, budgets, how)]
    engine.run()
    return [engine.take_result(i) for i in ids]


@pytest.mark.parametrize("name,dtype,graphs,drawn", [("B", "f32", True, False), ("C", "f32", True, False),
                                                     ("B", "f32", False, False), ("B", "bf16", True, False),
                                                     ("B", "f32", True, True), ("C", "f32", False, True)])
def test_steps_queued_ahead_change_no_token(model_dirs, name, dtype, graphs, drawn):
    """Requests of different budgets, one of them ended by a stop token in the middle: with the next step
    queued before a step's tokens are read, every request has the tokens, and the ending, that it has in
    an engine that reads every step's tokens before it plans the next.  ``drawn``: most requests draw
    their tokens (with seeds), which the sampling kernel does behind each step."""
    from paged_llm_rs_amd import Engine

    long_name = "float32" if dtype == "f32" else "bfloat16"
    d = model_dirs(name, long_name)
    vocab = TINY_INIT[name]["config"]["vocab_size"]
    prompts = list(ru.make_prompts(vocab, [9, 21, 4, 14, 30], seed=11).values())
    budgets = [40, 12, 33, 25, 18]
    settings = dict(dtype=dtype, block_size=8, num_blocks=96, max_batch=8, chunk=64, prefix_cache=False, graphs=graphs)
    free = _generate_each(Engine(d, ahead=False, **settings), prompts, budgets, [], drawn)
    # a token that a request produces in the middle and not before stops it there (and whomever else it meets)
    who, at = next((r, i) for r in (2, 0, 3) for i in range(6, len(free[r].tokens) - 2)
                   if free[r].tokens[i] not in free[r].tokens[:i])
    mine = free[who].tokens
    stop = [mine[at]]
    want = _generate_each(Engine(d, ahead=False, **settings), prompts, budgets, stop, drawn)
    assert want[who].finish == "stop" and want[who].tokens == mine[:at]
    engine = Engine(d, ahead=True, **settings)
    got = _generate_each(engine, prompts, budgets, stop, drawn)
    if dtype == "f32":
        assert [g.tokens for g in got] == [w.tokens for w in want]
        assert [g.finish for g in got] == [w.finish for w in want]
    else:
        # (in bfloat16 the row that runs once more for the stopped request is rounding noise to the others)
        for prompt, g, budget in zip(prompts, got, budgets):
            plain_greedy_check(d, prompt, g.tokens, 2e-2)
            assert g.finish == "stop" or len(g.tokens) == budget
    m = engine.metrics()
    assert m["steps_ahead"] >= 20, "hardly a step was queued ahead"
    assert m["available"] == m["total"]
    # and a second round on the same engine: whatever was in flight at the end of the first is gone
    again = _generate_each(engine, prompts, budgets, stop, drawn)
    assert [g.tokens for g in again] == [g.tokens for g in got]


@pytest.mark.parametrize("name,chunk,drawn", [("B", 64, False), ("C", None, False), ("B", None, True)])
def test_steps_are_queued_ahead_in_a_crowded_engine(model_dirs, name, chunk, drawn):
    """More requests than rows and than the pages hold at once: some wait in the queue, some residents have no
    row in a step.  Steps are queued ahead all the same while the queue cannot move, rows of requests that had
    none in the step before bring their own token beside rows that are fed on the device, and every request has
    the tokens and the ending of an engine that reads every step's tokens first."""
    from paged_llm_rs_amd import Engine

    d = model_dirs(name, "float32")
    vocab = TINY_INIT[name]["config"]["vocab_size"]
    prompts = list(ru.make_prompts(vocab, [9, 21, 4, 14, 30, 7, 12], seed=23).values())
    budgets = [30, 9, 26, 17, 12, 21, 5]
    settings = dict(dtype="f32", block_size=8, num_blocks=16, max_batch=3, chunk=chunk, prefix_cache=False)
    want = _generate_each(Engine(d, ahead=False, **settings), prompts, budgets, [], drawn)
    engine = Engine(d, ahead=True, **settings)
    got = _generate_each(engine, prompts, budgets, [], drawn)
    assert [g.tokens for g in got] == [w.tokens for w in want]
    assert [g.finish for g in got] == [w.finish for w in want]
    m = engine.metrics()
    assert m["steps_ahead"] >= 0.5 * m["decode_steps"], (m["steps_ahead"], m["decode_steps"])
    assert m["admission_stalls"] > 0 and m["preemptions"] > 0, "the engine was not crowded"
    assert m["available"] == m["total"]


@pytest.mark.parametrize("case", range(8))
def test_steps_queued_ahead_change_no_token_under_drawn_loads(model_dirs, case):
    """Drawn loads on drawn engines, most of them crowded (few rows, few pages, stop tokens that end requests in the
    middle, some requests drawing their tokens): every request has the tokens and the ending it has in an engine
    that reads every step's tokens before it plans the next, and every page comes back."""
    import random

    from paged_llm_rs_amd import Engine

    rng = random.Random(1000 + case)
    name = rng.choice("ABC")
    d = model_dirs(name, "float32")
    vocab = TINY_INIT[name]["config"]["vocab_size"]
    n = rng.randint(3, 24)
    prompts = [[rng.randrange(vocab) for _ in range(rng.choice([rng.randint(1, 12), rng.randint(20, 60)]))] for _ in range(n)]
    budgets = [rng.randint(1, 40) for _ in range(n)]
    bs = rng.choice([4, 8, 16])
    need_one = -(-max(len(p) + b for p, b in zip(prompts, budgets)) // bs)
    settings = dict(dtype="f32", block_size=bs, num_blocks=rng.choice([need_one + 1, need_one * 2, need_one * 3, 8 * need_one]),
                    max_batch=rng.choice([1, 2, 3, 5, 8, 40]), chunk=rng.choice([None, 4, 16, 64]), prefix_cache=False,
                    graphs=rng.random() < 0.7)
    drawn = rng.random() < 0.4
    stops = [rng.randrange(vocab) for _ in range(rng.choice([0, 0, 3, 12]))]
    results = {}
    for ahead in (False, True):
        engine = Engine(d, ahead=ahead, **settings)
        ids = [engine.submit(p, b, stop_tokens=stops, **(dict(temperature=0.9, seed=50 + i) if drawn and i % 2 else dict(temperature=0.0)))
               for i, (p, b) in enumerate(zip(prompts, budgets))]
        engine.run()
        results[ahead] = [engine.take_result(i) for i in ids]
        m = engine.metrics()
        assert m["available"] == m["total"], "pages were lost"
    assert [(r.tokens, r.finish) for r in results[True]] == [(r.tokens, r.finish) for r in results[False]], settings


@pytest.mark.parametrize("case", range(6))
def test_without_stop_tokens_steps_queued_ahead_change_no_step(model_dirs, case):
    """In bfloat16 a token may depend on what else was in its step (another count of rows is another kernel, another
    rounding).  Where no stop token ends a request the engine runs the very same steps with and without queueing
    them ahead, so even there every request has the same tokens, bit for bit: crowded engines, requests all
    there from the start (one that arrives while a step is queued ahead comes in a step later, by design)."""
    import random

    from paged_llm_rs_amd import Engine

    rng = random.Random(4000 + case)
    name = rng.choice("ABC")
    d = model_dirs(name, "bfloat16")
    vocab = TINY_INIT[name]["config"]["vocab_size"]
    n = rng.randint(6, 24)
    prompts = [[rng.randrange(vocab) for _ in range(rng.choice([rng.randint(1, 12), rng.randint(20, 60)]))] for _ in range(n)]
    budgets = [rng.randint(1, 40) for _ in range(n)]
    bs = rng.choice([8, 16])
    need_one = -(-max(len(p) + b for p, b in zip(prompts, budgets)) // bs)
    settings = dict(dtype="bf16", block_size=bs, num_blocks=rng.choice([need_one + 1, need_one * 2, need_one * 3]),
                    max_batch=rng.choice([2, 3, 5, 8]), chunk=rng.choice([None, 16, 64]), prefix_cache=False)
    results, steps = {}, {}
    for ahead in (False, True):
        engine = Engine(d, ahead=ahead, **settings)
        ids = [engine.submit(p, b, stop_tokens=[], **(dict(temperature=0.9, seed=50 + i) if i % 2 else dict(temperature=0.0)))
               for i, (p, b) in enumerate(zip(prompts, budgets))]
        engine.run()
        results[ahead] = [engine.take_result(i).tokens for i in ids]
        m = engine.metrics()
        steps[ahead] = (m["steps"], m["decode_steps"], m["mixed_steps"], m["preemptions"])
    assert steps[True] == steps[False]
    assert results[True] == results[False], settings
    assert m["steps_ahead"] > 0


def test_an_engine_whose_model_takes_no_ids_from_the_device_plans_nothing_ahead(model_dirs, monkeypatch):
    """Taking a row's id from the step before on the device is something a model offers (``takes_fed_tokens``).  One
    that does not is driven the ordinary way, every step's tokens read before the next is planned: its decode
    graphs have no piece that names rows of the step before, and it generates what the model that offers it does."""
    from paged_llm_rs_amd import Engine
    from paged_llm_rs_amd.parts.model import DecoderModel

    d = model_dirs("B", "float32")
    vocab = TINY_INIT["B"]["config"]["vocab_size"]
    prompts = list(ru.make_prompts(vocab, [9, 21, 4], seed=5).values())
    settings = dict(dtype="f32", block_size=8, num_blocks=64, max_batch=4, chunk=64, prefix_cache=False)
    want = Engine(d, **settings).generate(prompts, max_tokens=20, stop_tokens=[])
    monkeypatch.setattr(DecoderModel, "takes_fed_tokens", False)
    engine = Engine(d, **settings)
    assert not engine.ahead
    got = engine.generate(prompts, max_tokens=20, stop_tokens=[])
    assert [g["tokens"] for g in got] == [w["tokens"] for w in want]
    assert engine.metrics()["steps_ahead"] == 0
    graphs = [g for g in engine.runner._graphs.values()]
    assert graphs and all(g.batch.token_src is None for g in graphs)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_step_takes_the_tokens_of_the_step_before_on_the_device(model_dirs, dtype):
    """The step runner alone: decoding steps whose entries name rows of the step before, in another order
    and fewer of them, give bit for bit the logits of steps that are handed the tokens."""
    import numpy as np

    from paged_llm_rs_amd.cache import PagedCache
    from paged_llm_rs_amd.engine.batch import CannotFeed, StepEntry
    from paged_llm_rs_amd.engine.step import StepRunner, commit_step
    from paged_llm_rs_amd.parts.model import DTYPES, load_model

    d = model_dirs("B", dtype)
    _, model = load_model(d, dtype, "cuda:0")
    vocab = model.spec.vocab_size
    prompts = ru.make_prompts(vocab, [11, 5, 19, 8], seed=5)

    def play(fed: bool):
        cache = PagedCache(model.cache_layout, 8, 64, DTYPES[dtype], "cuda:0", max_seqs=8)
        runner = StepRunner(model, cache)
        manager = cache.manager
        ids = {}
        for i, (name, toks) in enumerate(prompts.items(), start=1):
            manager.add_sequence(i)
            assert manager.reserve(i, len(toks))
            ids[name] = i
        first = [StepEntry(ids[n], t, 0, [len(t) - 1]) for n, t in prompts.items()]
        out = runner.run(first)
        commit_step(cache, first)
        tokens = dict(zip(ids.values(), out.greedy_on_host()))
        rows, logits, refused = None, [], 0
        orders = [[1, 2, 3, 4], [1, 2, 3, 4], [3, 1, 4, 2], [4, 3], [3, 4], [3], [3], [4, 3]]
        for order in orders:
            for i in order:
                assert manager.reserve(i, 1)
            plain = [StepEntry(i, [tokens[i]], manager.tokens(i), [0]) for i in order]
            entries = plain
            if fed and rows is not None and all(i in rows for i in order):
                entries = [StepEntry(i, [0], manager.tokens(i), [0], fed_row=rows[i]) for i in order]
            try:
                out = runner.run(entries)
            except CannotFeed:
                refused += 1
                out = runner.run(plain)
            commit_step(cache, entries)
            logits.append(out.logits.cpu().numpy().copy())
            chosen = out.greedy_on_host()
            assert chosen == out.logits.argmax(-1).tolist()
            tokens.update(zip(order, chosen))
            rows = {i: row for row, i in enumerate(order)}
        return logits, refused, runner

    handed, _, _ = play(False)
    taken, refused, runner = play(True)
    assert refused == 2, "a step that has to be captured first (of 2 requests, of 1) cannot be fed"
    for step, (a, b) in enumerate(zip(handed, taken)):
        assert np.array_equal(a, b), f"step {step}"
    # a row that the step before did not have, and a step of more than single tokens, are refused too
    with pytest.raises(CannotFeed):
        runner.run([StepEntry(3, [0], runner.cache.manager.tokens(3), [0], fed_row=2)])
    with pytest.raises(CannotFeed):
        runner.run([StepEntry(3, [0, 1], runner.cache.manager.tokens(3), [1], fed_row=0)])


@pytest.mark.parametrize("ahead,fails_in", [(False, "run"), (True, "run"), (True, "read")])
def test_a_step_that_fails_fails_its_requests_and_nothing_else(model_dirs, ahead, fails_in, monkeypatch):
    """The step function refuses a step (forced from the host: the runner is replaced by one that raises; or the
    read of a step's tokens is): the requests of that step end as failed, nothing of them stays in the cache or the
    scheduler, whether or not a step was queued ahead, and the engine serves the next request as if nothing had
    been (reference: engine.rs:340-348)."""
    from paged_llm_rs_amd import Engine
    from paged_llm_rs_amd.engine.step import StepOutput
    from paged_llm_rs_amd.errors import PagedLLMError, TensorError

    d = model_dirs("B", "float32")
    prompts = list(ru.make_prompts(384, [9, 21, 4], seed=2).values())
    settings = dict(dtype="f32", block_size=8, num_blocks=64, max_batch=4, chunk=64, prefix_cache=False)
    want = Engine(d, ahead=False, **settings).generate(prompts[:1], max_tokens=10, stop_tokens=[])
    engine = Engine(d, ahead=ahead, **settings)
    ids = [engine.submit(p, 30, temperature=0.0, stop_tokens=[]) for p in prompts]
    for _ in range(5):
        engine.step()
    assert engine.open_requests == 3 and (engine.metrics()["steps_ahead"] > 0) == ahead

    def refuse(*args, **kwargs):
        raise TensorError("the device said no")

    with monkeypatch.context() as patched:
        if fails_in == "run":
            patched.setattr(engine.runner, "run", refuse)
        else:
            patched.setattr(StepOutput, "greedy_on_host", refuse)
        with pytest.raises(PagedLLMError, match="said no"):
            engine.step()
    assert engine.open_requests == 0
    for i in ids:
        done = engine.take_result(i)
        assert done.finish == "failed" and 1 <= len(done.tokens) < 30
    m = engine.metrics()
    assert m["available"] == m["total"] and engine.scheduler.running == 0 and engine.scheduler.waiting == 0
    again = engine.generate(prompts[:1], max_tokens=10, stop_tokens=[])
    assert again[0]["tokens"] == want[0]["tokens"] and again[0]["finish"] == "length"
