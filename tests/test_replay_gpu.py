"""The engine against the plain implementation, replayed four ways, in 32-bit
and in bfloat16: each request alone and whole; most of it in one step and the
last 32 tokens one by one; in portions of changing size; mixed with other
requests and so few pages that they are used again."""

from __future__ import annotations

import json
import subprocess
import sys
from pathlib import Path

import numpy as np
import pytest
import torch

import replay_util as ru
from conftest import ROOT, TINY_INIT

pytestmark = pytest.mark.gpu

# max|got - want| / max|want|.  32-bit: the reference's own bound for its tiny
# fixture (tests/fixtures/tiny/manifest.json: 1e-5).  bfloat16: inputs of every
# product are rounded to 8 bits of mantissa (2^-9 = 2e-3 a rounding); through two
# or three layers and a head that is a few times 1e-3 of the largest logit.
TOLERANCE = {"float32": 1e-5, "bfloat16": 2e-2}
LENGTHS = {"A": [5, 17, 33, 70, 100, 41], "B": [1, 9, 24, 40, 129, 66], "C": [3, 50, 97, 64, 20, 35],
           "D": [300, 70, 33, 150], "E": [260, 70, 33, 150],
           # whole requests of these lengths put 70 and 150 rows (the library), 33, 20 and 50 rows (the three
           # shapes of the product for 17 to 64 rows) before the projection onto the vocabulary
           "V": [70, 33, 150, 20, 50]}


@pytest.fixture(scope="module")
def setups(model_dirs):
    """(model name, dtype) -> (model dir, prompts, plain logits)."""
    made = {}

    def get(name, dtype):
        if (name, dtype) not in made:
            d = model_dirs(name, dtype)
            prompts = ru.make_prompts(TINY_INIT[name]["config"]["vocab_size"], LENGTHS[name], seed=11)
            made[(name, dtype)] = (d, prompts, ru.plain_logits(d, prompts))
        return made[(name, dtype)]

    return get


class LeftoversInFreePages:
    """A replayer whose free pages hold what a page's last owner may have left there (infinities, NaNs,
    the largest finite numbers): all pages at the start, and a request's pages again when it ends."""

    def __init__(self, replayer):
        self.r = replayer
        self.spoil(range(replayer.cache.num_blocks))

    def spoil(self, pages, group=None):
        cache = self.r.cache
        bs = cache.block_size
        pattern = torch.tensor([float("inf"), float("nan"), 3e38, float("-inf")], device=cache.device)
        for g in cache.layout.groups if group is None else [group]:
            for layer in g.layers:
                for pool in cache.layer_pools(layer):
                    at = (torch.arange(bs, device=cache.device)[:, None] + torch.arange(pool.shape[1], device=cache.device)[None]) % 4
                    rows = pattern[at].to(pool.dtype)
                    for page in pages:
                        pool[page * bs:(page + 1) * bs] = rows

    def step(self, entries, end=()):
        out = self.r.step(entries, [])
        manager = self.r.cache.manager
        for name in end:
            seq = self.r.ids.pop(name)
            held = [[p for p in manager.table(seq, gi) if p >= 0] for gi in range(len(self.r.cache.layout.groups))]
            manager.free_sequence(seq)
            for gi, pages in enumerate(held):
                self.spoil(pages, self.r.cache.layout.groups[gi])
        return out


def replay(model_dir, dtype, prompts, steps, max_live, block_size=16, leftovers=False, pages=None):
    from paged_llm_rs_amd.engine.replay import Replayer

    r = Replayer(model_dir, dtype, max_tokens=ru.pool_tokens(prompts, max_live), block_size=block_size, pages=pages)
    got = ru.collect(LeftoversInFreePages(r) if leftovers else r, steps)
    assert r.cache.manager.live_sequences == 0
    assert r.cache.manager.available() == r.cache.manager.total(), "every page came back"
    return got


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C", "D", "E", "V"])
def test_whole_requests(setups, name, dtype):
    d, prompts, want = setups(name, dtype)
    got = replay(d, dtype, prompts, ru.whole(prompts), max_live=1)
    assert len(got) == sum(len(t) for t in prompts.values())
    worst, where = ru.worst_error(got, want)
    assert worst <= TOLERANCE[dtype], f"{worst:.3e} at {where}"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name,block_size", [("A", 16), ("B", 8), ("C", 4), ("D", 16), ("E", 16), ("V", 16)])
def test_last_tokens_decoded_one_by_one(setups, name, dtype, block_size):
    d, prompts, want = setups(name, dtype)
    got = replay(d, dtype, prompts, ru.tail_decoded(prompts, 32), max_live=1, block_size=block_size)
    worst, where = ru.worst_error(got, want)
    assert worst <= TOLERANCE[dtype], f"{worst:.3e} at {where}"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name,block_size", [("A", 16), ("B", 8), ("C", 4), ("D", 16), ("E", 16), ("V", 16)])
def test_portions_of_changing_size(setups, name, dtype, block_size):
    d, prompts, want = setups(name, dtype)
    # the large model gets portions of more than one tile of the attention kernel as well
    steps = ru.portions(prompts, sizes=(130, 2, 64, 7, 33, 16)) if name in "DEV" else ru.portions(prompts)
    got = replay(d, dtype, prompts, steps, max_live=1, block_size=block_size)
    worst, where = ru.worst_error(got, want)
    assert worst <= TOLERANCE[dtype], f"{worst:.3e} at {where}"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name,block_size,seed", [("A", 16, 1), ("B", 8, 2), ("C", 4, 3), ("B", 16, 4), ("D", 16, 5),
                                                    ("E", 16, 6), ("V", 16, 7)])
def test_mixed_requests_with_pages_used_again(setups, name, dtype, block_size, seed):
    d, prompts, want = setups(name, dtype)
    steps = ru.mixed(prompts, seed=seed, max_live=4)
    assert max(len(s["entries"]) for s in steps) >= 3
    assert any(len(e["tokens"]) > 1 for s in steps for e in s["entries"] if len(s["entries"]) > 1)
    got = replay(d, dtype, prompts, steps, max_live=4, block_size=block_size)
    worst, where = ru.worst_error(got, want)
    assert worst <= TOLERANCE[dtype], f"{worst:.3e} at {where}"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name,block_size", [("A", 16), ("B", 8), ("C", 4), ("D", 16), ("E", 16), ("V", 16)])
@pytest.mark.parametrize("schedule", ["whole", "tail", "portions", "mixed"])
def test_what_free_pages_hold_changes_no_logit(setups, name, dtype, block_size, schedule):
    """A page keeps what its last owner wrote.  Whatever that is, numbers that are not finite among them,
    the next owner's logits are the bits they are over pages of zeros: what a kernel reads beyond a
    request's keys is replaced, never multiplied by zero."""
    d, prompts, want = setups(name, dtype)
    live = 4 if schedule == "mixed" else 1
    steps = {"whole": lambda: ru.whole(prompts), "tail": lambda: ru.tail_decoded(prompts, 32),
             "portions": lambda: ru.portions(prompts, sizes=(130, 2, 64, 7, 33, 16)) if name in "DEV" else ru.portions(prompts),
             "mixed": lambda: ru.mixed(prompts, seed=21, max_live=4)}[schedule]()
    clean = replay(d, dtype, prompts, steps, max_live=live, block_size=block_size)
    spoiled = replay(d, dtype, prompts, steps, max_live=live, block_size=block_size, leftovers=True)
    assert clean.keys() == spoiled.keys()
    for key, row in clean.items():
        assert np.isfinite(spoiled[key]).all(), f"{key}: not finite"
        assert np.array_equal(row, spoiled[key]), f"{key}: differs by {np.abs(row - spoiled[key]).max():.3e}"
    worst, where = ru.worst_error(spoiled, want)
    assert worst <= TOLERANCE[dtype], f"{worst:.3e} at {where}"


def pages_at_the_peak(steps, block_size: int) -> int:
    """The most pages that the live requests of a trace hold at once."""
    held, peak = {}, 0
    for step in steps:
        for e in step["entries"]:
            held[e["id"]] = held.get(e["id"], 0) + len(e["tokens"])
        peak = max(peak, sum(-(-n // block_size) for n in held.values()))
        for name in step["end"]:
            held.pop(name)
    return peak


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name,block_size,seed", [("A", 16, 1), ("B", 8, 2), ("C", 4, 3), ("D", 16, 5)])
def test_a_pool_of_exactly_the_pages_a_trace_needs(setups, name, dtype, block_size, seed):
    """The mixed trace in a pool with not one page to spare: every page that comes back is handed out again
    (the trace allocates more pages than the pool has), and with one page fewer the trace does not fit."""
    from paged_llm_rs_amd.errors import ConfigError

    d, prompts, want = setups(name, dtype)
    steps = ru.mixed(prompts, seed=seed, max_live=4)
    peak = pages_at_the_peak(steps, block_size)
    handed_out = sum(-(-len(t) // block_size) for t in prompts.values())
    assert handed_out > peak, "pages have to be used again"
    got = replay(d, dtype, prompts, steps, max_live=4, block_size=block_size, pages=peak)
    worst, where = ru.worst_error(got, want)
    assert worst <= TOLERANCE[dtype], f"{worst:.3e} at {where}"
    with pytest.raises(ConfigError, match="--max-tokens is too small"):
        replay(d, dtype, prompts, steps, max_live=4, block_size=block_size, pages=peak - 1)


@pytest.mark.parametrize("name,block_size,seed", [("B", 8, 2), ("D", 16, 5), ("E", 16, 6), ("V", 16, 7)])
def test_the_weights_in_strips_change_no_bit(setups, name, block_size, seed, monkeypatch):
    """A model that keeps its matrices a second time in strips (the products of few rows read those) and one
    that does not give bit for bit the same logits, over a mixed schedule and over tails decoded one by one: the
    layout is another order of the same numbers, summed in the same order.  (Large matrices that only go to
    this product when they are there in strips are kept from it here: another product rounds otherwise.)"""
    from paged_llm_rs_amd import kernels
    from paged_llm_rs_amd.engine.replay import Replayer
    from paged_llm_rs_amd.parts.linear import linears_of

    monkeypatch.setattr(kernels, "SKINNY_STRIPS_ROWS", 0)

    d, prompts, _ = setups(name, "bfloat16")
    for steps, live in ((ru.mixed(prompts, seed=seed, max_live=4), 4), (ru.tail_decoded(prompts, 32), 1)):
        got = []
        for strips in (True, False):
            r = Replayer(d, "bfloat16", max_tokens=ru.pool_tokens(prompts, live), block_size=block_size, strips=strips)
            kept = [l.strips is not None for l in linears_of(r.model)]
            assert (any(kept) if strips else not any(kept)) and len(kept) >= 5
            got.append(ru.collect(r, steps))
        assert got[0].keys() == got[1].keys()
        for key in got[0]:
            assert np.array_equal(got[0][key], got[1][key]), f"{key}: the strips change a logit"


def test_schedules_agree_with_each_other_in_32_bit(setups):
    """The logits at a position do not depend on how the tokens were cut, beyond rounding."""
    d, prompts, _ = setups("B", "float32")
    a = replay(d, "float32", prompts, ru.whole(prompts), max_live=1, block_size=8)
    b = replay(d, "float32", prompts, ru.mixed(prompts, seed=9), max_live=4, block_size=8)
    scale = max(float(np.abs(v).max()) for v in a.values())
    worst = max(float(np.abs(a[k] - v).max()) / scale for k, v in b.items())
    assert worst <= 2e-6, f"{worst:.3e}"


def test_trace_run_names_the_line_it_cannot_take(setups, tmp_path):
    """A line that is no step, a token outside the vocabulary and a trace that outgrows --max-tokens each end the
    program with the status 1 and one line that names the input's line; the steps before it are done."""
    d, prompts, _ = setups("A", "float32")
    vocab = TINY_INIT["A"]["config"]["vocab_size"]
    good = {"step": 0, "entries": [{"id": "a", "tokens": [1, 2, 3], "want": [2]}], "end": []}
    for bad, says in [("{\"step\": 1, \"entries\": [", "line 2"), ("[1, 2]", "line 2"),
                      (json.dumps({"step": 1, "entries": [{"id": "a", "tokens": [vocab], "want": []}], "end": []}), "vocabulary"),
                      (json.dumps({"step": 1, "entries": [{"id": "a", "want": []}], "end": []}), "line 2"),
                      (json.dumps({"step": 1, "entries": [{"id": "b", "tokens": [1] * 200, "want": []}], "end": []}), "--max-tokens")]:
        proc = subprocess.run(
            [sys.executable, str(ROOT / "bin" / "trace_run"), "--model", str(d), "--dtype", "float32",
             "--out", str(tmp_path / "out"), "--max-tokens", "128"],
            input=json.dumps(good) + "\n" + bad + "\n", capture_output=True, text=True, timeout=600)
        assert proc.returncode == 1, proc.stderr[-2000:]
        assert proc.stdout.split("\n")[0] == "done 0" and "done 1" not in proc.stdout
        last = proc.stderr.strip().split("\n")[-1]
        assert last.startswith("[trace_run] error") and says in last, last


def test_trace_run_program(setups, tmp_path):
    """The program itself: JSON lines in, <step>.f32 out, a ``done`` line after each step."""
    d, prompts, want = setups("A", "float32")
    steps = ru.mixed(prompts, seed=5)
    proc = subprocess.run(
        [sys.executable, str(ROOT / "bin" / "trace_run"), "--model", str(d), "--dtype", "float32",
         "--out", str(tmp_path / "out"), "--max-tokens", str(ru.pool_tokens(prompts, 4))],
        input="".join(json.dumps(s) + "\n" for s in steps), capture_output=True, text=True, timeout=600)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert proc.stdout.split("\n")[:len(steps)] == [f"done {s['step']}" for s in steps]
    vocab = TINY_INIT["A"]["config"]["vocab_size"]
    fed: dict = {}
    got = {}
    for s in steps:
        wanted = sum(len(e["want"]) for e in s["entries"])
        path = tmp_path / "out" / f"{s['step']}.f32"
        assert path.exists() == (wanted > 0)
        rows = np.fromfile(path, dtype="<f4").reshape(wanted, vocab) if wanted else None
        row = 0
        for e in s["entries"]:
            start = fed.get(e["id"], 0)
            for w in e["want"]:
                got[(e["id"], start + w)] = rows[row]
                row += 1
            fed[e["id"]] = start + len(e["tokens"])
    worst, where = ru.worst_error(got, want)
    assert worst <= TOLERANCE["float32"], f"{worst:.3e} at {where}"


def drawn_configuration(case: int):
    """A configuration, a page size and four prompt lengths drawn from the sizes kernels have to take: heads
    of every multiple of 16, groups of one to sixteen, widths and vocabularies that are no multiple of eight."""
    import random

    rng = random.Random(case)
    d = rng.choice([16, 32, 48, 64, 80, 96, 112, 128, 144, 160, 192, 256])
    nkv = rng.choice([1, 2, 3, 5, 8])
    group = min(rng.choice([1, 2, 3, 4, 7, 8, 16]), max(1, 4096 // (nkv * d)))
    config = {
        "architectures": ["Qwen3ForCausalLM"], "model_type": "qwen3", "hidden_act": "silu", "attention_bias": False,
        "hidden_size": rng.choice([64, 72, 100, 136, 200, 520, 1000, 2056, 2304]),
        "intermediate_size": rng.choice([96, 130, 212, 500, 1030, 2500]),
        "num_hidden_layers": rng.choice([1, 2, 3]), "num_attention_heads": nkv * group, "num_key_value_heads": nkv,
        "head_dim": d, "rms_norm_eps": rng.choice([1e-6, 1e-5, 3e-4]), "rope_theta": rng.choice([10000.0, 1e6]),
        "vocab_size": rng.choice([97, 256, 331, 1001, 5003]), "max_position_embeddings": 4096,
        "tie_word_embeddings": rng.choice([True, False]),
    }
    block_size = rng.choice([1, 2, 4, 8, 16, 32, 64, 128, 24, 3])
    lengths = [rng.randint(1, 40), rng.randint(300, 900) if case % 3 == 0 else rng.randint(30, 140), rng.randint(60, 300),
               rng.randint(2, 90)]
    return config, block_size, lengths


@pytest.mark.parametrize("case", range(12))
def test_drawn_configurations_mixed_and_decoded(tmp_path, case):
    """Sizes that no other test has: every one is served right, in 32-bit and in bfloat16, or refused."""
    from paged_llm_rs_amd.weights import write_random_model

    config, block_size, lengths = drawn_configuration(case)
    prompts = ru.make_prompts(config["vocab_size"], lengths, seed=case)
    for dtype in ("float32", "bfloat16"):
        folder = tmp_path / dtype
        write_random_model(folder, config, seed=case, std=0.05 if config["hidden_size"] <= 200 else 0.02, gain_std=0.1,
                           dtype=dtype)
        want = ru.plain_logits(folder, prompts)
        for steps, live in ((ru.mixed(prompts, seed=case, max_live=4), 4), (ru.tail_decoded(prompts, 32), 1)):
            got = replay(folder, dtype, prompts, steps, max_live=live, block_size=block_size)
            worst, where = ru.worst_error(got, want)
            assert worst <= TOLERANCE[dtype], f"{config} pages of {block_size}, {dtype}: {worst:.3e} at {where}"


# --- the reference's own checkpoint -------------------------------------------------------------------

from conftest import REFERENCE_FIXTURE  # noqa: E402

needs_fixture = pytest.mark.skipif(not (REFERENCE_FIXTURE / "activations.safetensors").exists(),
                                   reason="the reference's fixture is not readable here")


def fixture_metric(got, want) -> float:
    """The reference's own measure (tests/common/mod.rs:20-43): the largest difference over the
    largest wanted magnitude, which counts as one at least."""
    got, want = np.asarray(got, dtype=np.float64), np.asarray(want, dtype=np.float64)
    assert got.size == want.size, f"{got.shape} against {want.shape}"
    return float(np.abs(got.reshape(want.shape) - want).max() / max(1.0, np.abs(want).max()))


@needs_fixture
@pytest.mark.parametrize("cut", ["whole", "one by one", "1, 3, 4"])
def test_the_engine_on_the_references_own_checkpoint(cut):
    """The reference's tiny checkpoint, written by another program (extra keys in config.json, the rotary
    base under rope_parameters, an untied head, a width of 24), read in place through the engine's own
    loader and run in 32-bit: logits and the chosen token at every position against the outputs the
    reference holds, at its own tolerance (tests/forward.rs:53-79); the prompt whole, token by token, and in
    portions of 1, 3 and 4 tokens over pages of 4 (tests/batching.rs:308-312)."""
    from safetensors.torch import load_file

    from paged_llm_rs_amd.engine.replay import Replayer

    manifest = json.loads((REFERENCE_FIXTURE / "manifest.json").read_text())
    held = load_file(str(REFERENCE_FIXTURE / "activations.safetensors"))
    prompt = manifest["prompt"]
    sizes = {"whole": [len(prompt)], "one by one": [1] * len(prompt), "1, 3, 4": [1, 3, 4]}[cut]
    assert sum(sizes) == len(prompt)
    r = Replayer(REFERENCE_FIXTURE, "float32", max_tokens=64, block_size=4)
    rows, at = [], 0
    for n in sizes:
        rows.append(r.step([{"id": "p", "tokens": prompt[at:at + n], "want": list(range(n))}], []))
        at += n
    got = np.concatenate(rows)
    want = held["logits"][0].numpy()
    assert fixture_metric(got, want) <= manifest["relative_tolerance"]
    assert got.argmax(-1).tolist() == want.argmax(-1).tolist()


@needs_fixture
@pytest.mark.parametrize("cut", ["whole", "1, 3, 4"])
def test_every_module_of_the_engine_on_the_references_own_checkpoint(cut):
    """All 36 named activations that the reference holds for its checkpoint (tests/forward.rs:23-51,
    manifest.json), from the engine's 32-bit path with its recorder of named activations on."""
    from safetensors.torch import load_file

    from paged_llm_rs_amd.engine.replay import Replayer

    manifest = json.loads((REFERENCE_FIXTURE / "manifest.json").read_text())
    held = load_file(str(REFERENCE_FIXTURE / "activations.safetensors"))
    prompt = manifest["prompt"]
    sizes = {"whole": [len(prompt)], "1, 3, 4": [1, 3, 4]}[cut]
    r = Replayer(REFERENCE_FIXTURE, "float32", max_tokens=64, block_size=4)
    parts, at = [], 0
    for n in sizes:
        trace: dict = {}
        r.step([{"id": "p", "tokens": prompt[at:at + n], "want": list(range(n))}], [], trace=trace)
        parts.append(trace)
        at += n
    assert len(manifest["tensors"]) == 36 and set(manifest["tensors"]) <= set(parts[0]), sorted(set(manifest["tensors"]) - set(parts[0]))
    for name in manifest["tensors"]:
        got = torch.cat([p[name] for p in parts]).cpu().numpy()
        worst = fixture_metric(got, held[name].numpy())
        assert worst <= manifest["relative_tolerance"], f"{name}: {worst:.3e}"


def test_named_activations_are_refused_in_bfloat16(setups):
    from paged_llm_rs_amd.engine.replay import Replayer
    from paged_llm_rs_amd.errors import UnsupportedError

    d, prompts, _ = setups("A", "bfloat16")
    r = Replayer(d, "bfloat16", max_tokens=64)
    with pytest.raises(UnsupportedError, match="32-bit"):
        r.step([{"id": "p", "tokens": [1, 2, 3], "want": [2]}], [], trace={})


@pytest.mark.parametrize("name,block_size", [("A", 16), ("B", 8), ("C", 4)])
def test_every_module_against_the_plain_implementation(setups, name, block_size):
    """The engine's named activations beside the plain implementation's, module by module (the plain
    implementation is itself held to the reference's 36 recorded tensors): a difference in the logits is
    then found at the module where it begins.  A prompt whole, and a second one in portions beside it."""
    from paged_llm_rs_amd.engine.replay import Replayer

    d, prompts, _ = setups(name, "float32")
    cfg, weights = ru.load_plain(d)
    a, b = prompts["r3"], prompts["r4"]
    want = {}
    for key, tokens in (("a", a), ("b", b)):
        trace: dict = {}
        ru.plain.forward(weights, cfg, tokens, trace=trace)
        want[key] = trace
    r = Replayer(d, "float32", max_tokens=ru.pool_tokens({"a": a, "b": b}, 2), block_size=block_size)
    # step 1: a whole, beside the first 7 tokens of b; step 2: the rest of b
    steps = [[("a", a), ("b", b[:7])], [("b", b[7:])]]
    got = {"a": [], "b": []}
    for step in steps:
        trace = {}
        r.step([{"id": k, "tokens": t, "want": list(range(len(t)))} for k, t in step], [], trace=trace)
        row = 0
        for k, t in step:
            got[k].append({n: v[row:row + len(t)] for n, v in trace.items()})
            row += len(t)
    names = [n for n in want["a"] if n in got["a"][0]]
    assert len(names) == 4 + 16 * cfg["num_hidden_layers"], sorted(set(want["a"]) ^ set(got["a"][0]))
    for key in ("a", "b"):
        for n in names:
            mine = torch.cat([part[n] for part in got[key]]).double().cpu()
            ref = want[key][n].double()
            worst = float((mine.reshape(ref.shape) - ref).abs().max() / max(1.0, float(ref.abs().max())))
            assert worst <= 1e-5, f"request {key}, {n}: {worst:.3e}"


@pytest.mark.parametrize("name,block_size", [("A", 16), ("B", 8), ("C", 4)])
def test_a_recorded_step_computes_what_the_unrecorded_step_computes(setups, name, block_size):
    """Named activations come from an arrangement of the layer in which nothing is fused.  The same mixed
    steps with the recorder on and off, on caches that start equal: the logits agree to rounding (the
    fused kernels add in another order) and the pages hold the same keys and values afterwards."""
    from paged_llm_rs_amd.engine.replay import Replayer

    d, prompts, _ = setups(name, "float32")
    a, b, c = prompts["r3"], prompts["r4"], prompts["r2"]
    steps = [[("a", a[:-3]), ("b", b[:5])], [("a", a[-3:-2]), ("b", b[5:]), ("c", c)], [("a", a[-2:-1])], [("a", a[-1:])]]
    runs = []
    for recorded in (False, True):
        r = Replayer(d, "float32", max_tokens=ru.pool_tokens({"a": a, "b": b, "c": c}, 3), block_size=block_size)
        logits = []
        for step in steps:
            entries = [{"id": k, "tokens": t, "want": list(range(len(t)))} for k, t in step]
            logits.append(r.step(entries, [], trace={} if recorded else None))
        pools = [pool.clone() for layer in range(len(r.model.blocks)) for pool in r.cache.layer_pools(layer)]
        tables = [r.cache.manager.table(r.ids[k], 0) for k in "abc"]
        runs.append((logits, pools, tables))
    (plain_logits, plain_pools, plain_tables), (traced_logits, traced_pools, traced_tables) = runs
    assert plain_tables == traced_tables
    for got, want in zip(traced_logits, plain_logits):
        assert got.shape == want.shape
        assert np.abs(got - want).max() <= 1e-6 * max(1.0, np.abs(want).max())
    rows = sorted({page * block_size + i for table in plain_tables for page in table if page >= 0 for i in range(block_size)})
    for got, want in zip(traced_pools, plain_pools):
        # the keys and values of the first layer are bit for bit the same; later layers see the stream after
        # sums in another order
        assert torch.allclose(got[rows], want[rows], rtol=0, atol=2e-6 * float(want[rows].abs().max()))
    assert torch.equal(traced_pools[0][rows], plain_pools[0][rows]) and torch.equal(traced_pools[1][rows], plain_pools[1][rows])


def test_head_sizes_that_are_no_multiple_of_16_run_in_32_bit(tmp_path):
    """config.json may give any head size; the 32-bit path takes every one up to 256, the bfloat16 kernels
    work in units of 16 and say so."""
    from paged_llm_rs_amd.engine.replay import Replayer
    from paged_llm_rs_amd.errors import UnsupportedError
    from paged_llm_rs_amd.weights import write_random_model

    config = dict(TINY_INIT["A"]["config"], hidden_size=60, num_attention_heads=3, num_key_value_heads=1, head_dim=20,
                  intermediate_size=100, vocab_size=131, tie_word_embeddings=False)
    prompts = ru.make_prompts(config["vocab_size"], [40, 7, 23, 61], seed=2)
    folder = write_random_model(tmp_path / "f32", config, seed=8, std=0.05, gain_std=0.2, dtype="float32")
    want = ru.plain_logits(folder, prompts)
    for steps, live in ((ru.whole(prompts), 1), (ru.mixed(prompts, seed=3, max_live=4), 4), (ru.tail_decoded(prompts, 16), 1)):
        got = replay(folder, "float32", prompts, steps, max_live=live, block_size=4)
        worst, where = ru.worst_error(got, want)
        assert worst <= TOLERANCE["float32"], f"{worst:.3e} at {where}"
    half = write_random_model(tmp_path / "bf16", config, seed=8, std=0.05, gain_std=0.2, dtype="bfloat16")
    with pytest.raises(UnsupportedError, match="multiples of 16"):
        Replayer(half, "bfloat16", max_tokens=64)
