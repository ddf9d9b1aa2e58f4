"""Building traces for replay tests and comparing what comes back with the
plain implementation."""

from __future__ import annotations

import random

import numpy as np
import torch

import plain_qwen3 as plain
from conftest import load_plain


def make_prompts(vocab: int, lengths, seed: int) -> dict:
    rng = random.Random(seed)
    return {f"r{i}": [rng.randrange(vocab) for _ in range(n)] for i, n in enumerate(lengths)}


def plain_logits(model_dir, prompts: dict, device="cpu") -> dict:
    """name -> float64 logits [len, vocab] of the whole sequence, no cache."""
    cfg, weights = load_plain(model_dir)
    return {name: plain.forward(weights, cfg, toks, device=device) for name, toks in prompts.items()}


# --- schedules: lists of steps {"step", "entries", "end"} ------------------------------------

def whole(prompts: dict, want_all: bool = True) -> list:
    """Each request alone and whole, one step each."""
    steps = []
    for i, (name, toks) in enumerate(prompts.items()):
        want = list(range(len(toks))) if want_all else [len(toks) - 1]
        steps.append({"step": i, "entries": [{"id": name, "tokens": toks, "want": want}], "end": [name]})
    return steps


def tail_decoded(prompts: dict, tail: int = 32) -> list:
    """Most of each request in one step, the last ``tail`` tokens one by one."""
    steps = []
    for name, toks in prompts.items():
        head = max(len(toks) - tail, 1)
        steps.append({"step": len(steps), "entries": [{"id": name, "tokens": toks[:head], "want": [head - 1]}], "end": []})
        for p in range(head, len(toks)):
            steps.append({"step": len(steps), "entries": [{"id": name, "tokens": [toks[p]], "want": [0]}],
                          "end": [name] if p == len(toks) - 1 else []})
        if head == len(toks):
            steps[-1]["end"] = [name]
    return steps


def portions(prompts: dict, sizes=(2, 7, 3, 16, 5, 2, 33, 4, 9)) -> list:
    """Each request in portions of changing size, down to two tokens."""
    steps = []
    for name, toks in prompts.items():
        at, k = 0, 0
        while at < len(toks):
            n = min(sizes[k % len(sizes)], len(toks) - at)
            k += 1
            want = sorted({0, n - 1})
            steps.append({"step": len(steps), "entries": [{"id": name, "tokens": toks[at:at + n], "want": want}],
                          "end": [name] if at + n == len(toks) else []})
            at += n
    return steps


def mixed(prompts: dict, seed: int, max_live: int = 4, tail: int = 12) -> list:
    """Up to ``max_live`` live requests: portions of some beside decoded tokens of
    others, requests skipped now and then; a request that ends makes room for the
    next, so pages are used again."""
    rng = random.Random(seed)
    waiting = list(prompts.items())
    live: dict = {}
    steps = []
    while waiting or live:
        while waiting and len(live) < max_live and (not live or rng.random() < 0.6):
            name, toks = waiting.pop(0)
            live[name] = [toks, 0]
        entries, end = [], []
        for name, (toks, at) in list(live.items()):
            if len(live) > 1 and rng.random() < 0.2:
                continue    # left out of this step, goes on later
            left = len(toks) - at
            if left > tail:
                n = min(rng.choice([2, 3, 5, 8, 13, 21]), left - tail) if left - tail >= 2 else left - tail
                n = max(n, 1)
                want = sorted(set(rng.sample(range(n), min(n, 2))) | {n - 1})
            else:
                n, want = 1, [0]
            entries.append({"id": name, "tokens": toks[at:at + n], "want": want})
            live[name][1] = at + n
            if at + n == len(toks):
                end.append(name)
                del live[name]
        if entries:
            steps.append({"step": len(steps), "entries": entries, "end": end})
    return steps


def pool_tokens(prompts: dict, max_live: int) -> int:
    """--max-tokens for a trace: the largest requests that can be live together,
    each rounded up to a multiple of 64."""
    sizes = sorted(((len(t) + 63) // 64 * 64 for t in prompts.values()), reverse=True)
    return sum(sizes[:max_live])


# --- running and comparing ----------------------------------------------------------------------

def collect(replayer, steps) -> dict:
    """(name, position) -> logits row, from running the steps through a Replayer."""
    fed: dict = {}
    got: dict = {}
    for step in steps:
        out = replayer.step(step["entries"], step["end"])
        row = 0
        for e in step["entries"]:
            start = fed.get(e["id"], 0)
            for w in e["want"]:
                got[(e["id"], start + w)] = out[row]
                row += 1
            fed[e["id"]] = start + len(e["tokens"])
        assert (out is None and row == 0) or out.shape[0] == row
        for name in step["end"]:
            fed.pop(name, None)
    return got


def worst_error(got: dict, want: dict):
    """Largest |got - want| over every compared row, relative to the largest |want| of the trace."""
    scale = max(float(want[n][p].abs().max()) for (n, p) in got)
    worst, where = 0.0, None
    for (n, p), row in got.items():
        ref = want[n][p].numpy()
        assert row.shape == ref.shape, f"shape {row.shape} against {ref.shape}"
        err = float(np.abs(row.astype(np.float64) - ref).max()) / scale
        if err > worst:
            worst, where = err, (n, p)
    return worst, where
