#!/usr/bin/env python3
"""The headline measurement: Qwen3-0.6B-shape decoding and prefill on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--shape 0.6b|8b|32b]

A step is one decode step of the engine's own step function on a batch of
requests, each with a context of 512 tokens at the start (2,048 and 4,096 for
the larger shapes): the cache write, the
attention over the pages, every projection, the output projection and the greedy
choice of the next token, which is what the next step is fed.  Weights are random
(the random-weights mode writes the model folder, the loader reads it back),
prompts are seeded uniform token ids.  One JSON line is printed.

The default sizes are the Qwen3-0.6B shape's.  Peaks are the published ones of the
MI355X: 8 TB/s of HBM, 2.5 PFLOP/s dense bf16.
"""

from __future__ import annotations

import argparse
import json
import math
import os
import random
import sys
import tempfile
import time
from pathlib import Path

ROOT = Path(__file__).resolve().parent
sys.path.insert(0, str(ROOT))

HBM_PEAK = 8.0e12            # bytes a second
MFMA_PEAK = {"bf16": 2.5e15, "fp16": 2.5e15, "fp8": 5.0e15, "fp32": 157.3e12}

COMMON = {
    "architectures": ["Qwen3ForCausalLM"], "model_type": "qwen3", "hidden_act": "silu",
    "attention_bias": False, "sliding_window": None, "head_dim": 128, "num_key_value_heads": 8,
    "rms_norm_eps": 1e-6, "rope_theta": 1000000.0, "vocab_size": 151936,
}
# The default is the Qwen3-0.6B shape; --shape 8b and 32b are the Qwen3-8B and Qwen3-32B shapes:
# (config.json keys, the context a decode step starts from, layers that the default run of that shape loads).
SHAPES = {
    "0.6b": ("Qwen3-0.6B", dict(COMMON, hidden_size=1024, intermediate_size=3072, num_hidden_layers=28,
                                num_attention_heads=16, max_position_embeddings=4096, tie_word_embeddings=True),
             512, 28),
    "8b": ("Qwen3-8B", dict(COMMON, hidden_size=4096, intermediate_size=12288, num_hidden_layers=36,
                            num_attention_heads=32, max_position_embeddings=8192, tie_word_embeddings=False),
           2048, 36),
    "32b": ("Qwen3-32B", dict(COMMON, hidden_size=5120, intermediate_size=25600, num_hidden_layers=64,
                              num_attention_heads=64, max_position_embeddings=16384, tie_word_embeddings=False),
            4096, 16),
}
PREFILL_TOKENS = 2048
BLOCK_SIZE = 16
LONG_CONTEXT = 3968          # a point of the default line: decode from contexts near the 0.6B shape's 4,096 positions
MIXED_SLICE = 512            # --only mixed: a slice of a prompt this long beside 63 decoded tokens
MIXED_DECODES = 63
# Layers of the two larger shapes in the default run's extra points (of 36 and 64).
OTHER_SHAPE_LAYERS = {"8b": 6, "32b": 4}


def say(message: str) -> None:
    print(f"[bench] {message}", file=sys.stderr, flush=True)


def model_bytes_and_flops(cfg: dict, element: int):
    """(bytes of weights a decode step reads once, matrix flops a token costs)."""
    H, I, L = cfg["hidden_size"], cfg["intermediate_size"], cfg["num_hidden_layers"]
    q = cfg["num_attention_heads"] * cfg["head_dim"]
    kv = cfg["num_key_value_heads"] * cfg["head_dim"]
    per_layer = H * (q + 2 * kv) + q * H + 2 * H * I + I * H
    norms = L * (2 * H + 2 * cfg["head_dim"]) + H
    head = cfg["vocab_size"] * H
    params = L * per_layer + head
    return (params + norms) * element, 2 * L * per_layer, 2 * head


def kv_bytes_per_token(cfg: dict, element: int) -> int:
    return 2 * cfg["num_hidden_layers"] * cfg["num_key_value_heads"] * cfg["head_dim"] * element


class DecodeBench:
    """B requests with ``context`` tokens each in the cache, then timed decode steps."""

    def __init__(self, model, cache, runner, batch: int, context: int, seed: int, ahead: bool = True):
        from paged_llm_rs_amd.engine.batch import CannotFeed, StepEntry

        self.model, self.cache, self.batch = model, cache, batch
        self.StepEntry, self.CannotFeed = StepEntry, CannotFeed
        self.ahead, self.flight = ahead, None
        rng = random.Random(seed)
        vocab = model.spec.vocab_size
        self.ids = list(range(1, batch + 1))
        self.next_tokens = None
        from paged_llm_rs_amd.engine.step import commit_step, run_step
        from paged_llm_rs_amd import kernels
        self.run_step, self.commit_step, self.kernels = run_step, commit_step, kernels
        self.runner = runner
        firsts = []
        for i in self.ids:
            cache.manager.add_sequence(i)
            prompt = [rng.randrange(vocab) for _ in range(context)]
            assert cache.manager.reserve(i, context)
            entry = [StepEntry(i, prompt, 0, [context - 1])]
            logits = run_step(model, cache, entry)
            commit_step(cache, entry)
            firsts.append(int(kernels.argmax(logits).item()))
        self.tokens = firsts

    def step(self) -> None:
        """Queue one decode step behind the one in flight, fed that step's tokens on the device, then read
        the tokens of the step in flight: what the engine does while nothing but greedy decoding goes on
        (``Engine._launch_ahead``).  Every step's tokens reach the host, one step late."""
        manager = self.cache.manager
        for i in self.ids:
            assert manager.reserve(i, 1)
        out = None
        if self.ahead and self.flight is not None:
            entries = [self.StepEntry(i, [0], manager.tokens(i), [0], fed_row=row) for row, i in enumerate(self.ids)]
            try:
                out = self.runner.run(entries)
            except self.CannotFeed:
                pass
        if self.flight is not None:
            self.tokens = self.flight.greedy_on_host()
            self.flight = None
        if out is None:
            entries = [self.StepEntry(i, [tok], manager.tokens(i), [0]) for i, tok in zip(self.ids, self.tokens)]
            out = self.runner.run(entries)
        self.commit_step(self.cache, entries)      # queued: written, for every step behind it
        self.flight = out

    def free(self) -> None:
        if self.flight is not None:
            self.tokens, self.flight = self.flight.greedy_on_host(), None
        for i in self.ids:
            self.cache.manager.free_sequence(i)


def timed(fn, steps: int, warmup: int) -> float:
    import torch

    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    start = time.perf_counter()
    for _ in range(steps):
        fn()
    torch.cuda.synchronize()
    return (time.perf_counter() - start) / steps


class Workbench:
    """A random model of one of the shapes with some of its layers, its cache and a step runner, and the
    measurements that are taken on it."""

    def __init__(self, shape: str, layers: int, device, largest_batch: int, steps: int, graphs: bool = True,
                 context: int | None = None, prefill_room: bool = True, most_tokens: int = 0):
        import torch

        from paged_llm_rs_amd import write_random_model
        from paged_llm_rs_amd.cache import PagedCache
        from paged_llm_rs_amd.engine.step import StepRunner
        from paged_llm_rs_amd.parts.model import load_model

        self.model_name, config, self.context, _ = SHAPES[shape]
        if context is not None:
            self.context = context
        self.full_layers = config["num_hidden_layers"]
        self.layers = layers
        self.cfg = dict(config)
        self.cfg["num_hidden_layers"] = layers
        self.tmp = tempfile.TemporaryDirectory()
        say(f"writing a random {layers}-layer model folder of the {self.model_name} shape")
        t0 = time.time()
        self.folder = write_random_model(Path(self.tmp.name) / "model", self.cfg, seed=0, std=0.02, gain_std=0.1,
                                         dtype="bfloat16")
        say(f"written in {time.time() - t0:.0f} s; loading")
        self.config, self.model = load_model(self.folder, "bfloat16", device)
        say("loaded")
        self.weight_bytes, self.layer_flops, self.head_flops = model_bytes_and_flops(self.cfg, 2)
        self.kv_token = kv_bytes_per_token(self.cfg, 2)
        # (most_tokens: what the largest of the points keeps in the cache at once, where that is more)
        tokens = max(largest_batch * (self.context + steps + 64), most_tokens)
        pages = (tokens + (PREFILL_TOKENS + 64 if prefill_room else 0)) // BLOCK_SIZE + largest_batch
        self.cache = PagedCache(self.model.cache_layout, BLOCK_SIZE, pages, torch.bfloat16, device, max_seqs=largest_batch + 1)
        self.runner = StepRunner(self.model, self.cache, graphs=graphs)

    def close(self) -> None:
        import gc

        import torch

        self.runner = self.cache = self.model = None
        self.tmp.cleanup()
        gc.collect()
        torch.cuda.empty_cache()

    def decode_point(self, batch: int, steps: int, warmup: int, context: int | None = None):
        """(seconds a step, tokens a second, bytes a step has to read) of decode steps at ``batch``, from
        contexts of ``context`` tokens (the shape's own where not given)."""
        context = self.context if context is None else context
        bench = DecodeBench(self.model, self.cache, self.runner, batch, context, seed=batch)
        seconds = timed(bench.step, steps, warmup)
        context_mid = context + warmup + steps / 2
        bench.free()
        return seconds, batch / seconds, self.weight_bytes + batch * context_mid * self.kv_token

    def prefill_point(self, eager: bool = False, tokens: int = PREFILL_TOKENS):
        from paged_llm_rs_amd.engine.batch import StepEntry
        from paged_llm_rs_amd.engine.step import run_step

        say(f"prefill, {tokens} tokens")
        rng = random.Random(2048)
        prompt = [rng.randrange(self.cfg["vocab_size"]) for _ in range(tokens)]
        cache, model, runner = self.cache, self.model, self.runner

        def prefill():
            cache.manager.add_sequence(1000)
            assert cache.manager.reserve(1000, tokens)
            entry = [StepEntry(1000, prompt, 0, [tokens - 1])]
            if eager:
                run_step(model, cache, entry)
            else:
                runner.run(entry)        # as the engine runs it: a shape of step that comes again is replayed from a graph
            cache.manager.free_sequence(1000)

        seconds_prefill = timed(prefill, 10, 5)
        d, nq = self.cfg["head_dim"], self.cfg["num_attention_heads"]
        attention_flops = self.layers * 4 * nq * d * (tokens * (tokens + 1) // 2)
        flops = self.layer_flops * tokens + self.head_flops + attention_flops
        return {"value": round(tokens / seconds_prefill, 1), "tokens": tokens,
                "ms": round(seconds_prefill * 1e3, 3),
                "frac": round(flops / seconds_prefill / MFMA_PEAK["bf16"], 4)}

    def mixed_point(self, steps: int, warmup: int):
        """One step of the third slice of a prompt beside 63 requests that bring one token each.  The step is
        not committed, so every run of it writes the same places of the cache again."""
        from paged_llm_rs_amd.engine.batch import StepEntry
        from paged_llm_rs_amd.engine.step import commit_step, run_step

        cache, model, runner, cfg, context = self.cache, self.model, self.runner, self.cfg, self.context
        say(f"mixed step: {MIXED_DECODES} decoded tokens at context {context} beside a slice of {MIXED_SLICE}")
        bench = DecodeBench(model, cache, runner, MIXED_DECODES, context, seed=3)
        rng = random.Random(512)
        long_prompt = [rng.randrange(cfg["vocab_size"]) for _ in range(PREFILL_TOKENS)]
        behind = 2 * MIXED_SLICE
        cache.manager.add_sequence(1000)
        assert cache.manager.reserve(1000, behind)
        first = [StepEntry(1000, long_prompt[:behind], 0, [])]
        run_step(model, cache, first)
        commit_step(cache, first)
        assert cache.manager.reserve(1000, MIXED_SLICE)
        entries = [StepEntry(1000, long_prompt[behind:behind + MIXED_SLICE], behind, [])]
        for i, tok in zip(bench.ids, bench.tokens):
            assert cache.manager.reserve(i, 1)
            entries.append(StepEntry(i, [tok], cache.manager.tokens(i), [0]))
        seconds = timed(lambda: runner.run(entries).greedy_tokens(), steps, warmup)
        cache.manager.free_sequence(1000)
        bench.free()
        rows = MIXED_SLICE + MIXED_DECODES
        d, nq = cfg["head_dim"], cfg["num_attention_heads"]
        attention_flops = self.layers * 4 * nq * d * (MIXED_SLICE * (behind + (MIXED_SLICE + 1) // 2) + MIXED_DECODES * context)
        flops = self.layer_flops * rows + self.head_flops * MIXED_DECODES + attention_flops
        step_bytes = self.weight_bytes + (MIXED_DECODES * context + behind + MIXED_SLICE) * self.kv_token
        return {
            "model": f"{self.model_name} shape", "layers": self.layers, "layers_full": self.full_layers, "rows": rows,
            "decode_context": context, "ms": round(seconds * 1e3, 3), "tokens_per_s": round(rows / seconds, 1),
            "hbm_floor_ms": round(step_bytes / HBM_PEAK * 1e3, 3), "mfma_floor_ms": round(flops / MFMA_PEAK["bf16"] * 1e3, 3),
            "frac_hbm": round(step_bytes / seconds / HBM_PEAK, 4), "frac_mfma": round(flops / seconds / MFMA_PEAK["bf16"], 4),
        }


def products_table(torch) -> int:
    """Microseconds of y = x . w^T over large weight matrices that come from memory (several copies of each
    matrix in turn, inside one captured graph), by the library, the skinny and the streamed product, and
    which of them `Linear` takes.  One JSON line."""
    from paged_llm_rs_amd import kernels
    from paged_llm_rs_amd.engine.step import require_gpu

    device = require_gpu("cuda:0")

    def microseconds(calls):
        for call in calls[:2]:
            call()
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            for call in calls:
                call()
        graph.replay()
        torch.cuda.synchronize()
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        graph.replay()
        graph.replay()
        stop.record()
        torch.cuda.synchronize()
        return start.elapsed_time(stop) / len(calls) / 2 * 1e3

    shapes = [("32b_qkv", 10240, 5120), ("32b_o", 5120, 8192), ("32b_gate_up", 51200, 5120), ("32b_down", 5120, 25600),
              ("8b_qkv", 6144, 4096), ("8b_o", 4096, 4096), ("8b_gate_up", 24576, 4096), ("8b_down", 4096, 12288)]
    table = {}
    for name, columns, width in shapes:
        copies = max(2, min(24, int(1.5e9 // (columns * width * 2))))
        weights = [(torch.randn(columns, width, device=device) / math.sqrt(width)).bfloat16() for _ in range(copies)]
        strips = [kernels.weights_in_strips(w) for w in weights]
        for rows in (8, 16, 32, 64):
            x = torch.randn(rows, width, device=device).bfloat16()
            entry = {"MB": round(columns * width * 2 / 1e6),
                     "library_us": round(microseconds([lambda w=w: torch.mm(x, w.t()) for w in weights]), 1),
                     "stream_us": round(microseconds([lambda w=w: kernels.gemm_stream(x, w) for w in weights]), 1),
                     "skinny_us": round(microseconds([lambda w=w: kernels.gemm_skinny(x, w) for w in weights]), 1),
                     "skinny_strips_us": (round(microseconds([lambda w=w, s=s: kernels.gemm_skinny(x, w, strips=s)
                                                              for w, s in zip(weights, strips)]), 1)
                                          if kernels.strips_apply(rows, columns, width) else None),
                     "taken": "stream" if kernels.stream_wins(rows, columns, width) else
                              ("skinny" if kernels.skinny_wins(rows, columns, width) else "library")}
            table[f"{name}_rows{rows}"] = entry
            print(f"[bench] {name} {rows} rows: {entry}", file=sys.stderr, flush=True)
        del weights, strips
    print(json.dumps({"metric": "products of few rows over large weights, microseconds", "unit": "us", "dtype": "bf16",
                      "data": "synthetic: random weights from memory", "products": table}))
    return 0


def main() -> int:
    parser = argparse.ArgumentParser()
    parser.add_argument("--gpus", type=int, default=1)
    parser.add_argument("--steps", type=int, default=50)
    parser.add_argument("--warmup", type=int, default=10)
    parser.add_argument("--batch", type=int, default=8)
    parser.add_argument("--shape", choices=sorted(SHAPES), default="0.6b",
                        help="layer sizes: the headline 0.6b, or the 8b and 32b shapes")
    parser.add_argument("--layers", type=int, default=None,
                        help="fewer layers than the model has, where memory or time needs it; both numbers are reported")
    parser.add_argument("--no-graphs", action="store_true", help="run decode steps eagerly instead of as HIP graphs")
    parser.add_argument("--skip-points", action="store_true", help="leave out batch 1 and 64 and the prefill")
    parser.add_argument("--no-other-shapes", action="store_true",
                        help="leave out the points of the 8b shape (a mixed step) and the 32b shape (decode at batch 64)")
    parser.add_argument("--prefill-eager", action="store_true",
                        help="launch the prefill step kernel by kernel every time (a prompt length seen once)")
    parser.add_argument("--ahead", choices=["on", "off"], default="on",
                        help="--only engine: whether the engine queues a decoding step before it has read the tokens "
                             "of the one before")
    parser.add_argument("--only", choices=["decode", "prefill", "engine", "mixed", "serving", "products"], default=None,
                        help="run one part alone: the decode steps at --batch, the prefill, or (not part of the "
                             "default line) the whole engine on 1/4/16/32/64/128 requests at once, 16 prompt tokens and "
                             "128 generated each, as the reference's own table of clients does; mixed: one step of a "
                             "512-token slice of a prompt beside 63 decoded tokens; serving: the reference's two other "
                             "tables, first tokens behind a shared preamble with the prefix cache off and on, and the "
                             "gaps between the tokens of four running requests when a long prompt arrives, by --chunk; "
                             "products: the layer products of the 8B and 32B shapes at 8 to 64 rows, weights from memory, "
                             "by the library and by the two hand-written products of few rows")
    args = parser.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py measures one GPU; this engine has no multi-GPU path (N must be 1)")
        return 2

    import torch

    if args.only == "products":
        return products_table(torch)

    from paged_llm_rs_amd.engine.batch import StepEntry
    from paged_llm_rs_amd.engine.step import commit_step, require_gpu, run_step

    device = require_gpu("cuda:0")
    model_name, CONFIG, CONTEXT, default_layers = SHAPES[args.shape]
    FULL_LAYERS = CONFIG["num_hidden_layers"]
    if args.layers is None:
        args.layers = default_layers
    long_points = args.shape == "0.6b" and not args.skip_points and args.only is None
    bench = Workbench(args.shape, args.layers, device, largest_batch=max(64, args.batch),
                      steps=args.steps + args.warmup, graphs=not args.no_graphs,
                      most_tokens=max(64, args.batch) * (LONG_CONTEXT + 128) if long_points else 0)
    cfg, model, cache, runner, folder, tmp = bench.cfg, bench.model, bench.cache, bench.runner, bench.folder, bench.tmp
    weight_bytes, layer_flops, head_flops, kv_token = bench.weight_bytes, bench.layer_flops, bench.head_flops, bench.kv_token
    decode_point = bench.decode_point

    def prefill_point():
        return bench.prefill_point(eager=args.prefill_eager)

    if args.only == "prefill":
        print(json.dumps({"prefill": prefill_point()}), flush=True)
        tmp.cleanup()
        return 0
    if args.only == "mixed":
        print(json.dumps({"mixed": bench.mixed_point(args.steps, args.warmup)}), flush=True)
        tmp.cleanup()
        return 0
    if args.only == "serving":
        from paged_llm_rs_amd.engine.engine import Engine

        del runner, cache
        vocab = cfg["vocab_size"]

        def drive(engine, arrivals):
            """Submit the (step, prompt, max_tokens) arrivals when their step comes, run to the end; per request
            the times of its tokens, counted from its arrival."""
            pending = sorted(arrivals, key=lambda a: a[0])
            arrived, stamps, step = {}, {}, 0
            while pending or engine.open_requests:
                while pending and pending[0][0] <= step:
                    _, prompt, budget = pending.pop(0)
                    arrived[engine.submit(prompt, max_tokens=budget, temperature=0.0, stop_tokens=[])] = time.perf_counter()
                outcome = engine.step()
                step += 1
                if outcome is None:
                    continue
                now = time.perf_counter()
                for seq_id, _ in outcome.tokens:
                    stamps.setdefault(seq_id, []).append(now - arrived[seq_id])
            for seq_id in stamps:
                engine.take_result(seq_id)
            return [stamps[k] for k in sorted(stamps)]

        def percentile(values, q):
            ordered = sorted(values)
            return ordered[min(len(ordered) - 1, int(q * len(ordered)))]

        result = {"prefix_cache": {}, "chunk": {}}
        rng = random.Random(11)
        preamble = [rng.randrange(vocab) for _ in range(384)]
        shared = [preamble + [rng.randrange(vocab) for _ in range(16)] for _ in range(16)]
        apart = [[rng.randrange(vocab) for _ in range(400)] for _ in range(16)]
        for workload, prompts in (("one shared preamble", shared), ("nothing in common", apart)):
            for cache_on in (False, True):
                engine = Engine(folder, dtype="bf16", block_size=BLOCK_SIZE, num_blocks=2048, max_batch=16, chunk=128,
                                prefix_cache=cache_on)
                for run, timed_run in enumerate((False, False, True)):   # shapes of step are captured when they come again
                    # other tokens every run: what an earlier run left in the cache must not make this one a hit
                    prompts_run = [[(t + 7 * run) % vocab for t in p] for p in prompts]
                    before = engine.metrics().get("cached_tokens", 0)
                    torch.cuda.synchronize()
                    start = time.perf_counter()
                    times = drive(engine, [(0, p, 64) for p in prompts_run])
                    seconds = time.perf_counter() - start
                firsts = [t[0] for t in times]
                result["prefix_cache"][f"{workload}, cache {'on' if cache_on else 'off'}"] = {
                    "ttft_ms": round(sum(firsts) / len(firsts) * 1e3, 2), "p95_ttft_ms": round(percentile(firsts, 0.95) * 1e3, 2),
                    "tokens_per_s": round(sum(len(t) for t in times) / seconds, 1),
                    "cached_tokens": engine.metrics().get("cached_tokens", 0) - before}
                say(f"prefix cache, {workload}, {'on' if cache_on else 'off'}: {result['prefix_cache'][f'{workload}, cache ' + ('on' if cache_on else 'off')]}")
                del engine
        long_prompt = [rng.randrange(vocab) for _ in range(1100)]
        residents = [[rng.randrange(vocab) for _ in range(12)] for _ in range(4)]
        for chunk in ("off", 512, 128, 64, 32):
            engine = Engine(folder, dtype="bf16", block_size=BLOCK_SIZE, num_blocks=1024, max_batch=16, chunk=chunk,
                            prefix_cache=False)
            for timed_run in (False, False, True):
                times = drive(engine, [(0, p, 160) for p in residents] + [(40, long_prompt, 16)])
            gaps = [b - a for t in times[:4] for a, b in zip(t, t[1:])]
            result["chunk"][str(chunk)] = {
                "median_gap_ms": round(percentile(gaps, 0.5) * 1e3, 3), "worst_gap_ms": round(max(gaps) * 1e3, 3),
                "newcomer_first_token_ms": round(times[4][0] * 1e3, 2)}
            say(f"chunk {chunk}: {result['chunk'][str(chunk)]}")
            del engine
        print(json.dumps({"serving": result}), flush=True)
        tmp.cleanup()
        return 0
    if args.only == "engine":
        # scheduler, cache manager, step function, sampling and the read-back of every token: generate()
        from paged_llm_rs_amd.engine.engine import Engine

        del runner, cache
        engine = Engine(folder, dtype="bf16", block_size=BLOCK_SIZE, num_blocks=64 * 12 + 64, max_batch=64, chunk=128,
                        ahead=args.ahead == "on")
        rng = random.Random(7)
        result = {}
        # (128 requests are more than the engine has rows and pages for at once: some wait in the queue)
        for clients in (1, 4, 16, 32, 64, 128):
            prompts = [[rng.randrange(cfg["vocab_size"]) for _ in range(16)] for _ in range(clients)]
            for timed_run in (False, False, True):      # a shape of step is captured when it comes the second time
                torch.cuda.synchronize()
                start = time.perf_counter()
                out = engine.generate(prompts, max_tokens=128, temperature=0.0, stop_tokens=[])
                seconds = time.perf_counter() - start
            made = sum(len(o["tokens"]) for o in out)
            result[f"clients_{clients}"] = {"tokens_per_s": round(made / seconds, 1), "seconds": round(seconds, 3)}
            say(f"engine, {clients} requests: {made / seconds:.0f} tokens/s")
        print(json.dumps({"engine": result}), flush=True)
        tmp.cleanup()
        return 0

    say(f"decode, batch {args.batch}")
    seconds, value, step_bytes = decode_point(args.batch, args.steps, args.warmup)
    line = {
        "metric": f"{model_name} bf16: decode tok/s @ batch {args.batch}, ctx {CONTEXT}",
        "value": round(value, 1), "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(seconds * 1e3, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "bf16", "data": "synthetic: random weights, uniform random token ids",
        "config": {
            "model": f"{model_name} shape", "global_batch": args.batch, "seq_len": CONTEXT, "parallelism": "none",
            "layers": args.layers, "layers_full": FULL_LAYERS, "hidden": cfg["hidden_size"],
            "q_heads": cfg["num_attention_heads"], "kv_heads": cfg["num_key_value_heads"],
            "head_dim": cfg["head_dim"], "intermediate": cfg["intermediate_size"], "vocab": cfg["vocab_size"],
            "tied": cfg["tie_word_embeddings"], "block_size": BLOCK_SIZE, "max_context": cfg["max_position_embeddings"],
            "prefill_tokens": PREFILL_TOKENS,
        },
        "roofline": {"bound": "hbm", "achieved": round(step_bytes / seconds / 1e9, 1), "peak": HBM_PEAK / 1e9,
                     "unit": "GB/s", "frac": round(step_bytes / seconds / HBM_PEAK, 4)},
    }

    if not args.skip_points and args.only is None:
        points = {}
        for batch in (1, 64):
            say(f"decode, batch {batch}")
            s, v, _ = decode_point(batch, max(args.steps // 2, 5), max(args.warmup // 2, 2))
            points[f"decode_b{batch}"] = round(v, 1)
        if args.shape == "0.6b":
            # the same batch as the headline from contexts eight times as long: the step is the attention's then
            say(f"decode, batch {args.batch}, context {LONG_CONTEXT}")
            s_long, v_long, bytes_long = decode_point(args.batch, 20, 5, context=LONG_CONTEXT)
            points[f"decode_b{args.batch}_ctx{LONG_CONTEXT}"] = round(v_long, 1)
            points[f"decode_b{args.batch}_ctx{LONG_CONTEXT}_frac_hbm"] = round(bytes_long / s_long / HBM_PEAK, 4)
            say(f"decode, batch 64, context {LONG_CONTEXT}")
            s_long, v_long, bytes_long = decode_point(64, 12, 4, context=LONG_CONTEXT)
            points[f"decode_b64_ctx{LONG_CONTEXT}"] = round(v_long, 1)
            points[f"decode_b64_ctx{LONG_CONTEXT}_frac_hbm"] = round(bytes_long / s_long / HBM_PEAK, 4)
        line["points"] = points
        line["prefill"] = prefill_point()
        if args.shape == "0.6b" and not args.no_other_shapes:
            # The two larger shapes, with fewer layers than they have (both numbers are in ``config``): the time
            # of a layer is what their fractions of the peaks need, and the whole run stays a few minutes.
            bench.close()
            other = Workbench("8b", OTHER_SHAPE_LAYERS["8b"], device, largest_batch=MIXED_DECODES + 1, steps=8)
            mixed = other.mixed_point(30, 10)       # (ten untimed steps: the chip has idled while the model was made)
            # The times of these points are of steps over a few layers (and the whole projection onto the
            # vocabulary); they are no model's rate.  What carries over to the whole model is the share of
            # the peak that binds: for this step the memory (63 contexts of keys and values beside the
            # weights outweigh the 575 rows of arithmetic), for the decode steps the memory as well.
            points["mixed_8b_ms"] = mixed["ms"]
            points["mixed_8b_frac_hbm"] = mixed["frac_hbm"]
            points["mixed_8b_frac_mfma"] = mixed["frac_mfma"]
            points["mixed_8b_bound"] = "hbm" if mixed["hbm_floor_ms"] >= mixed["mfma_floor_ms"] else "mfma"
            say("decode, batch 8, of the 8B shape")
            s8, _, bytes8 = other.decode_point(8, 20, 6)
            # a whole prompt of the shape's own context: 8,192 tokens give every compute unit eight workgroups of
            # attention and the library whole tiles, which 2,048 tokens of the small shape do not
            long_prefill = other.prefill_point(tokens=SHAPES["8b"][1]["max_position_embeddings"])
            points["prefill_8b_8192_ms"] = long_prefill["ms"]
            points["prefill_8b_8192_frac_mfma"] = long_prefill["frac"]
            other.close()
            points["decode_8b_b8_ms"] = round(s8 * 1e3, 3)
            points["decode_8b_b8_frac_hbm"] = round(bytes8 / s8 / HBM_PEAK, 4)
            other = Workbench("32b", OTHER_SHAPE_LAYERS["32b"], device, largest_batch=64, steps=20, prefill_room=False)
            say("decode, batch 64, of the 32B shape")
            s32, v32, bytes32 = other.decode_point(64, 12, 6)
            other.close()
            points["decode_32b_b64_ms"] = round(s32 * 1e3, 3)
            points["decode_32b_b64_frac_hbm"] = round(bytes32 / s32 / HBM_PEAK, 4)
            line["config"].update({"layers_8b": OTHER_SHAPE_LAYERS["8b"], "layers_8b_full": SHAPES["8b"][1]["num_hidden_layers"],
                                   "layers_32b": OTHER_SHAPE_LAYERS["32b"], "layers_32b_full": SHAPES["32b"][1]["num_hidden_layers"]})

    print(json.dumps(line), flush=True)
    tmp.cleanup()
    return 0


if __name__ == "__main__":
    sys.exit(main())
