"""The command line: a model folder and prompts of token ids to generated tokens.

The options the reference's server has keep their names, defaults and meanings
(crates/pagedllm-server/src/main.rs:20-71): --model, --dtype, --require-gpu,
--max-tokens, --block-size, --cache-mib, --max-batch, --attention,
--prefix-cache, --chunk.  --host and --port are gone with the server.  Prompts
are token ids, because text is outside this engine.
"""

from __future__ import annotations

import argparse
import json
import sys
from pathlib import Path

from .errors import ConfigError, IoError, PagedLLMError


def parser() -> argparse.ArgumentParser:
    p = argparse.ArgumentParser(prog="pagedllm", description=__doc__,
                                formatter_class=argparse.RawDescriptionHelpFormatter)
    p.add_argument("--model", required=True, help="directory holding config.json and model.safetensors")
    p.add_argument("--dtype", default="auto", choices=["auto", "f32", "bf16"],
                   help="convert the weights on load; auto keeps the checkpoint's own dtype")
    p.add_argument("--require-gpu", action="store_true",
                   help="refuse to start without a GPU (this engine always does; kept for the reference's scripts)")
    p.add_argument("--max-tokens", type=int, default=512, help="token budget for a request that names none")
    p.add_argument("--block-size", type=int, default=16, help="tokens per cache block")
    p.add_argument("--cache-mib", type=int, default=3584, help="bytes the KV cache may take, in mebibytes")
    p.add_argument("--max-batch", type=int, default=16, help="rows in one decode pass")
    p.add_argument("--attention", default="kernel", choices=["tensor", "kernel"],
                   help="kernel: the matrix-core attention kernels; tensor: the plain 32-bit-arithmetic kernel "
                        "they are checked against")
    p.add_argument("--prefix-cache", default="on", choices=["on", "off"],
                   help="whether a request may start from blocks a previous one left behind")
    p.add_argument("--chunk", default="128",
                   help="most tokens one forward pass may carry, or off to run a prompt whole")
    # what the reference takes over HTTP
    p.add_argument("--prompt-ids", action="append", default=[],
                   help="a prompt as comma-separated token ids; may be given several times")
    p.add_argument("--prompt-file", help="a file with one prompt a line: comma- or space-separated ids, or a JSON list")
    p.add_argument("--temperature", type=float, default=None)
    p.add_argument("--top-k", type=int, default=None)
    p.add_argument("--top-p", type=float, default=None)
    p.add_argument("--seed", type=int, default=None)
    p.add_argument("--stop-ids", default=None, help="comma-separated token ids that end a generation")
    p.add_argument("--sampler", default="device", choices=["device", "host"])
    p.add_argument("--strips", default="on", choices=["on", "off"],
                   help="keep the weight matrices a second time in the order decoding reads them fastest "
                        "(their memory again); off reads them as stored")
    # the random-weights mode
    p.add_argument("--random-weights", metavar="CONFIG_JSON",
                   help="write a model folder at --model from this config.json and --init-seed, then run it")
    p.add_argument("--init-seed", type=int, default=0)
    p.add_argument("--init-std", type=float, default=0.02)
    p.add_argument("--init-gain-std", type=float, default=0.1)
    return p


def parse_ids(text: str) -> list:
    text = text.strip()
    try:
        if text.startswith("["):
            return [int(t) for t in json.loads(text)]
        return [int(t) for t in text.replace(",", " ").split()]
    except (ValueError, TypeError):
        shown = text if len(text) <= 60 else text[:57] + "..."
        raise ConfigError(f"token ids are whole numbers, separated by commas or spaces or as a JSON list: {shown!r}") from None


def read_text(path, what: str) -> str:
    try:
        return Path(path).read_text()
    except OSError as e:
        raise IoError(f"reading {what} {path}: {e}") from e


def main(argv=None) -> int:
    args = parser().parse_args(argv)
    try:
        if args.chunk == "off":
            chunk = None
        else:
            try:
                chunk = int(args.chunk)
            except ValueError:
                raise ConfigError(f"--chunk {args.chunk!r}, which is neither a token count nor \"off\"") from None
            if chunk == 0:
                raise ConfigError("--chunk 0 would carry nothing")
        if args.random_weights:
            from .weights import write_random_model

            try:
                config = json.loads(read_text(args.random_weights, "--random-weights"))
            except json.JSONDecodeError as e:
                raise ConfigError(f"--random-weights {args.random_weights} is not JSON: {e}") from None
            write_random_model(args.model, config, seed=args.init_seed, std=args.init_std,
                               gain_std=args.init_gain_std,
                               dtype="float32" if args.dtype == "f32" else "bfloat16")
        prompts = [parse_ids(p) for p in args.prompt_ids]
        if args.prompt_file:
            prompts += [parse_ids(line) for line in read_text(args.prompt_file, "--prompt-file").splitlines() if line.strip()]
        from . import kernels
        from .engine import Engine

        kernels.set_attention(args.attention)
        engine = Engine(args.model, dtype=args.dtype, block_size=args.block_size, cache_mib=args.cache_mib,
                        max_batch=args.max_batch, chunk=chunk, prefix_cache=args.prefix_cache == "on",
                        max_tokens=args.max_tokens, sampler=args.sampler, strips=args.strips == "on")
        print(engine.describe(), file=sys.stderr, flush=True)
        if not prompts:
            return 0
        stops = None if args.stop_ids is None else parse_ids(args.stop_ids)
        ids = [engine.submit(p, None, args.temperature, args.top_k, args.top_p,
                             None if args.seed is None else args.seed + i, stops)
               for i, p in enumerate(prompts)]
        engine.run()
        for i in ids:
            c = engine.take_result(i)
            print(json.dumps({"tokens": c.tokens, "finish": c.finish, "prompt_tokens": c.prompt_tokens,
                              "completion_tokens": len(c.tokens), "preemptions": c.preemptions}), flush=True)
        print(json.dumps({"metrics": engine.metrics()}), file=sys.stderr, flush=True)
        return 0
    except PagedLLMError as e:
        print(f"error: {e}", file=sys.stderr)
        return 1


if __name__ == "__main__":
    sys.exit(main())
