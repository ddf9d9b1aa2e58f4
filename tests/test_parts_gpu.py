"""Each part alone against the plain implementation's function for it, a toy
mixer with state of its own registered from outside the package, long decoding,
the first tokens of a sequence, and long portions over earlier context."""

from __future__ import annotations

import math
import types
from dataclasses import dataclass

import numpy as np
import pytest
import torch

import plain_qwen3 as plain
import replay_util as ru
from conftest import TINY_INIT, load_plain, rel_err

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
TOL = {torch.float32: 2e-5, torch.bfloat16: 2e-2}


def randn(*shape, std=1.0, seed=0):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(*shape, generator=g) * std


# --- norm -----------------------------------------------------------------------------------------

@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("width,eps", [(100, 1e-5), (1024, 1e-6)])
def test_norm_part(dtype, width, eps):
    from paged_llm_rs_amd.config import NormSpec
    from paged_llm_rs_amd.parts import NORMS

    gain = (1 + randn(width, std=0.2, seed=1)).to(dtype)
    part = NORMS["rms_norm"](NormSpec("rms_norm", eps), width, {"weight": gain.to(DEV)}, dtype, DEV)
    resid = randn(7, width, seed=2)
    delta = randn(7, width, seed=3).to(dtype)
    stream = resid.to(DEV).clone()
    out = part.apply(stream, delta.to(DEV), dtype)
    summed = resid.double() + delta.double()
    assert rel_err(stream, summed) < 1e-6, "the residual sum is 32-bit and written back"
    assert rel_err(out, plain.rms_norm(summed, gain.double(), eps)) < TOL[dtype]
    rows = torch.tensor([5, 0, 5], dtype=torch.int32, device=DEV)
    picked = part.apply(stream, None, dtype, rows=rows)
    assert rel_err(picked, plain.rms_norm(summed[[5, 0, 5]], gain.double(), eps)) < TOL[dtype]


# --- position encoding -------------------------------------------------------------------------------

@pytest.mark.parametrize("dim,theta", [(16, 10000.0), (48, 1e6)])
def test_position_part(dim, theta):
    from paged_llm_rs_amd.config import PositionSpec
    from paged_llm_rs_amd.parts import POSITIONS

    tables = POSITIONS["rotary_half"](PositionSpec("rotary_half", dim, theta, 300), DEV)
    positions = torch.tensor([0, 1, 7, 299])
    cos, sin = plain.rope_tables(dim, positions, theta)       # [n, dim], the half table twice
    assert rel_err(tables.cos[positions], cos[:, :dim // 2]) < 1e-6
    assert rel_err(tables.sin[positions], sin[:, :dim // 2]) < 1e-6


# --- feed-forward --------------------------------------------------------------------------------------

@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("rows", [3, 70])
def test_feed_forward_part(dtype, rows):
    from paged_llm_rs_amd.config import GatedMlpSpec
    from paged_llm_rs_amd.parts import FEED_FORWARDS

    hidden, inter = 96, 200
    w = {"m.gate_proj.weight": randn(inter, hidden, std=0.1, seed=1).to(dtype),
         "m.up_proj.weight": randn(inter, hidden, std=0.1, seed=2).to(dtype),
         "m.down_proj.weight": randn(hidden, inter, std=0.1, seed=3).to(dtype)}
    part = FEED_FORWARDS["gated_mlp"](GatedMlpSpec("gated_mlp", inter, "silu"), hidden,
                                      {k[2:]: v.to(DEV) for k, v in w.items()}, dtype, DEV, {})
    x = randn(rows, hidden, seed=4).to(dtype)
    want = plain.swiglu_mlp(x.double(), {k: v.double() for k, v in w.items()}, "m")
    assert rel_err(part.forward(x.to(DEV)), want) < TOL[dtype]


@pytest.mark.parametrize("rows,columns,width,route", [
    (8, 1024, 2048, "skinny"), (40, 1024, 2048, "skinny"), (300, 1024, 2048, "library"),
    (8, 2048, 16384, "stream"), (40, 4096, 8192, "stream"), (64, 4096, 8192, "stream"), (65, 4096, 8192, "library"),
    (40, 8192, 4096, "library"), (300, 4096, 12288, "split"), (1100, 4096, 12288, "split"), (1500, 4096, 12288, "library")])
def test_a_linear_by_each_of_its_products(rows, columns, width, route):
    """Which kernel runs a projection is decided by its shape alone, in one place; whichever it is, the plain
    product, the one that adds into the 32-bit stream and the gated one agree with 64-bit products of the same
    bfloat16 numbers."""
    from paged_llm_rs_amd import kernels
    from paged_llm_rs_amd.parts.linear import Linear

    took = ("stream" if kernels.stream_wins(rows, columns, width) else
            "skinny" if kernels.skinny_wins(rows, columns, width) else
            "split" if kernels.library_splits(rows, columns, width) > 1 else "library")
    assert took == route
    w = (torch.randn(columns, width, device=DEV) / math.sqrt(width)).bfloat16()
    x = torch.randn(rows, width, device=DEV).bfloat16()
    want = x.double() @ w.double().T
    linear = Linear(w)
    assert rel_err(linear.forward(x), want) < TOL[torch.bfloat16]
    stream = torch.randn(rows, columns, device=DEV)
    before = stream.clone()
    back = linear.forward(x, add_into=stream)
    total = stream if back is None else before + back.float()
    assert rel_err(total.double() - before.double(), want) < TOL[torch.bfloat16]
    if back is None:
        assert rel_err(stream.double() - before.double(), want) < 1e-5, "added in 32-bit, not through bfloat16"
    gated = linear.forward(x, swiglu=True)
    half = columns // 2
    assert gated.shape == (rows, half)
    assert rel_err(gated, torch.nn.functional.silu(want[:, :half]) * want[:, half:]) < TOL[torch.bfloat16]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("activation", ["gelu_pytorch_tanh", "gelu", "silu"])
@pytest.mark.parametrize("rows,hidden,inter", [(3, 96, 200), (70, 96, 200), (300, 128, 256), (1500, 64, 192)])
def test_gated_feed_forward_with_other_activations(dtype, activation, rows, hidden, inter):
    """The activation on the gate branch is the spec's: SiLU for this architecture, the two GELUs for others.  Few
    rows take it as the last stage of the product kernel, some hundred as the tiled product's, many as a kernel of
    its own behind the library's product."""
    from paged_llm_rs_amd.config import GatedMlpSpec
    from paged_llm_rs_amd.parts import FEED_FORWARDS

    w = {"gate_proj.weight": randn(inter, hidden, std=0.1, seed=1).to(dtype),
         "up_proj.weight": randn(inter, hidden, std=0.1, seed=2).to(dtype),
         "down_proj.weight": randn(hidden, inter, std=0.1, seed=3).to(dtype)}
    part = FEED_FORWARDS["gated_mlp"](GatedMlpSpec("gated_mlp", inter, activation), hidden,
                                      {k: v.to(DEV) for k, v in w.items()}, dtype, DEV, {})
    x = (randn(rows, hidden, seed=4) * 2).to(dtype)
    d = {k: v.double() for k, v in w.items()}
    gate, up = x.double() @ d["gate_proj.weight"].T, x.double() @ d["up_proj.weight"].T
    act = {"silu": torch.nn.functional.silu, "gelu": torch.nn.functional.gelu,
           "gelu_pytorch_tanh": lambda t: torch.nn.functional.gelu(t, approximate="tanh")}[activation]
    want = (act(gate) * up) @ d["down_proj.weight"].T
    assert rel_err(part.forward(x.to(DEV)), want) < TOL[dtype]


def test_an_activation_nobody_knows_is_refused():
    from paged_llm_rs_amd.config import GatedMlpSpec
    from paged_llm_rs_amd.errors import UnsupportedError
    from paged_llm_rs_amd.parts import FEED_FORWARDS

    w = {"gate_proj.weight": torch.zeros(8, 8, device=DEV), "up_proj.weight": torch.zeros(8, 8, device=DEV),
         "down_proj.weight": torch.zeros(8, 8, device=DEV)}
    with pytest.raises(UnsupportedError, match="relu"):
        FEED_FORWARDS["gated_mlp"](GatedMlpSpec("gated_mlp", 8, "relu"), 8, w, torch.float32, DEV, {})


# --- mixer ---------------------------------------------------------------------------------------------------

def one_layer_cache(mixer, block_size, pages, dtype):
    from paged_llm_rs_amd.cache import CacheLayout, PagedCache
    from paged_llm_rs_amd.config import ScheduleEntry

    layout = CacheLayout.from_blocks([types.SimpleNamespace(mixer=mixer)], [ScheduleEntry(0)])
    return PagedCache(layout, block_size, pages, dtype, DEV, max_seqs=4)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("nq,nkv,d,block_size", [(4, 2, 16, 4), (6, 1, 32, 16), (6, 3, 48, 8)])
def test_attention_part_in_portions(dtype, nq, nkv, d, block_size):
    """The mixer alone over its own pages: a sequence fed in portions (a long one, a short one, single
    tokens) gives what the plain attention gives for the whole sequence."""
    from paged_llm_rs_amd.config import AttentionSpec, NormSpec, PositionSpec
    from paged_llm_rs_amd.engine.batch import StepEntry, build_batch
    from paged_llm_rs_amd.parts import MIXERS, LayerContext

    hidden, eps, theta, n = 40, 1e-5, 5e5, 61
    cfg = {"num_attention_heads": nq, "num_key_value_heads": nkv, "head_dim": d, "rms_norm_eps": eps,
           "rope_theta": theta}
    w = {"a.q_proj.weight": randn(nq * d, hidden, std=0.2, seed=1), "a.k_proj.weight": randn(nkv * d, hidden, std=0.2, seed=2),
         "a.v_proj.weight": randn(nkv * d, hidden, std=0.2, seed=3), "a.o_proj.weight": randn(hidden, nq * d, std=0.2, seed=4),
         "a.q_norm.weight": 1 + randn(d, std=0.2, seed=5), "a.k_norm.weight": 1 + randn(d, std=0.2, seed=6)}
    w = {k: v.to(dtype) for k, v in w.items()}
    spec = AttentionSpec("paged_attention", nq, nkv, d, NormSpec("rms_norm", eps),
                         PositionSpec("rotary_half", d, theta, 128), None, None)
    mixer = MIXERS["paged_attention"](spec, hidden, {k[2:]: v.to(DEV) for k, v in w.items()}, dtype, DEV, {})
    cache = one_layer_cache(mixer, block_size, 24, dtype)
    x = randn(n, hidden, seed=7).to(dtype)
    want = plain.attention(x.double(), {k: v.double() for k, v in w.items()}, "a", cfg, torch.arange(n))
    cache.manager.add_sequence(1)
    got, at = [], 0
    for count in (20, 1, 17, 1, 1, 19, 2):
        assert cache.manager.reserve(1, count)
        entries = [StepEntry(1, [0] * count, at, [])]
        batch = build_batch(entries, cache.manager, 1, 10, 128, DEV)
        got.append(mixer.forward(x[at:at + count].to(DEV).contiguous(), LayerContext(batch, cache, 0, 0, True)))
        cache.manager.advance(1, count)
        at += count
    assert at == n
    assert rel_err(torch.cat(got), want) < TOL[dtype]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_attention_part_with_biases(dtype):
    """Projections with a bias each (another family's attention): the plain attention on the input with a column
    of ones appended and the biases as one more column of the weights gives the same q, k and v; the output
    projection's bias is added to its result.  Decoded tokens and portions, so that the fused and the unfused
    ways of a step are both taken."""
    from paged_llm_rs_amd.config import AttentionSpec, NormSpec, PositionSpec
    from paged_llm_rs_amd.engine.batch import StepEntry, build_batch
    from paged_llm_rs_amd.parts import MIXERS, LayerContext

    nq, nkv, d, block_size = 4, 2, 32, 8
    hidden, eps, theta, n = 40, 1e-5, 5e5, 45
    cfg = {"num_attention_heads": nq, "num_key_value_heads": nkv, "head_dim": d, "rms_norm_eps": eps, "rope_theta": theta}
    w = {"q_proj.weight": randn(nq * d, hidden, std=0.2, seed=1), "k_proj.weight": randn(nkv * d, hidden, std=0.2, seed=2),
         "v_proj.weight": randn(nkv * d, hidden, std=0.2, seed=3), "o_proj.weight": randn(hidden, nq * d, std=0.2, seed=4),
         "q_norm.weight": 1 + randn(d, std=0.2, seed=5), "k_norm.weight": 1 + randn(d, std=0.2, seed=6),
         "q_proj.bias": randn(nq * d, std=0.5, seed=7), "k_proj.bias": randn(nkv * d, std=0.5, seed=8),
         "v_proj.bias": randn(nkv * d, std=0.5, seed=9), "o_proj.bias": randn(hidden, std=0.5, seed=10)}
    w = {k: v.to(dtype) for k, v in w.items()}
    spec = AttentionSpec("paged_attention", nq, nkv, d, NormSpec("rms_norm", eps), PositionSpec("rotary_half", d, theta, 128),
                         None, None, qkv_bias=True, out_bias=True)
    cls = MIXERS["paged_attention"]
    assert {decl.name for decl in cls.declare(spec, hidden)} == set(w)
    mixer = cls(spec, hidden, {k: v.to(DEV) for k, v in w.items()}, dtype, DEV, {})
    cache = one_layer_cache(mixer, block_size, 24, dtype)
    x = randn(n, hidden, seed=11).to(dtype)
    ones = torch.ones(n, 1, dtype=torch.float64)
    wide = {f"a.{p}_proj.weight": torch.cat([w[f"{p}_proj.weight"].double(), w[f"{p}_proj.bias"].double()[:, None]], dim=1)
            for p in "qkv"}
    wide.update({"a.o_proj.weight": w["o_proj.weight"].double(), "a.q_norm.weight": w["q_norm.weight"].double(),
                 "a.k_norm.weight": w["k_norm.weight"].double()})
    want = plain.attention(torch.cat([x.double(), ones], dim=1), wide, "a", cfg, torch.arange(n)) + w["o_proj.bias"].double()
    cache.manager.add_sequence(1)
    got, at = [], 0
    for count in (20, 1, 1, 17, 1, 3, 2):
        assert cache.manager.reserve(1, count)
        batch = build_batch([StepEntry(1, [0] * count, at, [])], cache.manager, 1, 10, 128, DEV)
        got.append(mixer.forward(x[at:at + count].to(DEV).contiguous(), LayerContext(batch, cache, 0, 0, True)))
        cache.manager.advance(1, count)
        at += count
    assert at == n
    assert rel_err(torch.cat(got), want) < TOL[dtype]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_attention_part_with_the_rotation_of_neighbours(dtype):
    """A position encoding whose angles turn neighbouring elements, chosen by its kind in the spec.  Scores do not
    change when the elements of q and k are reordered alike, so the plain attention over weights whose q and k
    rows are gathered even-before-odd within each head (and gains alike) is the reference."""
    from paged_llm_rs_amd.config import AttentionSpec, NormSpec, PositionSpec
    from paged_llm_rs_amd.engine.batch import StepEntry, build_batch
    from paged_llm_rs_amd.parts import MIXERS, LayerContext

    nq, nkv, d, block_size = 4, 2, 32, 8
    hidden, eps, theta, n = 40, 1e-5, 1e4, 37
    cfg = {"num_attention_heads": nq, "num_key_value_heads": nkv, "head_dim": d, "rms_norm_eps": eps, "rope_theta": theta}
    w = {"q_proj.weight": randn(nq * d, hidden, std=0.2, seed=1), "k_proj.weight": randn(nkv * d, hidden, std=0.2, seed=2),
         "v_proj.weight": randn(nkv * d, hidden, std=0.2, seed=3), "o_proj.weight": randn(hidden, nq * d, std=0.2, seed=4),
         "q_norm.weight": 1 + randn(d, std=0.2, seed=5), "k_norm.weight": 1 + randn(d, std=0.2, seed=6)}
    w = {k: v.to(dtype) for k, v in w.items()}
    spec = AttentionSpec("paged_attention", nq, nkv, d, NormSpec("rms_norm", eps),
                         PositionSpec("rotary_neighbours", d, theta, 128), None, None)
    mixer = MIXERS["paged_attention"](spec, hidden, {k: v.to(DEV) for k, v in w.items()}, dtype, DEV, {})
    cache = one_layer_cache(mixer, block_size, 16, dtype)
    x = randn(n, hidden, seed=11).to(dtype)
    order = torch.cat([torch.arange(0, d, 2), torch.arange(1, d, 2)])
    gathered = {"a.q_proj.weight": w["q_proj.weight"].double().reshape(nq, d, hidden)[:, order].reshape(nq * d, hidden),
                "a.k_proj.weight": w["k_proj.weight"].double().reshape(nkv, d, hidden)[:, order].reshape(nkv * d, hidden),
                "a.v_proj.weight": w["v_proj.weight"].double(), "a.o_proj.weight": w["o_proj.weight"].double(),
                "a.q_norm.weight": w["q_norm.weight"].double()[order], "a.k_norm.weight": w["k_norm.weight"].double()[order]}
    want = plain.attention(x.double(), gathered, "a", cfg, torch.arange(n))
    cache.manager.add_sequence(1)
    got, at = [], 0
    for count in (20, 1, 1, 15):
        assert cache.manager.reserve(1, count)
        batch = build_batch([StepEntry(1, [0] * count, at, [])], cache.manager, 1, 10, 128, DEV)
        got.append(mixer.forward(x[at:at + count].to(DEV).contiguous(), LayerContext(batch, cache, 0, 0, True)))
        cache.manager.advance(1, count)
        at += count
    assert rel_err(torch.cat(got), want) < TOL[dtype]


# --- block ---------------------------------------------------------------------------------------------------------

@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_block_part(model_dirs, dtype):
    """One layer of a tiny model through the block class, fed the plain implementation's own input."""
    from paged_llm_rs_amd.cache import PagedCache
    from paged_llm_rs_amd.engine.batch import StepEntry, build_batch
    from paged_llm_rs_amd.parts import LayerContext, load_model

    name = "float32" if dtype == torch.float32 else "bfloat16"
    d = model_dirs("C", name)
    cfg, weights = load_plain(d)
    _, model = load_model(d, name, DEV)
    n = 23
    x = randn(n, cfg["hidden_size"], seed=9)
    want = plain.decoder_block(x.double(), {k: v.double() for k, v in weights.items()}, "model.layers.1", cfg, torch.arange(n))
    cache = PagedCache(model.cache_layout, 8, 8, dtype, DEV, max_seqs=2)
    cache.manager.add_sequence(1)
    assert cache.manager.reserve(1, n)
    batch = build_batch([StepEntry(1, [0] * n, 0, [])], cache.manager, 1, cfg["vocab_size"], 0, DEV)
    resid = x.to(DEV).clone()
    delta = model.blocks[1].forward(resid, None, LayerContext(batch, cache, 1, 1, True))
    assert rel_err(resid.double() + delta.double(), want) < TOL[dtype]


# --- a toy mixer with state of its own, defined here ---------------------------------------------------------------------

@dataclass(frozen=True)
class RunningMeanSpec:
    kind: str = "running_mean"


class RunningMeanMixer:
    """out[t] = W . mean(x[0..t]): the sum so far and the count are the request's state."""
    graph_safe = False      # it reads the step's layout on the host

    @staticmethod
    def declare(spec, hidden):
        from paged_llm_rs_amd.weights.loader import ParamDecl
        return [ParamDecl("proj.weight", (hidden, hidden))]

    def __init__(self, spec, hidden, params, dtype, device, shared):
        self.w, self.hidden = params["proj.weight"], hidden

    def cache_spec(self):
        return None

    def state_spec(self):
        from paged_llm_rs_amd.cache import StateSpec
        return StateSpec((self.hidden + 1,), torch.float32)

    def forward(self, x, ctx):
        batch, state, H = ctx.batch, ctx.state(), self.hidden
        out = torch.empty_like(x)
        starts, counts, slots = (t.cpu().tolist() for t in (batch.q_start, batch.q_len, batch.state_slots))
        for a, n, slot in zip(starts, counts, slots):
            assert slot >= 0, "a request of a model with state has a slot"
            sums = state[slot, :H] + x[a:a + n].float().cumsum(0)
            seen = state[slot, H] + torch.arange(1, n + 1, device=x.device)
            out[a:a + n] = ((sums / seen[:, None]) @ self.w.float().t()).to(x.dtype)
            state[slot, :H] = sums[-1]
            state[slot, H] = seen[-1]
        return out


class ToyConfig:
    """Layer 0 mixes by running mean, layer 1 by attention; both read ``hidden_size`` and so on from config.json."""

    def __init__(self, d):
        self.d = d

    @classmethod
    def from_dict(cls, d):
        return cls(dict(d))

    def to_dict(self):
        return dict(self.d)

    def model_spec(self):
        from paged_llm_rs_amd.config import (AttentionSpec, GatedMlpSpec, LayerSpec, ModelSpec, NormSpec, PositionSpec,
                                             ScheduleEntry)
        d = self.d
        norm = NormSpec("rms_norm", d["rms_norm_eps"])
        ffn = GatedMlpSpec("gated_mlp", d["intermediate_size"], "silu")
        attention = AttentionSpec("paged_attention", d["num_attention_heads"], d["num_key_value_heads"], d["head_dim"],
                                  norm, PositionSpec("rotary_half", d["head_dim"], d["rope_theta"],
                                                     d["max_position_embeddings"]), None, None)
        layers = (LayerSpec("pre_norm", RunningMeanSpec(), ffn, norm, "model.layers.0"),
                  LayerSpec("pre_norm", attention, ffn, norm, "model.layers.1"))
        return ModelSpec(d["hidden_size"], d["vocab_size"], layers, (ScheduleEntry(0), ScheduleEntry(1)), norm,
                         d["tie_word_embeddings"], d["max_position_embeddings"])


TOY = {"architectures": ["ToyForCausalLM"], "model_type": "toy", "hidden_size": 48, "intermediate_size": 80,
       "num_attention_heads": 2, "num_key_value_heads": 1, "head_dim": 16, "rms_norm_eps": 1e-5, "rope_theta": 1e4,
       "vocab_size": 97, "max_position_embeddings": 256, "tie_word_embeddings": True}


def toy_plain(weights, tokens):
    w = {k: v.double() for k, v in weights.items()}
    n = len(tokens)
    x = w["model.embed_tokens.weight"][torch.tensor(tokens)]
    eps = TOY["rms_norm_eps"]
    normed = plain.rms_norm(x, w["model.layers.0.input_layernorm.weight"], eps)
    mean = normed.cumsum(0) / torch.arange(1, n + 1, dtype=torch.float64)[:, None]
    x = x + mean @ w["model.layers.0.self_attn.proj.weight"].T
    x = x + plain.swiglu_mlp(plain.rms_norm(x, w["model.layers.0.post_attention_layernorm.weight"], eps), w, "model.layers.0.mlp")
    x = plain.decoder_block(x, w, "model.layers.1", TOY, torch.arange(n))
    return plain.rms_norm(x, w["model.norm.weight"], eps) @ w["model.embed_tokens.weight"].T


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_toy_mixer_with_state_is_registered_built_and_stepped(tmp_path, dtype):
    """A mixer that keeps a running mean in a state slot, an architecture that uses it in one layer
    beside attention in another: registered here, written by the random-weights mode, replayed in
    portions mixed with other requests, and generated from through the engine."""
    from safetensors.torch import load_file

    from paged_llm_rs_amd import Engine, register_architecture, write_random_model
    from paged_llm_rs_amd.engine.replay import Replayer
    from paged_llm_rs_amd.parts import register_mixer

    register_mixer("running_mean", RunningMeanMixer)
    register_architecture("ToyForCausalLM", ToyConfig, model_type="toy")
    folder = write_random_model(tmp_path / "toy", TOY, seed=5, std=0.1, gain_std=0.2, dtype=dtype)
    weights = load_file(str(folder / "model.safetensors"))
    assert "model.layers.0.self_attn.proj.weight" in weights and "model.layers.1.self_attn.q_proj.weight" in weights
    prompts = ru.make_prompts(TOY["vocab_size"], [30, 9, 41, 17, 25], seed=3)
    want = {name: toy_plain(weights, toks) for name, toks in prompts.items()}
    tolerance = 1e-5 if dtype == "float32" else 2e-2
    for steps, live in ((ru.whole(prompts), 1), (ru.mixed(prompts, seed=7, max_live=3), 3)):
        r = Replayer(folder, dtype, max_tokens=ru.pool_tokens(prompts, live), block_size=8, max_live=4)
        assert not r.runner.use_graphs and r.cache.layout.states, "the toy's state slots exist and its steps run eagerly"
        got = ru.collect(r, steps)
        worst, where = ru.worst_error(got, want)
        assert worst <= tolerance, f"{worst:.3e} at {where}"
        assert r.cache.manager.free_state_slots == 4, "every state slot came back"
    engine = Engine(folder, dtype="f32" if dtype == "float32" else "bf16", block_size=8, num_blocks=16, max_batch=3, chunk=8)
    out = engine.generate(list(prompts.values())[:3], max_tokens=5, temperature=0.0, stop_tokens=[])
    for prompt, result in zip(prompts.values(), out):
        tokens = list(prompt)
        for produced in result["tokens"]:
            logits = toy_plain(weights, tokens)[-1]
            best = int(torch.argmax(logits))
            if produced != best:
                assert float(logits[best] - logits[produced]) <= tolerance * float(logits.abs().max())
            tokens.append(produced)


class RunningSumMixer:
    """out[t] = W . sum(x[0..t]): the sum so far is the request's state.  Written with device operations only and
    tolerant of padding rows (position -1, state slot -1), so its steps may be captured as graphs."""
    graph_safe = True

    @staticmethod
    def declare(spec, hidden):
        from paged_llm_rs_amd.weights.loader import ParamDecl
        return [ParamDecl("proj.weight", (hidden, hidden))]

    def __init__(self, spec, hidden, params, dtype, device, shared):
        self.w, self.hidden = params["proj.weight"], hidden

    def cache_spec(self):
        return None

    def state_spec(self):
        from paged_llm_rs_amd.cache import StateSpec
        return StateSpec((self.hidden,), torch.float32)

    def forward(self, x, ctx):
        b, state = ctx.batch, ctx.state()
        seq, starts, counts, slots = b.seq_of.long(), b.q_start.long(), b.q_len.long(), b.state_slots.long()
        live = slots >= 0
        rows = torch.where((b.positions >= 0)[:, None], x.float(), torch.zeros((), device=x.device))
        through = rows.cumsum(0)
        before = torch.where((starts > 0)[:, None], through[(starts - 1).clamp_min(0)], torch.zeros((), device=x.device))
        held = torch.where(live[:, None], state[slots.clamp_min(0)], torch.zeros((), device=x.device))
        out = ((held[seq] + through - before[seq]) @ self.w.float().t()).to(x.dtype)
        brought = through[(starts + counts - 1).clamp_min(0)] - before
        state.index_add_(0, slots.clamp_min(0), torch.where((live & (counts > 0))[:, None], brought, torch.zeros((), device=x.device)))
        return out


@dataclass(frozen=True)
class RunningSumSpec:
    kind: str = "running_sum"


class SumToyConfig(ToyConfig):
    def model_spec(self):
        import dataclasses

        spec = super().model_spec()
        first = dataclasses.replace(spec.layers[0], mixer=RunningSumSpec())
        return dataclasses.replace(spec, layers=(first, spec.layers[1]))


def sum_toy_plain(weights, tokens):
    w = {k: v.double() for k, v in weights.items()}
    n = len(tokens)
    x = w["model.embed_tokens.weight"][torch.tensor(tokens)]
    eps = TOY["rms_norm_eps"]
    normed = plain.rms_norm(x, w["model.layers.0.input_layernorm.weight"], eps)
    x = x + normed.cumsum(0) @ w["model.layers.0.self_attn.proj.weight"].T
    x = x + plain.swiglu_mlp(plain.rms_norm(x, w["model.layers.0.post_attention_layernorm.weight"], eps), w, "model.layers.0.mlp")
    x = plain.decoder_block(x, w, "model.layers.1", TOY, torch.arange(n))
    return plain.rms_norm(x, w["model.norm.weight"], eps) @ w["model.embed_tokens.weight"].T


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_mixer_with_state_in_captured_steps(tmp_path, dtype):
    """A mixer that adds every token it sees into its request's state slot, in steps that are captured as graphs:
    the step that brings a capture about must advance the state once, like every other.  (The run before a
    capture and the capture itself go over idle rows.)  Steps of one token a request are captured at their first
    coming, steps of other shapes at their second; both happen here, and graphs on and off agree."""
    from safetensors.torch import load_file

    from paged_llm_rs_amd import register_architecture, write_random_model
    from paged_llm_rs_amd.engine.replay import Replayer
    from paged_llm_rs_amd.parts import register_mixer

    register_mixer("running_sum", RunningSumMixer)
    register_architecture("SumToyForCausalLM", SumToyConfig, model_type="sum_toy")
    config = dict(TOY, architectures=["SumToyForCausalLM"], model_type="sum_toy")
    folder = write_random_model(tmp_path / "toy", config, seed=6, std=0.05, gain_std=0.2, dtype=dtype)
    weights = load_file(str(folder / "model.safetensors"))
    prompts = ru.make_prompts(TOY["vocab_size"], [30, 9, 41, 17, 25, 12], seed=4)
    want = {name: sum_toy_plain(weights, toks) for name, toks in prompts.items()}
    tolerance = 1e-5 if dtype == "float32" else 2e-2
    # the same portion sizes for every request, so that shapes of step come again and are captured
    schedules = [(ru.tail_decoded(prompts, 8), 1), (ru.portions(prompts, sizes=(4, 4, 4, 4, 4, 4, 4, 4, 4, 4, 4)), 1),
                 (ru.mixed(prompts, seed=7, max_live=3), 3)]
    for steps, live in schedules:
        outcomes = []
        for graphs in (True, False):
            r = Replayer(folder, dtype, max_tokens=ru.pool_tokens(prompts, live), block_size=8, max_live=4, graphs=graphs)
            assert r.runner.use_graphs == graphs
            got = ru.collect(r, steps)
            worst, where = ru.worst_error(got, want)
            assert worst <= tolerance, f"graphs {graphs}: {worst:.3e} at {where}"
            if graphs:
                assert r.runner.graph_steps > 0, "some steps were replayed from graphs"
            outcomes.append(got)
        assert outcomes[0].keys() == outcomes[1].keys()


# --- a toy feed-forward with routing and a toy position encoding, defined here ----------------------------------------------

@dataclass(frozen=True)
class RoutedSpec:
    kind: str = "routed_mlp"
    experts: int = 3
    intermediate_size: int = 0
    top_k: int = 1


class RoutedMlp:
    """Experts of the gated form behind a router: the router's logits and their softmax in 32-bit, the
    ``top_k`` largest weights kept and scaled to sum to one, the experts' outputs mixed by them."""

    @staticmethod
    def declare(spec, hidden):
        from paged_llm_rs_amd.weights.loader import ParamDecl
        decls = [ParamDecl("router.weight", (spec.experts, hidden))]
        for e in range(spec.experts):
            decls += [ParamDecl(f"experts.{e}.gate_proj.weight", (spec.intermediate_size, hidden)),
                      ParamDecl(f"experts.{e}.up_proj.weight", (spec.intermediate_size, hidden)),
                      ParamDecl(f"experts.{e}.down_proj.weight", (hidden, spec.intermediate_size))]
        return decls

    def __init__(self, spec, hidden, params, dtype, device, shared):
        self.spec, self.params = spec, params

    def forward(self, x):
        spec, w = self.spec, self.params
        weights = torch.softmax(x.float() @ w["router.weight"].float().t(), dim=-1)
        if spec.top_k < spec.experts:
            kept = torch.zeros_like(weights).scatter_(1, weights.topk(spec.top_k, dim=-1).indices, 1.0)
            weights = weights * kept
            weights = weights / weights.sum(-1, keepdim=True)
        out = torch.zeros(x.shape, dtype=torch.float32, device=x.device)
        for e in range(spec.experts):
            gate = x @ w[f"experts.{e}.gate_proj.weight"].t()
            up = x @ w[f"experts.{e}.up_proj.weight"].t()
            y = (torch.nn.functional.silu(gate.float()) * up.float()).to(x.dtype) @ w[f"experts.{e}.down_proj.weight"].t()
            out += weights[:, e:e + 1] * y.float()
        return out.to(x.dtype)


class LinearAngles:
    """Angles that grow linearly with the pair's index instead of geometrically, over part of a head:
    position p turns pair i (elements i and i + dim/2 of the first ``dim``) by p * theta * (i + 1)."""

    def __init__(self, spec, device):
        self.dim, self.max_positions = spec.dim, spec.max_positions
        angle = (torch.arange(spec.max_positions, dtype=torch.float64)[:, None]
                 * spec.theta * torch.arange(1, spec.dim // 2 + 1, dtype=torch.float64)[None, :])
        self.cos = angle.cos().float().to(device).contiguous()
        self.sin = angle.sin().float().to(device).contiguous()


class RoutedConfig:
    """Two layers of attention with the linear angles over half of each head; the feed-forward of layer 0
    is routed, that of layer 1 the plain gated one."""

    def __init__(self, d):
        self.d = d

    @classmethod
    def from_dict(cls, d):
        return cls(dict(d))

    def to_dict(self):
        return dict(self.d)

    def model_spec(self):
        from paged_llm_rs_amd.config import (AttentionSpec, GatedMlpSpec, LayerSpec, ModelSpec, NormSpec, PositionSpec,
                                             ScheduleEntry)
        d = self.d
        norm = NormSpec("rms_norm", d["rms_norm_eps"])
        position = PositionSpec("linear_angles", d["rotated"], d["angle_step"], d["max_position_embeddings"])
        attention = AttentionSpec("paged_attention", d["num_attention_heads"], d["num_key_value_heads"], d["head_dim"],
                                  norm, position, None, None)
        routed = RoutedSpec("routed_mlp", d["num_experts"], d["expert_intermediate_size"], d["experts_per_token"])
        layers = (LayerSpec("pre_norm", attention, routed, norm, "model.layers.0"),
                  LayerSpec("pre_norm", attention, GatedMlpSpec("gated_mlp", d["intermediate_size"], "silu"), norm,
                            "model.layers.1"))
        return ModelSpec(d["hidden_size"], d["vocab_size"], layers, (ScheduleEntry(0), ScheduleEntry(1)), norm,
                         d["tie_word_embeddings"], d["max_position_embeddings"])


ROUTED = {"architectures": ["RoutedToyForCausalLM"], "model_type": "routed_toy", "hidden_size": 40, "intermediate_size": 72,
          "num_experts": 3, "expert_intermediate_size": 24, "experts_per_token": 1, "num_attention_heads": 3,
          "num_key_value_heads": 1, "head_dim": 32, "rotated": 16, "angle_step": 0.013, "rms_norm_eps": 1e-6,
          "vocab_size": 113, "max_position_embeddings": 192, "tie_word_embeddings": False}


def routed_plain(weights, cfg, tokens):
    w = {k: v.double() for k, v in weights.items()}
    n, eps = len(tokens), cfg["rms_norm_eps"]
    nq, nkv, d, rot = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"], cfg["rotated"]
    positions = torch.arange(n, dtype=torch.float64)
    angle = positions[:, None] * cfg["angle_step"] * torch.arange(1, rot // 2 + 1, dtype=torch.float64)[None, :]
    cos, sin = angle.cos()[:, None, :], angle.sin()[:, None, :]

    def turn(t):   # [n, heads, d]
        a, b, rest = t[..., :rot // 2], t[..., rot // 2:rot], t[..., rot:]
        return torch.cat([a * cos - b * sin, b * cos + a * sin, rest], dim=-1)

    def attend(x, prefix):
        q = plain.rms_norm((x @ w[f"{prefix}.q_proj.weight"].T).reshape(n, nq, d), w[f"{prefix}.q_norm.weight"], eps)
        k = plain.rms_norm((x @ w[f"{prefix}.k_proj.weight"].T).reshape(n, nkv, d), w[f"{prefix}.k_norm.weight"], eps)
        v = (x @ w[f"{prefix}.v_proj.weight"].T).reshape(n, nkv, d)
        k, v = plain.repeat_kv(turn(k), nq // nkv), plain.repeat_kv(v, nq // nkv)
        return plain.attention_core(turn(q), k, v, 1.0 / math.sqrt(d)).reshape(n, nq * d) @ w[f"{prefix}.o_proj.weight"].T

    def routed(x, prefix):
        weight = plain.softmax_last(x @ w[f"{prefix}.router.weight"].T)
        if cfg["experts_per_token"] < cfg["num_experts"]:
            kept = torch.zeros_like(weight).scatter_(1, weight.topk(cfg["experts_per_token"], dim=-1).indices, 1.0)
            weight = weight * kept / (weight * kept).sum(-1, keepdim=True)
        return sum(weight[:, e:e + 1] * plain.swiglu_mlp(x, w, f"{prefix}.experts.{e}") for e in range(cfg["num_experts"]))

    x = w["model.embed_tokens.weight"][torch.tensor(tokens)]
    for layer, feed in ((0, routed), (1, lambda t, prefix: plain.swiglu_mlp(t, w, prefix))):
        p = f"model.layers.{layer}"
        x = x + attend(plain.rms_norm(x, w[f"{p}.input_layernorm.weight"], eps), f"{p}.self_attn")
        x = x + feed(plain.rms_norm(x, w[f"{p}.post_attention_layernorm.weight"], eps), f"{p}.mlp")
    return plain.rms_norm(x, w["model.norm.weight"], eps) @ w["lm_head.weight"].T


@pytest.mark.parametrize("dtype,experts_per_token", [("float32", 1), ("float32", 2), ("bfloat16", 3)])
def test_a_toy_feed_forward_with_routing_and_a_toy_position_encoding(tmp_path, dtype, experts_per_token):
    """A routed feed-forward in one layer beside the framework's own in the other, and angles of another
    law over half of each head: registered here, built, replayed whole, decoded and mixed.  (In bfloat16
    every expert keeps its weight: a router that cuts experts off is not continuous, and a rounding
    that flips its choice at a near tie is no fault of the engine's.)"""
    from safetensors.torch import load_file

    from paged_llm_rs_amd import register_architecture, write_random_model
    from paged_llm_rs_amd.engine.replay import Replayer
    from paged_llm_rs_amd.parts import register_feed_forward, register_position

    register_feed_forward("routed_mlp", RoutedMlp)
    register_position("linear_angles", LinearAngles)
    register_architecture("RoutedToyForCausalLM", RoutedConfig, model_type="routed_toy")
    cfg = dict(ROUTED, experts_per_token=experts_per_token)
    folder = write_random_model(tmp_path / "routed", cfg, seed=8, std=0.15, gain_std=0.2, dtype=dtype)
    weights = load_file(str(folder / "model.safetensors"))
    assert "model.layers.0.mlp.experts.2.down_proj.weight" in weights and "model.layers.1.mlp.gate_proj.weight" in weights
    prompts = ru.make_prompts(cfg["vocab_size"], [40, 7, 66, 21], seed=4)
    want = {name: routed_plain(weights, cfg, toks) for name, toks in prompts.items()}
    tolerance = 1e-5 if dtype == "float32" else 2e-2
    for steps, live in ((ru.whole(prompts), 1), (ru.tail_decoded(prompts, 12), 1), (ru.mixed(prompts, seed=2, max_live=3), 3)):
        r = Replayer(folder, dtype, max_tokens=ru.pool_tokens(prompts, live), block_size=8, max_live=4)
        got = ru.collect(r, steps)
        worst, where = ru.worst_error(got, want)
        assert worst <= tolerance, f"{worst:.3e} at {where}"


# --- layers that see all keys beside layers that see a window of them ----------------------------------------------------

class WindowedConfig:
    """Layer 0 attends to every key, layers 1 and 2 to the last ``window`` keys: two groups of pages."""

    def __init__(self, d):
        self.d = d

    @classmethod
    def from_dict(cls, d):
        return cls(dict(d))

    def to_dict(self):
        return dict(self.d)

    def model_spec(self):
        from paged_llm_rs_amd.config import (AttentionSpec, GatedMlpSpec, LayerSpec, ModelSpec, NormSpec, PositionSpec,
                                             ScheduleEntry)
        d = self.d
        norm = NormSpec("rms_norm", d["rms_norm_eps"])
        ffn = GatedMlpSpec("gated_mlp", d["intermediate_size"], "silu")
        position = PositionSpec("rotary_half", d["head_dim"], d["rope_theta"], d["max_position_embeddings"])

        def attention(window):
            return AttentionSpec("paged_attention", d["num_attention_heads"], d["num_key_value_heads"], d["head_dim"],
                                 norm, position, window, None)

        layers = tuple(LayerSpec("pre_norm", attention(None if i == 0 else d["window"]), ffn, norm, f"model.layers.{i}")
                       for i in range(3))
        return ModelSpec(d["hidden_size"], d["vocab_size"], layers, tuple(ScheduleEntry(i) for i in range(3)), norm,
                         d["tie_word_embeddings"], d["max_position_embeddings"])


WINDOWED = {"architectures": ["WindowedToyForCausalLM"], "model_type": "windowed_toy", "hidden_size": 64,
            "intermediate_size": 96, "num_attention_heads": 4, "num_key_value_heads": 2, "head_dim": 32, "window": 21,
            "rms_norm_eps": 1e-6, "rope_theta": 1e4, "vocab_size": 101, "max_position_embeddings": 512,
            "tie_word_embeddings": True}


def windowed_plain(weights, tokens):
    w = {k: v.double() for k, v in weights.items()}
    x = w["model.embed_tokens.weight"][torch.tensor(tokens)]
    positions = torch.arange(len(tokens))
    for i in range(3):
        x = plain.decoder_block(x, w, f"model.layers.{i}", WINDOWED, positions, window=None if i == 0 else WINDOWED["window"])
    return plain.rms_norm(x, w["model.norm.weight"], WINDOWED["rms_norm_eps"]) @ w["model.embed_tokens.weight"].T


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_layers_with_a_window_beside_layers_without(tmp_path, dtype):
    """Two groups of pages in one model: the windowed layers give pages back while a request still runs,
    the others keep theirs; replayed whole, decoded, in portions and mixed with so few pages that they are
    used again, against the plain implementation with the window in its mask."""
    from safetensors.torch import load_file

    from paged_llm_rs_amd import register_architecture, write_random_model
    from paged_llm_rs_amd.engine.replay import Replayer

    register_architecture("WindowedToyForCausalLM", WindowedConfig, model_type="windowed_toy")
    folder = write_random_model(tmp_path / "windowed", WINDOWED, seed=12, std=0.08, gain_std=0.2, dtype=dtype)
    weights = load_file(str(folder / "model.safetensors"))
    prompts = ru.make_prompts(WINDOWED["vocab_size"], [90, 23, 141, 60], seed=6)
    want = {name: windowed_plain(weights, toks) for name, toks in prompts.items()}
    tolerance = 1e-5 if dtype == "float32" else 2e-2
    schedules = ((ru.whole(prompts), 1), (ru.tail_decoded(prompts, 32), 1), (ru.portions(prompts), 1),
                 (ru.mixed(prompts, seed=3, max_live=3), 3))
    for steps, live in schedules:
        r = Replayer(folder, dtype, max_tokens=ru.pool_tokens(prompts, live), block_size=8, max_live=4)
        assert len(r.cache.layout.groups) == 2, "the windowed layers have pages of their own"
        got = ru.collect(r, steps)
        worst, where = ru.worst_error(got, want)
        assert worst <= tolerance, f"{worst:.3e} at {where}"
        assert r.cache.manager.live_sequences == 0 and r.cache.manager.available() == r.cache.manager.total()
    # while a request runs, the windowed group holds the window and no more; the other group holds everything
    r = Replayer(folder, dtype, max_tokens=256, block_size=8, max_live=4)
    longest = prompts[max(prompts, key=lambda n: len(prompts[n]))]
    r.step([{"id": "x", "tokens": longest[:100], "want": []}], [])
    r.step([{"id": "x", "tokens": longest[100:], "want": [0]}], [])
    assert r.cache.manager.in_use(0) == -(-len(longest) // 8)
    assert r.cache.manager.in_use(1) <= -(-WINDOWED["window"] // 8) + 2
    r.step([], ["x"])
    assert r.cache.manager.in_use(0) == 0 and r.cache.manager.in_use(1) == 0
    # pages that a window gives back cannot be shared between requests: an engine asked to share them says that it does not
    from paged_llm_rs_amd import Engine

    engine = Engine(folder, dtype="f32" if dtype == "float32" else "bf16", block_size=8, num_blocks=64, max_batch=2, chunk=16,
                    prefix_cache=True)
    assert engine.metrics()["prefix_cache"].startswith("off (asked for") and "prefix cache off (asked for" in engine.describe()
    twice = engine.generate([prompts["r1"], prompts["r1"]], max_tokens=4, temperature=0.0, stop_tokens=[])
    assert twice[0]["tokens"] == twice[1]["tokens"] and engine.metrics()["cached_tokens"] == 0


# --- a layer that runs twice, and layers that read another layer's keys and values --------------------------------------

class SharingConfig:
    """Three layers run as 0, 1, 2 (with the keys and values of layer 0), 1 again (with what its first run wrote)."""

    def __init__(self, d):
        self.d = d

    @classmethod
    def from_dict(cls, d):
        return cls(dict(d))

    def to_dict(self):
        return dict(self.d)

    def model_spec(self):
        from paged_llm_rs_amd.config import (AttentionSpec, GatedMlpSpec, LayerSpec, ModelSpec, NormSpec, PositionSpec,
                                             ScheduleEntry)
        d = self.d
        norm = NormSpec("rms_norm", d["rms_norm_eps"])
        ffn = GatedMlpSpec("gated_mlp", d["intermediate_size"], "silu")
        attention = AttentionSpec("paged_attention", d["num_attention_heads"], d["num_key_value_heads"], d["head_dim"], norm,
                                  PositionSpec("rotary_half", d["head_dim"], d["rope_theta"], d["max_position_embeddings"]),
                                  None, None)
        layers = tuple(LayerSpec("pre_norm", attention, ffn, norm, f"model.layers.{i}") for i in range(3))
        schedule = (ScheduleEntry(0), ScheduleEntry(1), ScheduleEntry(2, cache_from=0), ScheduleEntry(1, cache_from=1))
        return ModelSpec(d["hidden_size"], d["vocab_size"], layers, schedule, norm, d["tie_word_embeddings"],
                         d["max_position_embeddings"])


SHARING = {"architectures": ["SharingToyForCausalLM"], "model_type": "sharing_toy", "hidden_size": 48, "intermediate_size": 64,
           "num_attention_heads": 6, "num_key_value_heads": 2, "head_dim": 16, "rms_norm_eps": 1e-5, "rope_theta": 1e4,
           "vocab_size": 89, "max_position_embeddings": 256, "tie_word_embeddings": True}


def sharing_plain(weights, tokens):
    cfg = SHARING
    w = {k: v.double() for k, v in weights.items()}
    n, eps = len(tokens), cfg["rms_norm_eps"]
    nq, nkv, d = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"]
    positions = torch.arange(n)
    held = {}       # layer -> the rotated keys and the values its own run computed

    def attend(x, layer, source):
        p = f"model.layers.{layer}.self_attn"
        q = plain.rms_norm((x @ w[f"{p}.q_proj.weight"].T).reshape(n, nq, d), w[f"{p}.q_norm.weight"], eps)
        q = plain.apply_rope(q, positions, cfg["rope_theta"])
        if source is None:
            k = plain.rms_norm((x @ w[f"{p}.k_proj.weight"].T).reshape(n, nkv, d), w[f"{p}.k_norm.weight"], eps)
            held[layer] = (plain.apply_rope(k, positions, cfg["rope_theta"]), (x @ w[f"{p}.v_proj.weight"].T).reshape(n, nkv, d))
            source = layer
        k, v = held[source]
        out = plain.attention_core(q, plain.repeat_kv(k, nq // nkv), plain.repeat_kv(v, nq // nkv), 1.0 / math.sqrt(d))
        return out.reshape(n, nq * d) @ w[f"{p}.o_proj.weight"].T

    x = w["model.embed_tokens.weight"][torch.tensor(tokens)]
    for layer, source in ((0, None), (1, None), (2, 0), (1, 1)):
        p = f"model.layers.{layer}"
        x = x + attend(plain.rms_norm(x, w[f"{p}.input_layernorm.weight"], eps), layer, source)
        x = x + plain.swiglu_mlp(plain.rms_norm(x, w[f"{p}.post_attention_layernorm.weight"], eps), w, f"{p}.mlp")
    return plain.rms_norm(x, w["model.norm.weight"], eps) @ w["model.embed_tokens.weight"].T


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_layer_that_runs_twice_and_layers_that_read_another_layers_cache(tmp_path, dtype):
    """The order of layers is data: layer 2 has no pages and attends over what layer 0 wrote, layer 1 runs a
    second time over what its first run wrote.  Two layers own pages; every schedule of replay agrees with the
    plain implementation."""
    from safetensors.torch import load_file

    from paged_llm_rs_amd import register_architecture, write_random_model
    from paged_llm_rs_amd.engine.replay import Replayer

    register_architecture("SharingToyForCausalLM", SharingConfig, model_type="sharing_toy")
    folder = write_random_model(tmp_path / "sharing", SHARING, seed=21, std=0.15, gain_std=0.2, dtype=dtype)
    weights = load_file(str(folder / "model.safetensors"))
    prompts = ru.make_prompts(SHARING["vocab_size"], [50, 13, 77, 34], seed=9)
    want = {name: sharing_plain(weights, toks) for name, toks in prompts.items()}
    tolerance = 1e-5 if dtype == "float32" else 2e-2
    for steps, live in ((ru.whole(prompts), 1), (ru.tail_decoded(prompts, 20), 1), (ru.portions(prompts), 1),
                        (ru.mixed(prompts, seed=5, max_live=3), 3)):
        r = Replayer(folder, dtype, max_tokens=ru.pool_tokens(prompts, live), block_size=8, max_live=4)
        assert [g.layers for g in r.cache.layout.groups] == [[0, 1]], "two layers own pages, the third borrows"
        got = ru.collect(r, steps)
        worst, where = ru.worst_error(got, want)
        assert worst <= tolerance, f"{worst:.3e} at {where}"


# --- a toy norm and a toy arrangement of a layer ----------------------------------------------------------------------------

class CenteredNorm:
    """(x - mean) / sqrt(var + eps) * weight + bias over the last axis, in 32-bit."""

    @staticmethod
    def declare(spec, width):
        from paged_llm_rs_amd.weights.loader import ParamDecl
        return [ParamDecl("weight", (width,), "gain"), ParamDecl("bias", (width,), "matrix")]

    def __init__(self, spec, width, params, dtype, device):
        self.eps, self.weight, self.bias = float(spec.eps), params["weight"].float(), params["bias"].float()

    def apply(self, resid, delta, out_dtype, rows=None):
        if delta is not None:
            resid += delta.float()                       # the residual sum: into the 32-bit stream, in place
        x = resid if rows is None else resid[rows.long()]
        centred = x - x.mean(-1, keepdim=True)
        return (centred * torch.rsqrt(centred.pow(2).mean(-1, keepdim=True) + self.eps) * self.weight + self.bias).to(out_dtype)


class ParallelBlock:
    """One norm, then mixer and feed-forward side by side on the same rows: x + mix(n(x)) + ff(n(x))."""

    @classmethod
    def declare(cls, layer, hidden):
        from paged_llm_rs_amd.parts.registry import FEED_FORWARDS, MIXERS, NORMS, lookup, prefixed
        return (prefixed(lookup(NORMS, layer.norm.kind, "norm").declare(layer.norm, hidden), "ln")
                + prefixed(lookup(MIXERS, layer.mixer.kind, "mixer").declare(layer.mixer, hidden), "attn")
                + prefixed(lookup(FEED_FORWARDS, layer.feed_forward.kind, "feed-forward").declare(layer.feed_forward, hidden), "ffn"))

    def __init__(self, layer, hidden, params, dtype, device, shared):
        from paged_llm_rs_amd.parts.registry import FEED_FORWARDS, MIXERS, NORMS, lookup, scoped
        self.dtype = dtype
        self.norm = lookup(NORMS, layer.norm.kind, "norm")(layer.norm, hidden, scoped(params, "ln"), dtype, device)
        self.mixer = lookup(MIXERS, layer.mixer.kind, "mixer")(layer.mixer, hidden, scoped(params, "attn"), dtype, device, shared)
        self.feed_forward = lookup(FEED_FORWARDS, layer.feed_forward.kind, "feed-forward")(
            layer.feed_forward, hidden, scoped(params, "ffn"), dtype, device, shared)

    def forward(self, resid, delta, ctx):
        x = self.norm.apply(resid, delta, self.dtype)
        return self.mixer.forward(x, ctx) + self.feed_forward.forward(x)


class ParallelConfig:
    def __init__(self, d):
        self.d = d

    @classmethod
    def from_dict(cls, d):
        return cls(dict(d))

    def to_dict(self):
        return dict(self.d)

    def model_spec(self):
        from paged_llm_rs_amd.config import (AttentionSpec, GatedMlpSpec, LayerSpec, ModelSpec, NormSpec, PositionSpec,
                                             ScheduleEntry)
        d = self.d
        norm = NormSpec("centered_norm", d["layer_norm_eps"])
        attention = AttentionSpec("paged_attention", d["num_attention_heads"], d["num_key_value_heads"], d["head_dim"], None,
                                  PositionSpec("rotary_half", d["rotary_dim"], d["rope_theta"], d["max_position_embeddings"]),
                                  None, d["attention_scale"])
        ffn = GatedMlpSpec("gated_mlp", d["intermediate_size"], "silu")
        layers = tuple(LayerSpec("parallel", attention, ffn, norm, f"transformer.h.{i}") for i in range(d["num_hidden_layers"]))
        return ModelSpec(d["hidden_size"], d["vocab_size"], layers, tuple(ScheduleEntry(i) for i in range(len(layers))), norm,
                         False, d["max_position_embeddings"], embed_name="transformer.wte.weight",
                         final_norm_name="transformer.ln_f.weight", head_name="lm_head.weight")


PARALLEL = {"architectures": ["ParallelToyForCausalLM"], "model_type": "parallel_toy", "hidden_size": 56, "intermediate_size": 88,
            "num_hidden_layers": 2, "num_attention_heads": 4, "num_key_value_heads": 4, "head_dim": 16, "rotary_dim": 16,
            "attention_scale": 0.3, "layer_norm_eps": 1e-5, "rope_theta": 1e4, "vocab_size": 71,
            "max_position_embeddings": 256}


def parallel_plain(weights, tokens):
    cfg = PARALLEL
    w = {k: v.double() for k, v in weights.items()}
    n, nh, d = len(tokens), cfg["num_attention_heads"], cfg["head_dim"]
    positions = torch.arange(n)

    def norm(x, prefix):
        c = x - x.mean(-1, keepdim=True)
        return c / torch.sqrt(c.pow(2).mean(-1, keepdim=True) + cfg["layer_norm_eps"]) * w[f"{prefix}.weight"] + w[f"{prefix}.bias"]

    x = w["transformer.wte.weight"][torch.tensor(tokens)]
    for i in range(cfg["num_hidden_layers"]):
        p = f"transformer.h.{i}"
        y = norm(x, f"{p}.ln")
        q = plain.apply_rope((y @ w[f"{p}.attn.q_proj.weight"].T).reshape(n, nh, d), positions, cfg["rope_theta"])
        k = plain.apply_rope((y @ w[f"{p}.attn.k_proj.weight"].T).reshape(n, nh, d), positions, cfg["rope_theta"])
        v = (y @ w[f"{p}.attn.v_proj.weight"].T).reshape(n, nh, d)
        mixed = plain.attention_core(q, k, v, cfg["attention_scale"]).reshape(n, nh * d) @ w[f"{p}.attn.o_proj.weight"].T
        x = x + mixed + plain.swiglu_mlp(y, w, f"{p}.ffn")
    return norm(x, "transformer.ln_f") @ w["lm_head.weight"].T


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_toy_norm_and_a_toy_arrangement_of_a_layer(tmp_path, dtype):
    """A norm with a mean and a bias, and a layer whose mixer and feed-forward read the same normalised rows,
    under tensor names of another family, with attention that has no q/k norm, one key head a query head and
    a scale of its own: registered here, built, replayed whole, decoded, in portions and mixed."""
    from safetensors.torch import load_file

    from paged_llm_rs_amd import register_architecture, write_random_model
    from paged_llm_rs_amd.engine.replay import Replayer
    from paged_llm_rs_amd.parts import register_block, register_norm

    register_norm("centered_norm", CenteredNorm)
    register_block("parallel", ParallelBlock)
    register_architecture("ParallelToyForCausalLM", ParallelConfig, model_type="parallel_toy")
    folder = write_random_model(tmp_path / "parallel", PARALLEL, seed=31, std=0.15, gain_std=0.2, dtype=dtype)
    weights = load_file(str(folder / "model.safetensors"))
    assert "transformer.h.1.ln.bias" in weights and "transformer.ln_f.bias" in weights and "lm_head.weight" in weights
    prompts = ru.make_prompts(PARALLEL["vocab_size"], [33, 8, 58, 19], seed=13)
    want = {name: parallel_plain(weights, toks) for name, toks in prompts.items()}
    tolerance = 1e-5 if dtype == "float32" else 2e-2
    for steps, live in ((ru.whole(prompts), 1), (ru.tail_decoded(prompts, 12), 1), (ru.portions(prompts), 1),
                        (ru.mixed(prompts, seed=4, max_live=3), 3)):
        r = Replayer(folder, dtype, max_tokens=ru.pool_tokens(prompts, live), block_size=8, max_live=4)
        got = ru.collect(r, steps)
        worst, where = ru.worst_error(got, want)
        assert worst <= tolerance, f"{worst:.3e} at {where}"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_the_same_arrangement_under_other_tensor_names(tmp_path, model_dirs, dtype):
    """The members of a layer carry this architecture's names unless the layer's spec gives others: the same
    weights under another family's names, through the same block class, give the same bits."""
    import dataclasses
    import json

    from safetensors.torch import load_file, save_file

    from paged_llm_rs_amd.config import register_architecture
    from paged_llm_rs_amd.config.qwen3 import Qwen3Config
    from paged_llm_rs_amd.engine.replay import Replayer
    from paged_llm_rs_amd.errors import ConfigError

    renamed = {"norm1": "ln_1", "mixer": "attn", "norm2": "ln_2", "feed_forward": "ffn"}

    class OtherNamesConfig(Qwen3Config):
        @classmethod
        def from_dict(cls, d):
            return super().from_dict({**d, "model_type": "qwen3", "architectures": ["Qwen3ForCausalLM"]})

        def model_spec(self):
            spec = super().model_spec()
            layers = tuple(dataclasses.replace(layer, names=renamed, weight_prefix=f"transformer.h.{i}")
                           for i, layer in enumerate(spec.layers))
            return dataclasses.replace(spec, layers=layers)

    register_architecture("OtherNamesForCausalLM", OtherNamesConfig, model_type="other_names")
    source = model_dirs("B", dtype)
    config = json.loads((source / "config.json").read_text())
    config.update(architectures=["OtherNamesForCausalLM"], model_type="other_names")
    folder = tmp_path / "other_names"
    folder.mkdir()
    (folder / "config.json").write_text(json.dumps(config))
    standard = {"input_layernorm": "ln_1", "self_attn": "attn", "post_attention_layernorm": "ln_2", "mlp": "ffn"}
    tensors = {}
    for name, tensor in load_file(str(source / "model.safetensors")).items():
        parts = name.split(".")
        if parts[:2] == ["model", "layers"]:
            parts = ["transformer", "h", parts[2], standard[parts[3]]] + parts[4:]
        tensors[".".join(parts)] = tensor
    save_file(tensors, str(folder / "model.safetensors"))
    prompts = ru.make_prompts(config["vocab_size"], [29, 7], seed=3)
    got = [ru.collect(Replayer(d, dtype, max_tokens=ru.pool_tokens(prompts, 1), block_size=8), ru.tail_decoded(prompts, 5))
           for d in (source, folder)]
    assert got[0].keys() == got[1].keys() and len(got[0]) > 10
    for place in got[0]:
        assert np.array_equal(np.asarray(got[0][place]), np.asarray(got[1][place])), place
    with pytest.raises(ConfigError, match="does not have"):
        bad = dataclasses.replace(OtherNamesConfig.from_dict(config).model_spec().layers[0], names={"norm3": "x"})
        from paged_llm_rs_amd.parts.block import PreNormBlock
        PreNormBlock.declare(bad, config["hidden_size"])


# --- toy transforms of the stream behind the embedding and of the logits ------------------------------------------------------

class ScaledEmbeddingWithLearnedPositions:
    """x * scale + table[position]: the table is a tensor of the checkpoint that the transform declares."""

    @staticmethod
    def declare(spec):
        from paged_llm_rs_amd.weights.loader import ParamDecl
        return [ParamDecl("model.embed_positions.weight", (spec.max_positions, spec.hidden_size), "matrix")]

    def __init__(self, spec, params, dtype, device):
        self.scale = float(spec.extra["embed_scale"])
        self.table = params["model.embed_positions.weight"].float()

    def __call__(self, x, batch):
        # (padding rows have position -1; what stands in their rows is never read)
        x.mul_(self.scale).add_(self.table[batch.positions.clamp(min=0).long()])
        return x


class SoftCap:
    """cap * tanh(logits / cap)"""

    def __init__(self, spec, params, dtype, device):
        self.cap = float(spec.extra["logit_cap"])

    def __call__(self, logits, batch):
        return torch.tanh(logits / self.cap) * self.cap


def transformed_config():
    import dataclasses

    from paged_llm_rs_amd.config.qwen3 import Qwen3Config

    class TransformedConfig(Qwen3Config):
        @classmethod
        def from_dict(cls, d):
            self = super().from_dict({**d, "model_type": "qwen3", "architectures": ["Qwen3ForCausalLM"]})
            object.__setattr__(self, "_toy", (d["embed_scale"], d["logit_cap"]))
            return self

        def model_spec(self):
            scale, cap = self._toy
            return dataclasses.replace(super().model_spec(), ignored_tensors=("*.inv_freq",), extra={
                "embed_transform": "scaled_with_learned_positions", "logit_transform": "soft_cap",
                "embed_scale": scale, "logit_cap": cap})

    return TransformedConfig


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_toy_transforms_of_the_embedding_and_of_the_logits(tmp_path, dtype):
    """A scale and a learned position on the stream behind the embedding, a soft cap on the logits, and a
    buffer in the checkpoint that the model does not use: named by the model's spec, registered here, without
    a change to the decoder.  Replayed whole, decoded, in portions and mixed (so also from captured steps)."""
    import json

    from safetensors.torch import load_file, save_file

    from paged_llm_rs_amd import register_architecture, write_random_model
    from paged_llm_rs_amd.engine.replay import Replayer
    from paged_llm_rs_amd.parts import register_embed_transform, register_logit_transform

    register_embed_transform("scaled_with_learned_positions", ScaledEmbeddingWithLearnedPositions)
    register_logit_transform("soft_cap", SoftCap)
    register_architecture("TransformedToyForCausalLM", transformed_config(), model_type="transformed_toy")
    from conftest import TINY_B
    config = {**TINY_B, "architectures": ["TransformedToyForCausalLM"], "model_type": "transformed_toy",
              "embed_scale": 3.0, "logit_cap": 1.0, "max_position_embeddings": 128}
    folder = write_random_model(tmp_path / "transformed", config, seed=5, std=0.05, gain_std=0.2, dtype=dtype)
    weights = load_file(str(folder / "model.safetensors"))
    assert weights["model.embed_positions.weight"].shape == (128, config["hidden_size"])
    stored = dict(weights)
    stored["model.layers.0.self_attn.rotary_emb.inv_freq"] = torch.zeros(16)      # ignored by the spec's pattern
    save_file(stored, str(folder / "model.safetensors"))
    prompts = ru.make_prompts(config["vocab_size"], [41, 9, 77, 20], seed=2)

    def plain_logits(tokens, cap):
        w = {k: v.double() for k, v in weights.items()}
        ids = torch.tensor(tokens)
        positions = torch.arange(len(tokens))
        x = w["model.embed_tokens.weight"][ids] * 3.0 + w["model.embed_positions.weight"][positions]
        for layer in range(config["num_hidden_layers"]):
            x = plain.decoder_block(x, w, f"model.layers.{layer}", config, positions)
        x = plain.rms_norm(x, w["model.norm.weight"], config["rms_norm_eps"])
        logits = x @ plain.lm_head_weight(w, config).T
        return logits if cap is None else torch.tanh(logits / cap) * cap

    # a cap at 0.6 of the largest logit, so that it bends what it caps; it goes into config.json
    largest = max(float(plain_logits(toks, None).abs().max()) for toks in prompts.values())
    cap = round(0.6 * largest, 3)
    config["logit_cap"] = cap
    (folder / "config.json").write_text(json.dumps(config))
    want = {name: plain_logits(toks, cap) for name, toks in prompts.items()}
    assert 0.75 * cap < max(float(v.abs().max()) for v in want.values()) < cap
    tolerance = 1e-5 if dtype == "float32" else 2e-2
    for steps, live in ((ru.whole(prompts), 1), (ru.tail_decoded(prompts, 12), 1), (ru.portions(prompts), 1),
                        (ru.mixed(prompts, seed=9, max_live=3), 3)):
        r = Replayer(folder, dtype, max_tokens=ru.pool_tokens(prompts, live), block_size=8, max_live=4)
        got = ru.collect(r, steps)
        worst, where = ru.worst_error(got, want)
        assert worst <= tolerance, f"{worst:.3e} at {where}"


# --- long decoding, first tokens, long portions -----------------------------------------------------------------------------

@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name,block_size", [("A", 16), ("C", 4)])
def test_long_decoding(model_dirs, name, dtype, block_size):
    """Three hundred tokens decoded one by one, two requests side by side, over many page edges."""
    from paged_llm_rs_amd.engine.replay import Replayer

    d = model_dirs(name, dtype)
    prompts = ru.make_prompts(TINY_INIT[name]["config"]["vocab_size"], [330, 301], seed=21)
    want = ru.plain_logits(d, prompts)
    steps = [{"step": 0, "entries": [{"id": n, "tokens": t[:20 + 11 * i], "want": [19 + 11 * i]}
                                     for i, (n, t) in enumerate(prompts.items())], "end": []}]
    at = {n: 20 + 11 * i for i, n in enumerate(prompts)}
    while at:
        entries = [{"id": n, "tokens": [prompts[n][p]], "want": [0]} for n, p in at.items()]
        at = {n: p + 1 for n, p in at.items()}
        end = [n for n, p in at.items() if p == len(prompts[n])]
        for n in end:
            del at[n]
        steps.append({"step": len(steps), "entries": entries, "end": end})
    r = Replayer(d, dtype, max_tokens=ru.pool_tokens(prompts, 2), block_size=block_size)
    got = ru.collect(r, steps)
    assert r.runner.graph_steps > 250, "decoding runs as captured graphs"
    worst, where = ru.worst_error(got, want)
    assert worst <= (1e-5 if dtype == "float32" else 2e-2), f"{worst:.3e} at {where}"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_the_first_tokens_of_a_sequence(model_dirs, name, dtype):
    """Positions 0, 1, 2, ...: fed one by one from an empty cache, as a portion of two, and whole."""
    from paged_llm_rs_amd.engine.replay import Replayer

    d = model_dirs(name, dtype)
    prompts = ru.make_prompts(TINY_INIT[name]["config"]["vocab_size"], [6, 1, 2, 3], seed=8)
    want = ru.plain_logits(d, prompts)
    one_by_one = []
    for n, t in prompts.items():
        for p, token in enumerate(t):
            one_by_one.append({"step": len(one_by_one), "entries": [{"id": n, "tokens": [token], "want": [0]}],
                               "end": [n] if p == len(t) - 1 else []})
    for steps in (one_by_one, ru.portions(prompts, sizes=(2, 1, 3)), ru.whole(prompts)):
        r = Replayer(d, dtype, max_tokens=64, block_size=4)
        worst, where = ru.worst_error(ru.collect(r, steps), want)
        assert worst <= (1e-5 if dtype == "float32" else 2e-2), f"{worst:.3e} at {where}"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name,block_size", [("A", 16), ("B", 8)])
def test_long_portions_over_earlier_context(model_dirs, name, dtype, block_size):
    """Portions of more than a hundred tokens that read hundreds of earlier keys through the pages (the tiled
    attention kernel's case in bfloat16), beside a request that decodes."""
    from paged_llm_rs_amd.engine.replay import Replayer

    d = model_dirs(name, dtype)
    prompts = ru.make_prompts(TINY_INIT[name]["config"]["vocab_size"], [450, 40], seed=31)
    want = ru.plain_logits(d, prompts)
    long, short = prompts["r0"], prompts["r1"]
    cuts = [0, 130, 131, 300, 429, 450]
    steps = [{"step": 0, "entries": [{"id": "r1", "tokens": short[:30], "want": [29]}], "end": []}]
    for i in range(len(cuts) - 1):
        a, b = cuts[i], cuts[i + 1]
        entries = [{"id": "r0", "tokens": long[a:b], "want": sorted({0, (b - a) // 2, b - a - 1})}]
        if 30 + i < len(short):
            entries.append({"id": "r1", "tokens": [short[30 + i]], "want": [0]})
        steps.append({"step": len(steps), "entries": entries, "end": ["r0"] if b == len(long) else []})
    steps.append({"step": len(steps), "entries": [{"id": "r1", "tokens": short[35:], "want": [0, 4]}], "end": ["r1"]})
    r = Replayer(d, dtype, max_tokens=ru.pool_tokens(prompts, 2), block_size=block_size)
    worst, where = ru.worst_error(ru.collect(r, steps), want)
    assert worst <= (1e-5 if dtype == "float32" else 2e-2), f"{worst:.3e} at {where}"


@pytest.mark.parametrize("name,total,dtype", [("D", 2600, "bfloat16"), ("L", 4240, "bfloat16"), ("L", 4240, "float32")])
def test_a_context_of_thousands_of_tokens_in_portions_and_decoded(model_dirs, name, total, dtype):
    """The 0.6B layer sizes over 2,600 and over 4,240 tokens (the context the benchmark decodes from): portions
    of 512 whose keys are dealt to several workgroups a token tile, block tables that outgrow their first width,
    then 40 single tokens whose keys are cut into many shares, beside a second request that decodes all along.
    (The plain implementation does its 64-bit arithmetic on the GPU here: thousands of tokens take it a minute
    on the CPU.)"""
    from paged_llm_rs_amd.engine.replay import Replayer

    d = model_dirs(name, dtype)
    prompts = ru.make_prompts(TINY_INIT[name]["config"]["vocab_size"], [total, 90], seed=41)
    want = ru.plain_logits(d, prompts, device="cuda:0")
    long, short = prompts["r0"], prompts["r1"]
    steps = [{"step": 0, "entries": [{"id": "r1", "tokens": short[:40], "want": [39]}], "end": []}]
    fed, at, portions_end = 40, 0, total - 40
    while at < portions_end:
        count = min(512, portions_end - at)
        entries = [{"id": "r0", "tokens": long[at:at + count], "want": [0, count - 1]}]
        if fed < len(short):
            entries.append({"id": "r1", "tokens": [short[fed]], "want": [0]})
            fed += 1
        steps.append({"step": len(steps), "entries": entries, "end": []})
        at += count
    for i in range(portions_end, total):
        entries = [{"id": "r0", "tokens": [long[i]], "want": [0]}]
        if fed < len(short):
            entries.append({"id": "r1", "tokens": [short[fed]], "want": [0]})
            fed += 1
        steps.append({"step": len(steps), "entries": entries, "end": ["r0"] if i == total - 1 else []})
    steps.append({"step": len(steps), "entries": [{"id": "r1", "tokens": short[fed:], "want": [0]}], "end": ["r1"]})
    r = Replayer(d, dtype, max_tokens=ru.pool_tokens(prompts, 2), block_size=16)
    got = ru.collect(r, steps)
    assert len(got) >= 2 * 5 + 40 + 40
    worst, where = ru.worst_error(got, want)
    assert worst <= (1e-5 if dtype == "float32" else 2e-2), f"{worst:.3e} at {where}"
