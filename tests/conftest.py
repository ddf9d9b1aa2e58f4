"""Shared fixtures: the import path, the ``gpu`` marker, tiny configurations and
random model folders made in temporary directories."""

from __future__ import annotations

import json
import os
import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))
if str(ROOT / "tests") not in sys.path:
    sys.path.insert(0, str(ROOT / "tests"))

# The reference's own tiny checkpoint with the activations it holds for it, read in place; where the
# reference lies elsewhere (a machine that has only a copy of that folder), the variable names the folder.
REFERENCE_FIXTURE = Path(os.environ.get("PAGEDLLM_REFERENCE_FIXTURE", "/root/reference/crates/pagedllm/tests/fixtures/tiny"))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def pytest_collection_modifyitems(config, items):
    """GPU tests are skipped where there is no GPU, so a plain ``pytest`` run
    on a CPU-only machine stays green."""
    import torch

    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no GPU in this machine")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


# Two tiny configurations of the architecture that differ in every size and
# option: layers, width, heads, groups (GQA 2 against MQA 6), head size (equal to
# and different from width/heads), feed-forward width, vocabulary, rotary base,
# eps, tied against untied head, and the two layouts of the rotary base.
TINY_A = {
    "architectures": ["Qwen3ForCausalLM"],
    "model_type": "qwen3",
    "hidden_act": "silu",
    "attention_bias": False,
    "sliding_window": None,
    "hidden_size": 64,
    "intermediate_size": 128,
    "num_hidden_layers": 2,
    "num_attention_heads": 4,
    "num_key_value_heads": 2,
    "head_dim": 16,
    "rms_norm_eps": 1e-6,
    "rope_theta": 10000.0,
    "vocab_size": 256,
    "max_position_embeddings": 512,
    "tie_word_embeddings": True,
}

TINY_B = {
    "architectures": ["Qwen3ForCausalLM"],
    "model_type": "qwen3",
    "hidden_act": "silu",
    "attention_bias": False,
    "sliding_window": None,
    "hidden_size": 96,
    "intermediate_size": 160,
    "num_hidden_layers": 3,
    "num_attention_heads": 6,
    "num_key_value_heads": 1,
    "head_dim": 32,
    "rms_norm_eps": 1e-5,
    "rope_parameters": {"rope_theta": 1000000.0, "rope_type": "default"},
    "vocab_size": 384,
    "max_position_embeddings": 1024,
    "tie_word_embeddings": False,
}

# Widths that are no multiple of eight, a head of 48, a group of three and a
# vocabulary that is no multiple of anything: the sizes kernels like least.
TINY_C = {
    "architectures": ["Qwen3ForCausalLM"],
    "model_type": "qwen3",
    "hidden_act": "silu",
    "attention_bias": False,
    "hidden_size": 100,
    "intermediate_size": 212,
    "num_hidden_layers": 2,
    "num_attention_heads": 6,
    "num_key_value_heads": 2,
    "head_dim": 48,
    "rms_norm_eps": 1e-6,
    "rope_theta": 500000.0,
    "vocab_size": 331,
    "max_position_embeddings": 2048,
    "tie_word_embeddings": False,
}

# The layer sizes of Qwen3-0.6B (the sizes the kernels are tuned for: heads of 128, pages of 16), two
# layers of them, with a vocabulary that is no multiple of anything.
LAYERS_0P6B = {
    "architectures": ["Qwen3ForCausalLM"],
    "model_type": "qwen3",
    "hidden_act": "silu",
    "attention_bias": False,
    "sliding_window": None,
    "hidden_size": 1024,
    "intermediate_size": 3072,
    "num_hidden_layers": 2,
    "num_attention_heads": 16,
    "num_key_value_heads": 8,
    "head_dim": 128,
    "rms_norm_eps": 1e-6,
    "rope_theta": 1000000.0,
    "vocab_size": 4099,
    "max_position_embeddings": 4096,
    "tie_word_embeddings": True,
}

# Layer sizes in the manner of the family's larger models, two layers of them: eight query heads a key
# head (single tokens then go through the tiled attention kernel, a group's heads as its rows), a width
# beyond what the product kernel normalises on the way in, and weights large enough that products of
# few rows go to the library.
LAYERS_WIDE = {
    "architectures": ["Qwen3ForCausalLM"],
    "model_type": "qwen3",
    "hidden_act": "silu",
    "attention_bias": False,
    "sliding_window": None,
    "hidden_size": 2560,
    "intermediate_size": 6912,
    "num_hidden_layers": 2,
    "num_attention_heads": 16,
    "num_key_value_heads": 2,
    "head_dim": 128,
    "rms_norm_eps": 1e-5,
    "rope_theta": 1000000.0,
    "vocab_size": 3001,
    "max_position_embeddings": 4096,
    "tie_word_embeddings": False,
}

# The same two layers under the family's real vocabulary, tied: the projection onto it walks its column
# tiles in a loop (few rows) or goes to the library (many), which no smaller vocabulary shows.
LAYERS_0P6B_REAL_VOCAB = dict(LAYERS_0P6B, vocab_size=151936)

# ... and with room for contexts beyond four thousand tokens.
LAYERS_0P6B_LONG = dict(LAYERS_0P6B, max_position_embeddings=8192)

TINY_INIT = {
    "A": dict(config=TINY_A, seed=0, std=0.02, gain_std=0.1),
    "B": dict(config=TINY_B, seed=1, std=0.05, gain_std=0.2),
    "C": dict(config=TINY_C, seed=2, std=0.08, gain_std=0.2),
    "D": dict(config=LAYERS_0P6B, seed=3, std=0.02, gain_std=0.1),
    "E": dict(config=LAYERS_WIDE, seed=4, std=0.02, gain_std=0.1),
    "V": dict(config=LAYERS_0P6B_REAL_VOCAB, seed=5, std=0.02, gain_std=0.1),
    "L": dict(config=LAYERS_0P6B_LONG, seed=6, std=0.02, gain_std=0.1),
}


def make_model_dir(tmp_path_factory, name: str, dtype: str = "float32") -> Path:
    """Write a random tiny model folder with the framework's random-weights mode."""
    from paged_llm_rs_amd.weights import write_random_model

    spec = TINY_INIT[name]
    out = tmp_path_factory.mktemp(f"tiny_{name}_{dtype}")
    write_random_model(out, spec["config"], seed=spec["seed"], std=spec["std"],
                       gain_std=spec["gain_std"], dtype=dtype)
    return out


@pytest.fixture(scope="session")
def model_dirs(tmp_path_factory):
    """Model folders by (name, dtype), made on first use."""
    made: dict[tuple[str, str], Path] = {}

    def get(name: str, dtype: str = "float32") -> Path:
        key = (name, dtype)
        if key not in made:
            made[key] = make_model_dir(tmp_path_factory, name, dtype)
        return made[key]

    return get


def load_plain(model_dir: Path):
    """Config dict and tensor dict for the plain implementation, read with the
    library loader (not the framework's own reader)."""
    from safetensors.torch import load_file

    cfg = json.loads((Path(model_dir) / "config.json").read_text())
    weights = load_file(str(Path(model_dir) / "model.safetensors"))
    return cfg, weights


def rel_err(got, want) -> float:
    """max|got-want| / max|want| with an exact shape check first
    (the reference's metric, tests/common/mod.rs:20-43, without its floor of 1)."""
    import torch

    got = torch.as_tensor(got).double().cpu()
    want = torch.as_tensor(want).double().cpu()
    assert tuple(got.shape) == tuple(want.shape), f"shape {tuple(got.shape)} against {tuple(want.shape)}"
    scale = want.abs().max().item()
    return (got - want).abs().max().item() / max(scale, 1e-30)
