"""The random-weights mode: a model folder from a configuration and a seed.

Linear and embedding weights are N(0, std), norm gains are 1 + N(0, gain_std)
so that a dropped gain cannot pass (the reference's fixture generator does the
same with a uniform gain, scripts/dump_reference.py:229-244).  Every tensor has
a generator of its own, seeded from (seed, tensor name), so a tensor's values do
not depend on which other tensors the model has.
"""

from __future__ import annotations

import json
from pathlib import Path

import torch

from ..config import load_config
from ..errors import ConfigError
from .safetensors_io import write_safetensors

_MASK = (1 << 64) - 1


def _tensor_seed(seed: int, name: str) -> int:
    h = 0xCBF29CE484222325
    for byte in name.encode():
        h = ((h ^ byte) * 0x100000001B3) & _MASK
    z = (h + (seed & _MASK) * 0x9E3779B97F4A7C15 + 0x9E3779B97F4A7C15) & _MASK
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & _MASK
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & _MASK
    return (z ^ (z >> 31)) & ((1 << 63) - 1)


def random_tensor(name: str, shape, role: str, seed: int, std: float, gain_std: float,
                  dtype: torch.dtype) -> torch.Tensor:
    g = torch.Generator(device="cpu")
    g.manual_seed(_tensor_seed(seed, name))
    x = torch.randn(tuple(shape), generator=g, dtype=torch.float32)
    if role == "gain":
        x = 1.0 + x * gain_std
    else:
        x = x * std
    return x.to(dtype)


def write_random_model(out_dir, config, seed: int = 0, std: float = 0.02, gain_std: float = 0.1,
                       dtype="bfloat16") -> Path:
    """Write ``config.json`` and ``model.safetensors`` into ``out_dir``.

    ``config`` is a dict of config.json keys or a typed configuration.  The
    tensors are the ones the registered model declares for it.
    """
    from ..parts.model import declare_parameters

    dtypes = {"bfloat16": torch.bfloat16, "float32": torch.float32, "bf16": torch.bfloat16,
              "f32": torch.float32, torch.bfloat16: torch.bfloat16, torch.float32: torch.float32}
    if dtype not in dtypes:
        raise ConfigError(f"dtype {dtype!r}, which is neither bfloat16 nor float32")
    torch_dtype = dtypes[dtype]
    config_dict = config if isinstance(config, dict) else config.to_dict()
    typed = load_config(config_dict)
    decls = [d for d in declare_parameters(typed.model_spec())
             if not (d.optional and typed.model_spec().tie_word_embeddings)]
    out_dir = Path(out_dir)
    out_dir.mkdir(parents=True, exist_ok=True)
    (out_dir / "config.json").write_text(json.dumps(config_dict, indent=2) + "\n")
    items = [
        (d.name, tuple(d.shape), torch_dtype,
         (lambda d=d: random_tensor(d.name, d.shape, d.role, seed, std, gain_std, torch_dtype)))
        for d in decls
    ]
    write_safetensors(out_dir / "model.safetensors", items,
                      metadata={"format": "pt", "seed": seed, "std": std, "gain_std": gain_std})
    return out_dir
