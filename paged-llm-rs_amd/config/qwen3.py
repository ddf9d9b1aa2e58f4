"""The typed Qwen3 configuration, read from the keys of its own config.json.

Fields the engine does not honour are parsed and then refused, because a model
that silently ignores a sliding window or a bias runs, generates fluent text
and is wrong (reference: config.rs:1-7, 87-131).
"""

from __future__ import annotations

import json
import math
from dataclasses import dataclass
from pathlib import Path
from typing import Optional

from ..errors import ConfigError, IoError, UnsupportedError
from .specs import (AttentionSpec, GatedMlpSpec, LayerSpec, ModelSpec, NormSpec, PositionSpec,
                    ScheduleEntry)

_REQUIRED = (
    "hidden_size", "intermediate_size", "num_hidden_layers", "num_attention_heads",
    "num_key_value_heads", "head_dim", "rms_norm_eps", "vocab_size",
    "max_position_embeddings", "tie_word_embeddings", "model_type", "hidden_act",
)


def _integer(d: dict, key: str) -> int:
    v = d[key]
    if isinstance(v, bool) or not isinstance(v, int) or v <= 0:
        raise ConfigError(f"{key} {v!r}, which has to be a positive integer")
    return v


@dataclass(frozen=True)
class Qwen3Config:
    """Architecture of a Qwen3 dense model (reference: config.rs:18-66)."""

    hidden_size: int
    intermediate_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    rms_norm_eps: float
    vocab_size: int
    max_position_embeddings: int
    tie_word_embeddings: bool
    model_type: str
    hidden_act: str
    rope_theta: float
    attention_bias: bool = False
    sliding_window: Optional[int] = None

    architecture = "Qwen3ForCausalLM"

    # -- reading ---------------------------------------------------------------

    @classmethod
    def from_file(cls, path) -> "Qwen3Config":
        return cls.from_dict(read_json(path))

    @classmethod
    def from_dict(cls, d: dict) -> "Qwen3Config":
        missing = [k for k in _REQUIRED if k not in d]
        if missing:
            raise ConfigError("config.json lacks " + ", ".join(missing))
        refuse = UnsupportedError
        # Refusals in the reference's order (config.rs:87-131).
        if d["model_type"] != "qwen3":
            raise refuse(f"model_type {d['model_type']!r}, only qwen3 is implemented")
        if d["hidden_act"] != "silu":
            raise refuse(f"hidden_act {d['hidden_act']!r}, only silu is implemented")
        if d.get("attention_bias", False):
            raise refuse("attention_bias, the projections here carry no bias")
        if d.get("sliding_window") is not None:
            raise refuse(f"sliding_window {d['sliding_window']}, attention here is dense")
        if d.get("rope_scaling") is not None:
            raise refuse("rope_scaling, the rotary table here is unscaled")
        nested = d.get("rope_parameters")
        if nested is not None and not isinstance(nested, dict):
            raise ConfigError(f"rope_parameters {nested!r}, which has to be an object")
        if nested is not None and nested.get("rope_type") not in (None, "default"):
            raise refuse(f"rope_type {nested.get('rope_type')!r}, the rotary table here is unscaled")
        if d.get("rope_theta") is not None:
            theta = d["rope_theta"]
        elif nested is not None and nested.get("rope_theta") is not None:
            theta = nested["rope_theta"]
        else:
            raise ConfigError("no rope_theta, in either the flat or the nested layout")
        if isinstance(theta, bool) or not isinstance(theta, (int, float)) or not theta > 0:
            raise ConfigError(f"rope_theta {theta!r}, which has to be a positive number")
        eps = d["rms_norm_eps"]
        if isinstance(eps, bool) or not isinstance(eps, (int, float)) or eps < 0 or not math.isfinite(eps):
            raise ConfigError(f"rms_norm_eps {eps!r}, which has to be a number of zero or above")
        if not isinstance(d["tie_word_embeddings"], bool):
            raise ConfigError(f"tie_word_embeddings {d['tie_word_embeddings']!r}, which has to be true or false")
        ints = {k: _integer(d, k) for k in _REQUIRED[:6] + ("vocab_size", "max_position_embeddings")}
        if ints["num_attention_heads"] % ints["num_key_value_heads"] != 0:
            raise refuse(
                f"{ints['num_attention_heads']} query heads over {ints['num_key_value_heads']} "
                "key heads, which do not group evenly"
            )
        if ints["head_dim"] % 2 != 0:
            raise refuse(f"head_dim {ints['head_dim']}, the rotation pairs the two halves of a head")
        return cls(
            rms_norm_eps=float(eps), tie_word_embeddings=d["tie_word_embeddings"],
            model_type=d["model_type"], hidden_act=d["hidden_act"], rope_theta=float(theta),
            attention_bias=False, sliding_window=None, **ints,
        )

    # -- derived widths (config.rs:148-160) ---------------------------------------

    @property
    def kv_group_size(self) -> int:
        return self.num_attention_heads // self.num_key_value_heads

    @property
    def query_width(self) -> int:
        return self.num_attention_heads * self.head_dim

    @property
    def kv_width(self) -> int:
        return self.num_key_value_heads * self.head_dim

    # -- the model this configuration describes ---------------------------------

    def model_spec(self) -> ModelSpec:
        """Every layer is the same here; the list form is what lets another
        architecture give different layers different parts."""
        norm = NormSpec("rms_norm", self.rms_norm_eps)
        position = PositionSpec("rotary_half", self.head_dim, self.rope_theta,
                                self.max_position_embeddings)
        layers = tuple(
            LayerSpec(
                block="pre_norm",
                mixer=AttentionSpec(
                    num_heads=self.num_attention_heads, num_kv_heads=self.num_key_value_heads,
                    head_dim=self.head_dim, qk_norm=norm, position=position, window=None,
                    scale=None,
                ),
                feed_forward=GatedMlpSpec(intermediate_size=self.intermediate_size,
                                          activation=self.hidden_act),
                norm=norm,
                weight_prefix=f"model.layers.{i}",
            )
            for i in range(self.num_hidden_layers)
        )
        return ModelSpec(
            hidden_size=self.hidden_size, vocab_size=self.vocab_size, layers=layers,
            schedule=tuple(ScheduleEntry(i) for i in range(self.num_hidden_layers)),
            final_norm=norm, tie_word_embeddings=self.tie_word_embeddings,
            max_positions=self.max_position_embeddings,
        )

    def to_dict(self) -> dict:
        """The config.json this configuration would be read back from."""
        return {
            "architectures": [self.architecture], "model_type": self.model_type,
            "hidden_act": self.hidden_act, "attention_bias": False, "sliding_window": None,
            "hidden_size": self.hidden_size, "intermediate_size": self.intermediate_size,
            "num_hidden_layers": self.num_hidden_layers,
            "num_attention_heads": self.num_attention_heads,
            "num_key_value_heads": self.num_key_value_heads, "head_dim": self.head_dim,
            "rms_norm_eps": self.rms_norm_eps, "rope_theta": self.rope_theta,
            "vocab_size": self.vocab_size,
            "max_position_embeddings": self.max_position_embeddings,
            "tie_word_embeddings": self.tie_word_embeddings,
        }


def read_json(path) -> dict:
    path = Path(path)
    try:
        text = path.read_text()
    except OSError as e:
        raise IoError(f"reading {path}: {e}") from e
    try:
        value = json.loads(text)
    except json.JSONDecodeError as e:
        raise ConfigError(f"{path}: {e}") from e
    if not isinstance(value, dict):
        raise ConfigError(f"{path}: not a JSON object")
    return value
