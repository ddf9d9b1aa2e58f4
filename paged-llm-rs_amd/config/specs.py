"""Descriptions of the parts a model is put together from.

A spec is plain data: a ``kind`` that names an entry of the part registry and
the sizes and constants that part needs.  A model is a list of layer specs plus
the order in which the layers run; nothing in a spec says which architecture it
came from, and nothing in a part reads anything but its own spec.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Optional


@dataclass(frozen=True)
class NormSpec:
    """A normalisation over the last axis."""
    kind: str = "rms_norm"
    eps: float = 1e-6


@dataclass(frozen=True)
class PositionSpec:
    """How positions enter a mixer.  ``rotary_half`` rotates the pairs
    (i, i + dim/2) of each head by position * theta^(-2i/dim)."""
    kind: str = "rotary_half"
    dim: int = 0
    theta: float = 10000.0
    max_positions: int = 0


@dataclass(frozen=True)
class AttentionSpec:
    """Grouped-query attention over a paged cache."""
    kind: str = "paged_attention"
    num_heads: int = 0
    num_kv_heads: int = 0
    head_dim: int = 0
    qk_norm: Optional[NormSpec] = None      # per-head norm on q and k before the position encoding
    position: Optional[PositionSpec] = None
    window: Optional[int] = None            # keys j with pos - window < j <= pos; None = all keys
    scale: Optional[float] = None           # None = 1/sqrt(head_dim)
    qkv_bias: bool = False                  # q, k and v projections carry a bias each
    out_bias: bool = False                  # the output projection carries one


@dataclass(frozen=True)
class GatedMlpSpec:
    """down(act(gate(x)) * up(x))."""
    kind: str = "gated_mlp"
    intermediate_size: int = 0
    activation: str = "silu"


@dataclass(frozen=True)
class LayerSpec:
    """One layer: which block arrangement, and its mixer, feed-forward and norm."""
    block: str = "pre_norm"
    mixer: Any = None
    feed_forward: Any = None
    norm: Any = None
    weight_prefix: str = ""
    names: Optional[dict] = None            # other tensor-name parts for the block's members (norm1, mixer, norm2, feed_forward)


@dataclass(frozen=True)
class ScheduleEntry:
    """One step of the order in which layers run.  A layer may appear twice;
    ``cache_from`` lets this run read the cache another layer wrote instead of
    writing its own."""
    layer: int
    cache_from: Optional[int] = None


@dataclass(frozen=True)
class ModelSpec:
    """Everything the generic decoder needs, independent of the architecture."""
    hidden_size: int
    vocab_size: int
    layers: tuple
    schedule: tuple
    final_norm: Any
    tie_word_embeddings: bool
    max_positions: int
    embed_name: str = "model.embed_tokens.weight"
    final_norm_name: str = "model.norm.weight"
    head_name: str = "lm_head.weight"
    # Tensors a checkpoint of this family carries and the model does not use (buffers, tables that are
    # computed here): shell patterns over tensor names, e.g. "*.rotary_emb.inv_freq".  They are neither
    # loaded nor reported as unexpected.
    ignored_tensors: tuple = ()
    # What the decoder does beside the layers, by the names of registered transforms:
    # ``extra["embed_transform"]`` is applied to the 32-bit stream right after the embedding gather (a scale,
    # a learned position added to it), ``extra["logit_transform"]`` to the 32-bit logits (a soft cap, a
    # scale).  Each transform reads its own constants from ``extra`` too.  None of the two by default.
    extra: dict = field(default_factory=dict)
