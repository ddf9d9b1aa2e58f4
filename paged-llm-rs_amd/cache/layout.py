"""What the layers of a model need from the cache, grouped.

Every mixer says what pages it needs (heads, head size, window) and what
fixed-size state it keeps for each request.  Layers with the same page needs
form a group: they share page numbers (one block table for the group) while
each layer has pools of its own.  A layer that reads another layer's cache has
no pools.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Optional

import torch

from ..errors import ConfigError


@dataclass(frozen=True)
class KVCacheSpec:
    """Keys and values of ``kv_heads`` heads of ``head_dim``; with a window only
    the last ``window`` positions are ever read."""
    kv_heads: int
    head_dim: int
    window: Optional[int] = None


@dataclass(frozen=True)
class StateSpec:
    """A tensor of fixed shape kept for each live request."""
    shape: tuple
    dtype: torch.dtype = torch.float32


@dataclass
class CacheGroupLayout:
    spec: KVCacheSpec
    layers: list          # layer indices that own pools in this group


class CacheLayout:
    def __init__(self, groups: list, layer_group: dict, states: dict):
        self.groups = groups            # [CacheGroupLayout]
        self.layer_group = layer_group  # layer index -> group index (layers that own pools)
        self.states = states            # layer index -> StateSpec

    @classmethod
    def from_blocks(cls, blocks, schedule) -> "CacheLayout":
        # A run of a layer either owns its cache or reads the one another run has written earlier in the
        # same pass.  Two owning runs of one layer would write the same pages twice, and what a later step
        # reads there would depend on how the tokens were cut into steps: refused.
        def spec_of(index):
            mixer = getattr(blocks[index], "mixer", None)
            return (mixer.cache_spec(), mixer.state_spec()) if mixer is not None else (None, None)

        written: set = set()
        for at, e in enumerate(schedule):
            kv, state = spec_of(e.layer)
            if e.cache_from is None:
                if e.layer in written and (kv is not None or state is not None):
                    raise ConfigError(f"the schedule runs layer {e.layer} twice with a cache of its own; the second run "
                                      f"can read what the first wrote (cache_from={e.layer})")
                written.add(e.layer)
            else:
                if e.cache_from not in written:
                    raise ConfigError(f"run {at} of the schedule reads the cache of layer {e.cache_from}, which no "
                                      "earlier run of the pass has written")
                if state is not None:
                    raise ConfigError(f"layer {e.layer} keeps a state of its own and cannot read another layer's cache")
                if spec_of(e.cache_from)[0] != kv:
                    raise ConfigError(f"layer {e.layer} reads the cache of layer {e.cache_from}, whose keys and values "
                                      "have another shape or window")
        owners = sorted(written)
        groups: list = []
        layer_group: dict = {}
        states: dict = {}
        for index in owners:
            mixer = getattr(blocks[index], "mixer", None)
            spec = mixer.cache_spec() if mixer is not None else None
            if spec is not None:
                for g, group in enumerate(groups):
                    if group.spec == spec:
                        group.layers.append(index)
                        layer_group[index] = g
                        break
                else:
                    groups.append(CacheGroupLayout(spec, [index]))
                    layer_group[index] = len(groups) - 1
            state = mixer.state_spec() if mixer is not None else None
            if state is not None:
                states[index] = state
        return cls(groups, layer_group, states)

    def bytes_per_token(self, element_size: int) -> int:
        """Bytes of keys and values one token takes over all layers
        (reference: batch.rs:43-46)."""
        return sum(2 * len(g.layers) * g.spec.kv_heads * g.spec.head_dim * element_size for g in self.groups)

    def blocks_within(self, budget_bytes: int, block_size: int, element_size: int) -> int:
        """Pages a byte budget holds, at least one (reference: batch.rs:54-57)."""
        per_block = block_size * self.bytes_per_token(element_size)
        return max(budget_bytes // max(per_block, 1), 1)
