"""The device side of the cache: for every layer that owns pages a key pool and
a value pool, [pages * page size, kv_heads * head_dim], allocated once and never
grown (reference: batch.rs:279-315); and for every layer with per-request state
a tensor [slots, ...].  Page numbers are shared by the layers of a group.
"""

from __future__ import annotations

from dataclasses import dataclass

import torch

from ..errors import ConfigError
from .layout import CacheLayout
from .manager import CacheManager, GroupGeometry


@dataclass
class LayerKV:
    """What an attention kernel needs of one layer's pages in one step."""
    k_pool: torch.Tensor
    v_pool: torch.Tensor
    block_table: torch.Tensor   # [requests of the step, pages a request], -1 where there is none
    block_size: int
    group: int


class PagedCache:
    def __init__(self, layout: CacheLayout, block_size: int, num_blocks: int, dtype: torch.dtype,
                 device, max_seqs: int = 64):
        if block_size < 1:
            raise ConfigError(f"block size {block_size}, which has to be at least one")
        if num_blocks < 1:
            raise ConfigError(f"a pool of {num_blocks} pages")
        self.layout = layout
        self.block_size = block_size
        self.num_blocks = num_blocks
        self.dtype = dtype
        self.device = torch.device(device)
        self.max_seqs = max_seqs
        geometry = [GroupGeometry(block_size, num_blocks, int(g.spec.window or 0)) for g in layout.groups]
        self.manager = CacheManager(geometry, state_slots=max_seqs if layout.states else 0)
        self._pools: dict = {}
        for g in layout.groups:
            width = g.spec.kv_heads * g.spec.head_dim
            for layer in g.layers:
                self._pools[layer] = (
                    torch.zeros((num_blocks * block_size, width), dtype=dtype, device=self.device),
                    torch.zeros((num_blocks * block_size, width), dtype=dtype, device=self.device),
                )
        self._states = {
            layer: torch.zeros((max_seqs, *spec.shape), dtype=spec.dtype, device=self.device)
            for layer, spec in layout.states.items()
        }

    @property
    def bytes(self) -> int:
        return sum(k.numel() * k.element_size() * 2 for k, _ in self._pools.values())

    def layer_view(self, layer: int, batch) -> LayerKV:
        if layer not in self._pools:
            raise ConfigError(f"layer {layer} owns no pages")
        group = self.layout.layer_group[layer]
        k, v = self._pools[layer]
        return LayerKV(k, v, batch.block_tables[group], self.block_size, group)

    def layer_pools(self, layer: int):
        return self._pools[layer]

    def layer_state(self, layer: int) -> torch.Tensor:
        if layer not in self._states:
            raise ConfigError(f"layer {layer} keeps no state")
        return self._states[layer]

    def clear_state_slot(self, slot: int) -> None:
        """A slot is cleared before a new request uses it."""
        for state in self._states.values():
            state[slot].zero_()
