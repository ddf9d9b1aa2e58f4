"""Rotary position tables (reference: model/rope.rs:32-63).

The angle position * theta^(-2i/dim) is computed in 64-bit on the host and the
tables are kept in 32-bit whatever the model's type is; the half table is stored
once, [max_positions, dim/2], since both halves of a head use the same angles.
"""

from __future__ import annotations

import torch

from ..errors import UnsupportedError
from .registry import POSITIONS, lookup, register_position


class RotaryTables:
    # which elements of a head an angle turns: i and i + dim/2 (False), or 2 i and 2 i + 1 (True)
    neighbours = False

    def __init__(self, spec, device):
        if spec.dim % 2 or spec.dim <= 0:
            raise UnsupportedError(f"a rotation over {spec.dim} values, which do not pair")
        self.dim = spec.dim
        half = spec.dim // 2
        inv = torch.tensor([1.0 / (spec.theta ** (2.0 * i / spec.dim)) for i in range(half)], dtype=torch.float64)
        angle = torch.arange(spec.max_positions, dtype=torch.float64)[:, None] * inv[None, :]
        self.cos = angle.cos().to(torch.float32).to(device).contiguous()
        self.sin = angle.sin().to(torch.float32).to(device).contiguous()
        self.max_positions = spec.max_positions


class RotaryNeighbourTables(RotaryTables):
    """The same angles, turning neighbouring elements: the layout of checkpoints that were not permuted for
    the half-split form."""
    neighbours = True


register_position("rotary_half", RotaryTables)
register_position("rotary_neighbours", RotaryNeighbourTables)


def rotary_tables(spec, device, shared: dict):
    """The tables of a position spec, built by the class its ``kind`` names; layers
    with the same spec share one pair."""
    key = ("position", spec, str(device))
    if key not in shared:
        shared[key] = lookup(POSITIONS, spec.kind, "position encoding")(spec, device)
    return shared[key]
