"""The gated feed-forward: down(silu(gate(x)) * up(x)), the activation on the
gate branch (reference: model/layers.rs:72-107)."""

from __future__ import annotations

import torch

from .. import kernels
from ..errors import UnsupportedError
from ..weights.loader import ParamDecl
from .linear import Linear
from .registry import register_feed_forward


class GatedMlp:
    @staticmethod
    def declare(spec, hidden: int) -> list:
        i = spec.intermediate_size
        return [ParamDecl("gate_proj.weight", (i, hidden)), ParamDecl("up_proj.weight", (i, hidden)),
                ParamDecl("down_proj.weight", (hidden, i))]

    def __init__(self, spec, hidden: int, params: dict, dtype, device, shared: dict):
        if spec.activation != "silu":
            raise UnsupportedError(f"activation {spec.activation!r}, only silu is implemented")
        # one product for gate and up: the output row is [gate | up]
        self.gate_up_proj = Linear.fused([params["gate_proj.weight"], params["up_proj.weight"]])
        self.down_proj = Linear(params["down_proj.weight"])

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        if kernels.skinny_applies(x):
            # few rows: the activation is the epilogue of the weight stream
            act = kernels.gemm_skinny(x, self.gate_up_proj.weight, swiglu=True)
        else:
            act = kernels.swiglu(self.gate_up_proj.forward(x))
        return self.down_proj.forward(act)


register_feed_forward("gated_mlp", GatedMlp)
