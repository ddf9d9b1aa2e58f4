"""The gated feed-forward: down(act(gate(x)) * up(x)), the activation on the
gate branch (reference: model/layers.rs:72-107, where it is SiLU; the spec names it)."""

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
        if spec.activation not in kernels.ACTIVATIONS:
            raise UnsupportedError(f"activation {spec.activation!r}, the kernels know {', '.join(sorted(kernels.ACTIVATIONS))}")
        self.activation = spec.activation
        # one product for gate and up: the output row is [gate | up]
        self.gate_up_proj = Linear.fused([params["gate_proj.weight"], params["up_proj.weight"]])
        self.down_proj = Linear(params["down_proj.weight"])

    # forward takes a norm still to run in place of rows, and may add its result into the stream
    fuses = True
    # ... and a recorder of named activations
    records = True
    # ... and room for the norm that follows the stream, which the product that adds into it may fill
    hands_forward = True

    def forward(self, x, residual: torch.Tensor | None = None, trace=None, hand=None):
        """``x``: normalised rows, or a PendingNorm.  With ``residual`` (the 32-bit stream) the
        result is added there where the product kernel can do it, and None comes back; ``hand``
        (``kernels.HandedNorm``) is then filled where that kernel can leave the next norm's work behind."""
        if trace is not None:
            both = self.gate_up_proj.forward(x)
            inter = both.shape[1] // 2
            trace.record("gate_proj.out", both[:, :inter])
            trace.record("up_proj.out", both[:, inter:])
            act = kernels.swiglu(both, activation=self.activation)
            trace.record("down_proj.in", act)
            out = self.down_proj.forward(act)
            trace.record("down_proj.out", out)
            return out
        # (few rows: the activation is the product's epilogue)
        act = self.gate_up_proj.forward(x, swiglu=True, activation=self.activation)
        return self.down_proj.forward(act, add_into=residual, hand=hand if residual is not None else None)


register_feed_forward("gated_mlp", GatedMlp)
