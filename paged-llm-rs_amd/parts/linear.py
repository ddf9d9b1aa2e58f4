"""y = x . W^T (+ b); W is kept as stored, [out, in] (reference:
model/layers.rs:9-36, which transposes at load and has no bias; here both
operands are read along their contiguous axis instead, and a bias is a vector
added behind the product)."""

from __future__ import annotations

import torch

from .. import kernels
from ..errors import TensorError
from .norm import PendingNorm


class Linear:
    # Whether a bfloat16 weight is kept a second time in the order the product of few rows reads fastest
    # (``kernels.weights_in_strips``): the decoding steps then read that copy, everything else the weight as
    # stored.  It doubles the memory of the weights; ``load_model(..., strips=False)`` builds a model without.
    keep_strips = True

    def __init__(self, weight: torch.Tensor, bias: torch.Tensor | None = None):
        if weight.dim() != 2:
            raise TensorError(f"a linear weight of shape {tuple(weight.shape)}")
        self.weight = weight.contiguous()
        self.strips = kernels.weights_in_strips(self.weight) if Linear.keep_strips else None
        self.out_features, self.in_features = weight.shape
        if bias is not None and tuple(bias.shape) != (self.out_features,):
            raise TensorError(f"a bias of shape {tuple(bias.shape)} for {self.out_features} outputs")
        self.bias = None if bias is None else bias.contiguous()

    @classmethod
    def fused(cls, weights, biases=None) -> "Linear":
        """One product for several projections of the same input: the weights
        (and the biases, if they have any) are stacked along the output axis,
        so the output row is their concatenation."""
        biases = [b for b in (biases or []) if b is not None]
        return cls(torch.cat(list(weights), dim=0), torch.cat(biases, dim=0) if biases else None)

    def forward(self, x, out_dtype: torch.dtype | None = None, add_into: torch.Tensor | None = None,
                swiglu: bool = False, activation: str = "silu", hand=None):
        """The product of ``x`` (rows, or a norm still to run) with the weight.

        ``swiglu``: the weight is [gate | up] stacked and act(gate) * up comes back (``activation``: silu or a gelu).
        ``add_into``: the 32-bit residual stream; where the product kernel can add its result
        there itself it does and None comes back, otherwise the result comes back unadded.
        ``hand``: room for the norm that follows the stream (``kernels.HandedNorm``); a product kernel that adds
        into the stream and can leave that norm's work behind fills it, any other way leaves it unfilled."""
        if self.bias is not None:
            # The bias is added behind the product by a kernel of its own; what the product would have fused
            # behind itself (the activation, the sum into the stream) then runs unfused as well.
            if isinstance(x, PendingNorm):
                x = x.materialize()
            y = self._product(x, out_dtype if not swiglu else None)
            kernels.add_bias(y, self.bias)
            return kernels.swiglu(y, activation=activation) if swiglu else y
        return self._product(x, out_dtype, add_into, swiglu, activation, hand)

    def _product(self, x, out_dtype: torch.dtype | None = None, add_into: torch.Tensor | None = None,
                 swiglu: bool = False, activation: str = "silu", hand=None):
        if isinstance(x, PendingNorm):
            if x.width != self.in_features:
                raise TensorError(f"a linear of {self.in_features} inputs given a stream of width {x.width}")
            columns = self.out_features // 2 if swiglu else self.out_features
            if (x.handed is not None and add_into is None and self.weight.dtype == torch.bfloat16
                    and kernels.takes_handed_norm(x.num_rows, columns, self.in_features, swiglu)):
                return kernels.gemm_skinny(None, self.weight, out_dtype or x.out_dtype, swiglu=swiglu,
                                           activation=activation, handed=x.handed, strips=self.strips)
            if (getattr(x.norm, "fuses_into_product", False) and add_into is None
                    and kernels.fused_norm_applies(x.num_rows, self.in_features, self.weight)
                    and self.out_features <= kernels.FUSED_NORM_MAX_COLUMNS):
                return kernels.gemm_skinny(x.resid, self.weight, out_dtype or x.out_dtype, swiglu=swiglu,
                                           norm_gain=x.norm.gain32, eps=x.norm.eps, rows=x.rows, activation=activation,
                                           strips=self.strips)
            x = x.materialize()
        if x.dim() != 2 or x.shape[1] != self.in_features:
            raise TensorError(f"a linear of {self.in_features} inputs given {tuple(x.shape)}")
        if x.dtype != self.weight.dtype:
            raise TensorError(f"a {self.weight.dtype} linear given {x.dtype}")
        out_dtype = out_dtype or x.dtype
        if x.dtype == torch.float32:
            # the true 32-bit path: vector-unit multiply-add only
            y = kernels.gemm_plain(x, self.weight, out_dtype=torch.float32)
            return kernels.swiglu(y, activation=activation) if swiglu else y
        if kernels.skinny_applies(x, self.weight, self.strips is not None):
            if add_into is not None and not swiglu:
                if hand is not None and not kernels.hands_norm_forward(x.shape[0], self.out_features, self.in_features):
                    hand = None
                kernels.gemm_skinny(x, self.weight, add_into=add_into, hand=hand, strips=self.strips)
                return None
            return kernels.gemm_skinny(x, self.weight, out_dtype, swiglu=swiglu, activation=activation,
                                       strips=self.strips)
        if kernels.stream_wins(x.shape[0], self.out_features, self.in_features):
            if add_into is not None and not swiglu:
                kernels.gemm_stream(x, self.weight, add_into=add_into)
                return None
            return kernels.gemm_stream(x, self.weight, out_dtype, swiglu=swiglu, activation=activation)
        if add_into is not None and not swiglu:
            splits = kernels.library_splits(x.shape[0], self.out_features, self.in_features)
            if splits > 1:
                kernels.gemm_split_library(x, self.weight, splits, add_into=add_into)
                return None
        if swiglu:
            if kernels.tiled_swiglu_wins(x.shape[0], self.out_features // 2, self.in_features):
                return kernels.gemm_tiled(x, self.weight, swiglu=True, activation=activation)
            return kernels.swiglu(kernels.linear_bf16(x, self.weight, x.dtype, self.strips), activation=activation)
        return kernels.linear_bf16(x, self.weight, out_dtype, self.strips)


def linears_of(part, seen=None, depth: int = 0):
    """Every ``Linear`` that ``part`` holds (its members, their members, the members of lists and tuples; a few
    levels deep): what a model's memory is made of."""
    import types

    seen = set() if seen is None else seen
    if id(part) in seen or depth > 8:
        return
    seen.add(id(part))
    if isinstance(part, Linear):
        yield part
    elif isinstance(part, (list, tuple)):
        for member in part:
            yield from linears_of(member, seen, depth + 1)
    elif hasattr(part, "__dict__") and not isinstance(part, (torch.Tensor, type, types.ModuleType, types.FunctionType)):
        for member in vars(part).values():
            if not isinstance(member, (torch.Tensor, str, int, float, bool, dict, type(None))):
                yield from linears_of(member, seen, depth + 1)
