"""y = x . W^T, no bias; W is kept as stored, [out, in] (reference:
model/layers.rs:9-36, which transposes at load; here both operands are read
along their contiguous axis instead)."""

from __future__ import annotations

import torch

from .. import kernels
from ..errors import TensorError


class Linear:
    def __init__(self, weight: torch.Tensor):
        if weight.dim() != 2:
            raise TensorError(f"a linear weight of shape {tuple(weight.shape)}")
        self.weight = weight.contiguous()
        self.out_features, self.in_features = weight.shape

    @classmethod
    def fused(cls, weights) -> "Linear":
        """One product for several projections of the same input: the weights
        are stacked along the output axis, so the output row is their
        concatenation."""
        return cls(torch.cat(list(weights), dim=0))

    def forward(self, x: torch.Tensor, out_dtype: torch.dtype | None = None) -> torch.Tensor:
        if x.dim() != 2 or x.shape[1] != self.in_features:
            raise TensorError(f"a linear of {self.in_features} inputs given {tuple(x.shape)}")
        if x.dtype != self.weight.dtype:
            raise TensorError(f"a {self.weight.dtype} linear given {x.dtype}")
        out_dtype = out_dtype or x.dtype
        if x.dtype == torch.float32:
            # the true 32-bit path: vector-unit multiply-add only
            return kernels.gemm_plain(x, self.weight, out_dtype=torch.float32)
        return kernels.linear_bf16(x, self.weight, out_dtype)
