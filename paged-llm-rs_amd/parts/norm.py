"""RMSNorm fused with the residual add (reference: model/layers.rs:40-65)."""

from __future__ import annotations

import torch

from .. import kernels
from ..weights.loader import ParamDecl
from .registry import register_norm


class RmsNorm:
    """x / sqrt(mean(x^2) + eps) * gain, statistic and product in 32-bit."""

    @staticmethod
    def declare(spec, width: int) -> list:
        return [ParamDecl("weight", (width,), "gain")]

    def __init__(self, spec, width: int, params: dict, dtype, device):
        self.eps = float(spec.eps)
        self.width = width
        self.gain = params["weight"]

    def apply(self, resid: torch.Tensor, delta, out_dtype: torch.dtype, rows=None) -> torch.Tensor:
        n = resid.shape[0] if rows is None else rows.numel()
        out = torch.empty((n, self.width), dtype=out_dtype, device=resid.device)
        return kernels.add_rmsnorm(resid, delta, self.gain, self.eps, out, rows=rows)


register_norm("rms_norm", RmsNorm)
