"""RMSNorm fused with the residual add (reference: model/layers.rs:40-65)."""

from __future__ import annotations

import torch

from .. import kernels
from ..weights.loader import ParamDecl
from .registry import register_norm


class PendingNorm:
    """A norm that has not run yet: the 32-bit stream it will read (every sum already in
    it), the norm, the type its output would have, and the rows wanted (all, or a list).

    A part that is handed one may pass it on to ``Linear.forward``, which runs norm and
    product as one kernel where that pays, or call ``materialize()`` for the normalised rows."""

    __slots__ = ("norm", "resid", "out_dtype", "rows", "handed")

    def __init__(self, norm, resid: torch.Tensor, out_dtype: torch.dtype, rows=None, handed=None):
        self.norm, self.resid, self.out_dtype, self.rows = norm, resid, out_dtype, rows
        # what the product that last added into the stream left of this norm's work (a filled
        # ``kernels.HandedNorm`` of this very norm, all rows), or None
        self.handed = handed if handed is not None and handed.filled and rows is None else None

    @property
    def num_rows(self) -> int:
        return self.resid.shape[0] if self.rows is None else self.rows.numel()

    @property
    def width(self) -> int:
        return self.resid.shape[1]

    def materialize(self) -> torch.Tensor:
        return self.norm.apply(self.resid, None, self.out_dtype, rows=self.rows)


class RmsNorm:
    """x / sqrt(mean(x^2) + eps) * gain, statistic and product in 32-bit."""

    # a product kernel can take this norm as its first stage: it needs ``gain32`` and ``eps`` only
    fuses_into_product = True

    @staticmethod
    def declare(spec, width: int) -> list:
        return [ParamDecl("weight", (width,), "gain")]

    def __init__(self, spec, width: int, params: dict, dtype, device):
        self.eps = float(spec.eps)
        self.width = width
        self.gain = params["weight"]
        # the product kernels that take the norm as their first stage read the gain in 32-bit
        self.gain32 = self.gain if self.gain.dtype == torch.float32 else self.gain.float()

    def handoff(self, rows: int, device):
        """Room for this norm handed forward by a product that adds into the stream (``kernels.HandedNorm``),
        or None where no product would take it: many rows, a wide stream."""
        if rows > kernels.SKINNY_ROWS or self.width > kernels.FUSED_NORM_MAX_WIDTH or self.width % 8:
            return None
        return kernels.HandedNorm(self.gain32, self.eps, rows, self.width, device)

    def apply(self, resid: torch.Tensor, delta, out_dtype: torch.dtype, rows=None) -> torch.Tensor:
        n = resid.shape[0] if rows is None else rows.numel()
        out = torch.empty((n, self.width), dtype=out_dtype, device=resid.device)
        return kernels.add_rmsnorm(resid, delta, self.gain, self.eps, out, rows=rows)


register_norm("rms_norm", RmsNorm)
