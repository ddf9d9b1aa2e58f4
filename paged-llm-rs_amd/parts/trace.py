"""Named activations of one forward pass, for finding the module at which an engine and a reference
part ways (reference: model/mod.rs:34-80, whose recorder names every module's output
``<module path>.out``, and ``.in`` for the inputs of o_proj and down_proj).

Only the 32-bit path records: there every module runs as a kernel of its own, so each named tensor
exists.  In bfloat16 norms, activations and residual sums are stages of product kernels and most of
these tensors are never written.  Recording copies; without a trace nothing here runs.
"""

from __future__ import annotations

import torch


class ActivationTrace:
    def __init__(self, store: dict, prefix: str = ""):
        self.store = store
        self.prefix = prefix

    def record(self, name: str, tensor: torch.Tensor) -> None:
        self.store[self.prefix + name] = tensor.detach().clone()

    def child(self, name: str) -> "ActivationTrace":
        """A recorder for the module ``name`` inside this one."""
        return ActivationTrace(self.store, f"{self.prefix}{name}.")
