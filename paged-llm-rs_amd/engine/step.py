"""The step function: run the tokens a step brings, as one batch, from the
cache, and return the logits at the wanted places (reference:
model/mod.rs:305-352).  Pages are written; the lengths in the cache manager do
not move: whoever asked for the step records it once it has succeeded."""

from __future__ import annotations

import torch

from ..errors import TensorError
from .batch import StepBatch, build_batch


def require_gpu(device) -> torch.device:
    device = torch.device(device)
    if device.type != "cuda" or not torch.cuda.is_available():
        raise TensorError("the engine runs on the GPU only; no GPU is visible to this process")
    return device


def run_step(model, cache, entries, check_start: bool = True) -> torch.Tensor:
    """32-bit logits [wanted places, vocabulary], in the order of the entries and of their ``want``."""
    batch = build_batch(entries, cache.manager, len(cache.layout.groups), model.spec.vocab_size,
                        model.spec.max_positions, model.device, check_start=check_start)
    for e in entries:
        if e.fresh_state and e.state_slot >= 0:
            cache.clear_state_slot(e.state_slot)
    return model.forward(batch, cache)


def commit_step(cache, entries) -> None:
    """Record that the step ran: every request has its tokens written."""
    for e in entries:
        cache.manager.advance(e.seq_id, len(e.tokens))
