"""How the next token is chosen (reference: crates/pagedllm/src/sampler.rs).

The host sampler is native (csrc/host/sampler.cpp).  Greedy never draws, so a
greedy request cannot shift the numbers a later sampled request gets.
"""

from __future__ import annotations

import ctypes
import math
from dataclasses import dataclass
from typing import Optional

import numpy as np

from .. import native
from ..errors import ConfigError


class Rng:
    """splitmix64: the same seed gives the same tokens on any machine."""

    def __init__(self, seed: int):
        self._state = ctypes.c_uint64(seed & (2 ** 64 - 1))

    @property
    def state(self) -> int:
        return self._state.value

    def next_u64(self) -> int:
        return native.library().plh_rng_next_u64(ctypes.byref(self._state))

    def next_f32(self) -> float:
        return native.library().plh_rng_next_f32(ctypes.byref(self._state))


@dataclass(frozen=True)
class Sampling:
    """temperature 0 means the most likely token every time, with no draw at all."""
    temperature: float = 0.0
    top_k: Optional[int] = None
    top_p: Optional[float] = None

    def __post_init__(self):
        problem = native.library().plh_sampling_problem(
            float(self.temperature) if not isinstance(self.temperature, bool) else -1.0,
            0 if self.top_k is None else 1, int(self.top_k or 0),
            0 if self.top_p is None else 1, float(self.top_p if self.top_p is not None else 1.0)).decode()
        if problem:
            raise ConfigError(f"temperature {self.temperature}, top_k {self.top_k}, top_p {self.top_p}: {problem}")

    @classmethod
    def greedy(cls) -> "Sampling":
        return cls(0.0, None, None)

    @property
    def is_greedy(self) -> bool:
        return self.temperature <= 0.0


def sample_host(sampling: Sampling, logits, rng: Rng) -> int:
    """One token id from a vector of logits: temperature, then top-k, then top-p, then the draw."""
    row = np.ascontiguousarray(logits, dtype=np.float32)
    token = native.library().plh_sample(
        float(sampling.temperature), int(sampling.top_k or 0),
        float(sampling.top_p if sampling.top_p is not None else 1.0), row.ctypes.data, row.size,
        ctypes.byref(rng._state))
    if token < 0:
        raise ConfigError(native.last_error())
    return token
