"""What generation_config.json says about how the model should be run
(reference: config.rs:171-231)."""

from __future__ import annotations

from dataclasses import dataclass, field
from pathlib import Path
from typing import Optional

from ..errors import PagedLLMError
from .qwen3 import read_json


def _token_ids(value) -> Optional[list]:
    """One id, or a list of them, or nothing."""
    if isinstance(value, bool):
        return None
    if isinstance(value, int) and 0 <= value < 2 ** 32:
        return [value]
    if isinstance(value, list):
        ids = [v for v in value if isinstance(v, int) and not isinstance(v, bool) and 0 <= v < 2 ** 32]
        return ids or None
    return None


@dataclass
class GenerationConfig:
    eos_token_ids: list = field(default_factory=list)
    temperature: Optional[float] = None
    top_p: Optional[float] = None
    top_k: Optional[int] = None

    @classmethod
    def from_dir(cls, directory) -> "GenerationConfig":
        directory = Path(directory)
        try:
            generation = read_json(directory / "generation_config.json")
        except PagedLLMError:
            generation = None
        if not isinstance(generation, dict):                 # (absent, or a file that holds no object)
            generation = None
        eos = _token_ids(generation.get("eos_token_id")) if generation else None
        if eos is None:
            try:
                config = read_json(directory / "config.json")
                eos = _token_ids(config.get("eos_token_id")) if isinstance(config, dict) else None
            except PagedLLMError:
                eos = None

        def number(key):
            if not generation:
                return None
            v = generation.get(key)
            return float(v) if isinstance(v, (int, float)) and not isinstance(v, bool) else None

        top_k = number("top_k")
        return cls(
            eos_token_ids=eos or [],
            temperature=number("temperature"),
            top_p=number("top_p"),
            top_k=int(top_k) if top_k is not None and int(top_k) > 0 else None,
        )
