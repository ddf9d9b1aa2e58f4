"""One registry from an architecture's name to its configuration class.

``config.json`` chooses the model everywhere in the package: by the first entry
of ``architectures`` or, when that key is absent, by ``model_type``.
"""

from __future__ import annotations

from pathlib import Path

from ..errors import ConfigError, UnsupportedError
from .qwen3 import Qwen3Config, read_json

_ARCHITECTURES: dict = {}
_MODEL_TYPES: dict = {}


def register_architecture(name: str, config_class, model_type: str | None = None) -> None:
    """``config_class`` needs ``from_dict(dict)`` and ``model_spec()``."""
    _ARCHITECTURES[name] = config_class
    if model_type is not None:
        _MODEL_TYPES[model_type] = config_class


def architectures() -> list:
    return sorted(_ARCHITECTURES)


def config_class_for(d: dict):
    if not isinstance(d, dict):
        raise ConfigError("config.json does not hold an object")
    names = d.get("architectures")
    if isinstance(names, list) and names:
        name = names[0]
        if isinstance(name, str) and name in _ARCHITECTURES:
            return _ARCHITECTURES[name]
        raise UnsupportedError(
            f"architecture {name!r}, the registry knows {', '.join(architectures())}"
        )
    model_type = d.get("model_type")
    if model_type is None:
        raise ConfigError("config.json names neither architectures nor model_type")
    if isinstance(model_type, str) and model_type in _MODEL_TYPES:
        return _MODEL_TYPES[model_type]
    raise UnsupportedError(
        f"model_type {model_type!r}, the registry knows {', '.join(sorted(_MODEL_TYPES))}"
    )


def load_config(source):
    """A typed configuration from a model folder, a config.json path or a dict."""
    if isinstance(source, dict):
        d = source
    else:
        path = Path(source)
        if path.is_dir():
            path = path / "config.json"
        d = read_json(path)
    return config_class_for(d).from_dict(d)


register_architecture("Qwen3ForCausalLM", Qwen3Config, model_type="qwen3")
