from .generation import GenerationConfig
from .qwen3 import Qwen3Config, read_json
from .registry import architectures, config_class_for, load_config, register_architecture
from .specs import (AttentionSpec, GatedMlpSpec, LayerSpec, ModelSpec, NormSpec, PositionSpec,
                    ScheduleEntry)

__all__ = [
    "GenerationConfig", "Qwen3Config", "read_json", "architectures", "config_class_for",
    "load_config", "register_architecture", "AttentionSpec", "GatedMlpSpec", "LayerSpec",
    "ModelSpec", "NormSpec", "PositionSpec", "ScheduleEntry",
]
