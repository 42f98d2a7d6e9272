from .specs import (AttentionSpec, GatedMLPSpec, LayerSpec, ModelSpec, NormSpec, PositionSpec,
                    ScheduleEntry, default_schedule)
from .qwen3 import ConfigError, Qwen3Config
from .registry import (Architecture, known_architectures, read_config, register_architecture,
                       resolve_architecture, unregister_architecture)

register_architecture(Qwen3Config.architecture, Qwen3Config, model_types=("qwen3",))

__all__ = [
    "AttentionSpec", "GatedMLPSpec", "LayerSpec", "ModelSpec", "NormSpec", "PositionSpec",
    "ScheduleEntry", "default_schedule", "ConfigError", "Qwen3Config", "Architecture",
    "known_architectures", "read_config", "register_architecture", "resolve_architecture",
    "unregister_architecture",
]
