from .specs import (AttentionSpec, DenseMLPSpec, GatedDeltaSpec, GatedMLPSpec, LayerSpec, ModelSpec, NormSpec, PositionSpec,
                    ScheduleEntry, default_schedule)
from .qwen3 import ConfigError, Qwen3Config
from .tirurax import TiruraxConfig
from .registry import (Architecture, known_architectures, read_config, register_architecture,
                       resolve_architecture, unregister_architecture)

register_architecture(Qwen3Config.architecture, Qwen3Config, model_types=("qwen3",))
register_architecture(TiruraxConfig.architecture, TiruraxConfig, model_types=("tirurax",))

__all__ = [
    "AttentionSpec", "DenseMLPSpec", "GatedDeltaSpec", "GatedMLPSpec", "LayerSpec", "ModelSpec", "NormSpec", "PositionSpec",
    "ScheduleEntry", "default_schedule", "ConfigError", "Qwen3Config", "TiruraxConfig", "Architecture",
    "known_architectures", "read_config", "register_architecture", "resolve_architecture",
    "unregister_architecture",
]
