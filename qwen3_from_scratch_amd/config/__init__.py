from .model_config import ConfigError, ModelConfig
from .registry import (
    architectures,
    load_model_config,
    lookup_architecture,
    lookup_part,
    part_names,
    register_architecture,
    register_part,
)
from .engine_config import EngineConfig, GenerationDefaults

__all__ = [
    "ConfigError",
    "ModelConfig",
    "EngineConfig",
    "GenerationDefaults",
    "architectures",
    "load_model_config",
    "lookup_architecture",
    "lookup_part",
    "part_names",
    "register_architecture",
    "register_part",
]
