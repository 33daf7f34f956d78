"""Configuration: typed per-architecture configs and the architecture registry."""

from .base import (ConfigError, LayerSpec, ModelConfig, ModelSpec, PartSpec,
                   ScheduleEntry)
from .registry import (config_class_for, config_from_dict, config_from_dir,
                       known_architectures, register_architecture,
                       unregister_architecture)
from .qwen3 import Qwen3Config

__all__ = [
    "ConfigError", "LayerSpec", "ModelConfig", "ModelSpec", "PartSpec", "ScheduleEntry",
    "config_class_for", "config_from_dict", "config_from_dir", "known_architectures",
    "register_architecture", "unregister_architecture", "Qwen3Config",
]
