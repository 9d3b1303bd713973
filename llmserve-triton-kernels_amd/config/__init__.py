"""Typed configuration of models and of the engine, and the architecture registry."""

from .engine_config import EngineConfig
from .model_config import ConfigError, LlamaConfig
from .registry import (ARCHITECTURES, Architecture, architecture_of, is_preset, preset, preset_names, read_config,
                       register_architecture)

__all__ = ["EngineConfig", "ConfigError", "LlamaConfig", "preset", "preset_names", "is_preset", "ARCHITECTURES",
           "Architecture", "architecture_of", "read_config", "register_architecture"]
