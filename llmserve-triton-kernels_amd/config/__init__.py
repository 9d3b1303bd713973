"""Typed configuration of models and of the engine, and the architecture registry."""

from .engine_config import EngineConfig
from .model_config import PRESETS, ConfigError, LlamaConfig, preset
from .registry import ARCHITECTURES, Architecture, architecture_of, read_config, register_architecture

__all__ = ["EngineConfig", "PRESETS", "ConfigError", "LlamaConfig", "preset", "ARCHITECTURES", "Architecture",
           "architecture_of", "read_config", "register_architecture"]
