"""One registry from an architecture's name (config.json "architectures"[0]) to what
builds it: the configuration class that reads its config.json and the function that turns
that configuration into a `ModelSpec`.  The reference has no such table: its loader always
constructs the one model class (src/llmserve/weights.py:45-46)."""

from __future__ import annotations

import json
from dataclasses import dataclass
from pathlib import Path
from typing import Any, Callable


@dataclass(frozen=True)
class Architecture:
    name: str
    config_class: Any  # has from_dict(dict) -> config, and config.to_dict()
    build_spec: Callable[[Any], Any]  # config -> parts.spec.ModelSpec
    model_type: str | None = None
    presets: Any = None  # named sizes of this architecture: name -> config.json dictionary


ARCHITECTURES: dict[str, Architecture] = {}
_MODEL_TYPES: dict[str, str] = {}  # config.json "model_type" -> architecture name, for files without "architectures"


def register_architecture(name: str, config_class, build_spec, model_type: str | None = None,
                          presets: dict[str, dict] | None = None) -> Architecture:
    """`presets`: named sizes of the architecture (name -> config.json keys), found by `preset(name)` and by
    `LLM(name, random_weights=True)`; the architecture's name and model type are filled in when one is asked for."""
    arch = Architecture(name, config_class, build_spec, model_type, dict(presets or {}))
    ARCHITECTURES[name] = arch
    if model_type:
        _MODEL_TYPES[model_type] = name
    return arch


def _preset_key(name: str) -> str:
    return name.lower().replace("_", "-")


def preset_names() -> list[str]:
    """Every named size of every registered architecture."""
    _ensure_builtin()
    return sorted(key for arch in ARCHITECTURES.values() for key in arch.presets)


def preset(name: str) -> dict:
    """config.json dictionary of a named size, whichever architecture registered it."""
    from .model_config import ConfigError

    _ensure_builtin()
    key = _preset_key(name)
    for arch in ARCHITECTURES.values():
        if key in arch.presets:
            d = dict(arch.presets[key])
            d.setdefault("architectures", [arch.name])
            if arch.model_type:
                d.setdefault("model_type", arch.model_type)
            return d
    raise ConfigError(f"unknown preset {name!r}; known: {preset_names()}")


def is_preset(name: str) -> bool:
    return _preset_key(name) in preset_names()


def _ensure_builtin() -> None:
    from .. import models  # noqa: F401  (registers the built-in architectures)


def architecture_of(config_dict: dict) -> Architecture:
    _ensure_builtin()
    names = config_dict.get("architectures")
    if names:
        name = names[0]
    elif config_dict.get("model_type") in _MODEL_TYPES:
        name = _MODEL_TYPES[config_dict["model_type"]]
    else:
        raise KeyError("config.json names no architecture (\"architectures\" is missing or empty and "
                       f"\"model_type\" is not one of {sorted(_MODEL_TYPES)}); "
                       f"registered architectures: {sorted(ARCHITECTURES)}")
    if name not in ARCHITECTURES:
        raise KeyError(f"architecture {name!r} is not registered; registered: {sorted(ARCHITECTURES)}")
    return ARCHITECTURES[name]


def read_config(model_dir: str | Path):
    """(architecture, typed configuration, raw dict) of a model folder."""
    path = Path(model_dir) / "config.json"
    if not path.exists():
        raise FileNotFoundError(f"no config.json in {model_dir}")
    raw = json.loads(path.read_text())
    arch = architecture_of(raw)
    return arch, arch.config_class.from_dict(raw), raw
