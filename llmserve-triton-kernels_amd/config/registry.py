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


ARCHITECTURES: dict[str, Architecture] = {}
_MODEL_TYPES: dict[str, str] = {}  # config.json "model_type" -> architecture name, for files without "architectures"


def register_architecture(name: str, config_class, build_spec, model_type: str | None = None) -> Architecture:
    arch = Architecture(name, config_class, build_spec)
    ARCHITECTURES[name] = arch
    if model_type:
        _MODEL_TYPES[model_type] = name
    return arch


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
