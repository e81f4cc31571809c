"""One registry from an architecture's name to its configuration class.

The configuration class parses config.json (``from_dict``) and describes the
model as data (``model_spec``); the model itself is assembled from that
description by ``vosti_amd.models.build_model``.  Unknown architectures are an
error (the reference's dispatch is a closed match: src/exec/model.rs:205-621,
src/model_config.rs:11-16).
"""
from __future__ import annotations

import json
from pathlib import Path
from typing import Any, Mapping


class ConfigError(ValueError):
    pass


_ARCHITECTURES: dict[str, type] = {}
_MODEL_TYPES: dict[str, str] = {}


def register_architecture(name: str, model_type: str | None = None):
    """Class decorator: ``name`` is the entry of config.json's "architectures" list."""
    def deco(cls):
        if name in _ARCHITECTURES and _ARCHITECTURES[name] is not cls:
            raise ConfigError(f"architecture {name!r} is already registered")
        _ARCHITECTURES[name] = cls
        if model_type is not None:
            _MODEL_TYPES[model_type] = name
        return cls
    return deco


def architecture_names() -> list[str]:
    return sorted(_ARCHITECTURES)


def model_types() -> dict[str, str]:
    """config.json ``model_type`` -> architecture name, for every architecture registered with one."""
    return dict(_MODEL_TYPES)


def resolve_architecture(raw: Mapping[str, Any]) -> str:
    archs = raw.get("architectures")
    if isinstance(archs, (list, tuple)) and archs:
        name = archs[0]
    elif raw.get("model_type") in _MODEL_TYPES:
        name = _MODEL_TYPES[raw["model_type"]]
    else:
        raise ConfigError("config.json names no architecture (key 'architectures') and no known 'model_type'")
    if name not in _ARCHITECTURES:
        raise ConfigError(f"unknown architecture {name!r}; registered: {', '.join(architecture_names()) or 'none'}")
    return name


def config_from_dict(raw: Mapping[str, Any]):
    return _ARCHITECTURES[resolve_architecture(raw)].from_dict(raw)


def load_config(model_dir: str | Path):
    path = Path(model_dir) / "config.json"
    if not path.is_file():
        raise ConfigError(f"{path} not found")
    try:
        raw = json.loads(path.read_text())
    except json.JSONDecodeError as e:
        raise ConfigError(f"{path} is not valid JSON: {e}") from None
    if not isinstance(raw, dict):
        raise ConfigError(f"{path} must hold a JSON object")
    return config_from_dict(raw)
