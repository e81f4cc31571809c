"""One registry from an architecture's name to its configuration class.

The configuration class parses config.json (``from_dict``) and describes the
model as data (``model_spec``); the model itself is assembled from that
description by ``vosti_amd.models.build_model``.  Unknown architectures are an
error (the reference's dispatch is a closed match: src/exec/model.rs:205-621,
src/model_config.rs:11-16).

An architecture lives in one of two places.  Those of the native library
(csrc/host: ``register_architecture`` there) need no Python code at all: their
rules are asked of the library (``describe``) and a config.json that names one
comes back as a ``NativeConfig``; a typed class such as ``Qwen3Config`` may sit
on top.  Those registered here with ``@register_architecture`` are written in
Python, for models made of parts that are added from Python.
"""
from __future__ import annotations

import json
from pathlib import Path
from typing import Any, Mapping

from .spec import LayerSpec, ModelSpec, PartSpec, ScheduleEntry


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
    """config.json ``model_type`` -> architecture name, for every architecture registered with one, here or in
    the native library."""
    from ..cache.host import native_model_types
    return {**native_model_types(), **_MODEL_TYPES}


def describe(raw: Mapping[str, Any]) -> dict:
    """The native library's description of the model that ``raw`` (the keys of a config.json) configures:
    ``{"architecture", "config": typed values, "embedding", "layers", "schedule", "names", ...}``."""
    from ..cache.host import UnknownArchitecture, describe_config
    try:
        return describe_config(dict(raw))
    except UnknownArchitecture as e:
        raise ConfigError(str(e)) from None
    except ValueError as e:
        raise ConfigError(str(e)) from None


def _part(d: Mapping[str, Any]) -> PartSpec:
    params: dict[str, Any] = dict(d["numbers"])
    params.update({name: _part(sub) for name, sub in d["parts"].items()})
    return PartSpec(d["kind"], params)


def spec_from_description(d: Mapping[str, Any]) -> ModelSpec:
    layers: list[LayerSpec] = []
    for l in d["layers"]:
        if "same_as" in l:
            first = layers[l["same_as"]]
            layers.append(LayerSpec(first.block, first.mixer, first.feed_forward, first.norms, dict(l["names"])))
        else:
            layers.append(LayerSpec(l["block"], _part(l["mixer"]), _part(l["feed_forward"]),
                                    {n: _part(p) for n, p in l["norms"].items()}, dict(l["names"])))
    return ModelSpec(architecture=d["architecture"], vocab_size=d["vocab_size"], hidden_size=d["hidden_size"],
                     max_positions=d["max_positions"], embedding=_part(d["embedding"]), layers=tuple(layers),
                     schedule=tuple(ScheduleEntry(l, None if c < 0 else c) for l, c in d["schedule"]),
                     final_norm=_part(d["final_norm"]), head=_part(d["head"]), names=dict(d["names"]),
                     ignored_names=tuple(d["ignored_names"]))


class NativeConfig:
    """A configuration of an architecture that only the native library knows: the raw keys, the typed
    values the library read from them (as attributes) and its description of the model."""

    def __init__(self, raw: Mapping[str, Any], description: Mapping[str, Any]):
        self._raw, self._description = dict(raw), description
        self.architecture = description["architecture"]

    def __getattr__(self, name: str):
        try:
            return self._description["config"][name]
        except KeyError:
            raise AttributeError(name) from None

    @classmethod
    def from_dict(cls, raw: Mapping[str, Any]) -> "NativeConfig":
        return cls(raw, describe(raw))

    def to_dict(self) -> dict[str, Any]:
        return dict(self._raw)

    def model_spec(self) -> ModelSpec:
        spec = spec_from_description(self._description)
        spec.validate()
        return spec


def resolve_architecture(raw: Mapping[str, Any]) -> str:
    """The architecture that a config.json names: the first entry of "architectures", else a registered
    "model_type"."""
    archs = raw.get("architectures")
    if isinstance(archs, (list, tuple)) and archs:
        return archs[0]
    types = model_types()
    if raw.get("model_type") in types:
        return types[raw["model_type"]]
    raise ConfigError("config.json names no architecture (key 'architectures') and no known 'model_type'")


def config_from_dict(raw: Mapping[str, Any]):
    name = resolve_architecture(raw)
    if name in _ARCHITECTURES:
        return _ARCHITECTURES[name].from_dict(raw)
    return NativeConfig.from_dict(raw)      # the library's architectures, or its error that names them


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
