"""What a model is made of, as data.

A configuration class (one per architecture) turns its config.json keys into a
``ModelSpec``: which part stands where, with which sizes and constants, layer
by layer, and in which order the layers run.  Nothing below the configuration
knows an architecture's name.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Mapping


@dataclass(frozen=True)
class PartSpec:
    """A part chosen by ``kind`` from its category's registry, with its parameters."""
    kind: str
    params: Mapping[str, Any] = field(default_factory=dict)


@dataclass(frozen=True)
class LayerSpec:
    """One layer: how its parts are arranged (``block``) and which parts they are.

    ``names`` maps a parameter path inside the layer ("mixer.q_proj",
    "norms.input") to the tensor's name in the weight files.
    """
    block: str
    mixer: PartSpec
    feed_forward: PartSpec
    norms: Mapping[str, PartSpec]
    names: Mapping[str, str]


@dataclass(frozen=True)
class ScheduleEntry:
    """One execution of a layer.  A layer may be named by several entries.

    ``cache_from``: index of an earlier entry whose cache this execution reads
    instead of writing one of its own.
    """
    layer: int
    cache_from: int | None = None


@dataclass(frozen=True)
class ModelSpec:
    architecture: str
    vocab_size: int
    hidden_size: int
    max_positions: int
    embedding: PartSpec
    layers: tuple[LayerSpec, ...]
    schedule: tuple[ScheduleEntry, ...]
    final_norm: PartSpec
    head: PartSpec
    # "embedding.weight", "final_norm.weight", "head.weight" -> tensor names.  Two parameters with the
    # same tensor name are one tensor: a head tied to the embedding is written so.
    names: Mapping[str, str]
    # Tensors that a checkpoint may hold although the model does not use them.
    ignored_names: tuple[str, ...] = ()

    def validate(self) -> None:
        for i, e in enumerate(self.schedule):
            if not 0 <= e.layer < len(self.layers):
                raise ValueError(f"schedule entry {i} names layer {e.layer}, but there are {len(self.layers)} layers")
            if e.cache_from is not None:
                if not 0 <= e.cache_from < i:
                    raise ValueError(f"schedule entry {i} reads the cache of entry {e.cache_from}, which does not run before it")
                if self.schedule[e.cache_from].cache_from is not None:
                    raise ValueError(f"schedule entry {i} reads the cache of entry {e.cache_from}, which has none of its own")
