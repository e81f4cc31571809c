"""A decoder assembled from parts as a ``ModelSpec`` says.

The model owns its parts and the order in which the layers run; it owns no
cache.  ``forward`` runs the tokens of one step and returns logits for the rows
that are asked for (src/exec/dense_swiglu_model.rs:131-1041: embedding, the
layers, final norm, row selection before the vocabulary projection).
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Iterator, Mapping

import torch

from ..config.spec import LayerSpec, ModelSpec
from ..kernels.ops import Kernels, kernels_for
from ..parts import Block, ParamSpec, Part, StepContext, build_part
from ..parts.base import _REGISTRY


def _build_block(spec: LayerSpec, kernels: Kernels) -> Block:
    try:
        cls = _REGISTRY[("block", spec.block)]
    except KeyError:
        raise ValueError(f"no block arrangement of kind {spec.block!r}") from None
    return cls(kernels=kernels,
               mixer=build_part("mixer", spec.mixer, kernels),
               feed_forward=build_part("feed_forward", spec.feed_forward, kernels),
               norms={name: build_part("norm", s, kernels) for name, s in spec.norms.items()})


def walk_params(part: Part, prefix: str = "") -> Iterator[tuple[str, Part, str, ParamSpec]]:
    """Yields (path, owner, local name, spec) for a part and everything below it."""
    for local, spec in part.params().items():
        yield prefix + local, part, local, spec
    for name, child in part.children().items():
        yield from walk_params(child, f"{prefix}{name}.")


@dataclass
class ExpectedTensor:
    """A tensor of the weight files: its shape and type rules, and every (part, local name) that gets it."""
    spec: ParamSpec
    owners: list[tuple[Part, str]] = field(default_factory=list)


def walk_parts(part: Part) -> Iterator[Part]:
    yield part
    for child in part.children().values():
        yield from walk_parts(child)


class DecoderModel:
    def __init__(self, spec: ModelSpec, kernels: Kernels):
        spec.validate()
        self.spec, self.kernels = spec, kernels
        self.embedding = build_part("embedding", spec.embedding, kernels)
        self.layers = [_build_block(ls, kernels) for ls in spec.layers]
        self.final_norm = build_part("norm", spec.final_norm, kernels)
        self.head = build_part("head", spec.head, kernels)
        self.schedule = spec.schedule
        self.loaded = False

    # ------------------------------------------------------------ weights
    def parts(self) -> Iterator[Part]:
        """Every part of the model, sub-parts included."""
        for root in (self.embedding, *self.layers, self.final_norm, self.head):
            yield from walk_parts(root)

    def expected_tensors(self) -> dict[str, ExpectedTensor]:
        """Tensor name in the weight files -> what it must look like and which parts get it.  Parameters
        that the specification gives the same tensor name share one tensor."""
        out: dict[str, ExpectedTensor] = {}

        def add(names: Mapping[str, str], root: Part, prefix: str):
            for path, owner, local, ps in walk_params(root, prefix):
                if path not in names:
                    raise ValueError(f"the configuration gives no tensor name for parameter {path!r}")
                e = out.setdefault(names[path], ExpectedTensor(ps))
                if tuple(e.spec.shape) != tuple(ps.shape):
                    raise ValueError(f"tensor {names[path]!r} is shared by parameters of different shapes: "
                                     f"{list(e.spec.shape)} and {list(ps.shape)} ({path!r})")
                e.owners.append((owner, local))

        add(self.spec.names, self.embedding, "embedding.")
        add(self.spec.names, self.final_norm, "final_norm.")
        add(self.spec.names, self.head, "head.")
        for ls, block in zip(self.spec.layers, self.layers):
            add(ls.names, block, "")
        return out

    def load_tensors(self, tensors: Mapping[str, torch.Tensor]) -> None:
        """``tensors``: file name -> GPU tensor, already checked against ``expected_tensors``."""
        per_part: dict[int, tuple[Part, dict[str, torch.Tensor]]] = {}
        for name, e in self.expected_tensors().items():
            for owner, local in e.owners:
                per_part.setdefault(id(owner), (owner, {}))[1][local] = tensors[name]
        for owner, group in per_part.values():
            owner.load(group)
        self.loaded = True

    # ------------------------------------------------------------- caches
    def cache_specs(self) -> list:
        """One entry per schedule entry: what its mixer keeps (None if it reads another entry's cache)."""
        return [None if e.cache_from is not None else self.layers[e.layer].mixer.cache_spec() for e in self.schedule]

    # ------------------------------------------------------------ forward
    def forward(self, ids: torch.Tensor, ctx: StepContext, caches: list, want_rows: torch.Tensor) -> torch.Tensor:
        """ids int32 [T]; caches: one object per schedule entry; want_rows int32 [R] -> logits [R, vocab]."""
        if not self.loaded:
            raise RuntimeError("the model has no weights yet")
        k = self.kernels
        hidden, residual = self.embedding.forward(ids), None
        for e, cache in zip(self.schedule, caches):
            hidden, residual = self.layers[e.layer].forward(hidden, residual, ctx, cache)
        if want_rows.shape[0] == 0:
            return k.empty(0, self.spec.vocab_size)
        hidden = k.gather_rows(hidden, want_rows)
        if residual is None:
            normed = self.final_norm.forward(hidden)   # a model without layers
        else:
            normed = self.final_norm.forward_add(hidden, k.gather_rows(residual, want_rows))
        return self.head.forward(normed)


def build_model(config, dtype) -> DecoderModel:
    """config: an architecture's configuration object (it has ``model_spec()``)."""
    return DecoderModel(config.model_spec(), kernels_for(dtype))


def load_model(model_dir, dtype) -> DecoderModel:
    """A model folder (config.json, safetensors) -> a model with its weights on the GPU.
    The architecture is chosen by config.json through the registry."""
    from ..config import load_config
    from ..weights import load_weights
    model = build_model(load_config(model_dir), dtype)
    load_weights(model, model_dir)
    return model
