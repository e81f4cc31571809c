"""Interfaces and registries of the parts a model is assembled from.

Categories: ``embedding``, ``norm``, ``position``, ``mixer``, ``feed_forward``,
``block``, ``head``.  A part is a class registered under (category, kind); it is
built from the parameters of its ``PartSpec`` and a ``Kernels`` object, declares
the tensors it needs (``params``), receives them (``load``) and computes
(``forward``).  No part knows which model it is in: sizes and constants arrive
as parameters, tensor names are the architecture's business.

To add a part, subclass the category's base class, decorate it with
``@register_part(category, kind)`` and name the kind in a ``PartSpec``.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Callable, Mapping

import numpy as np
import torch

from ..config.spec import PartSpec
from ..kernels.ops import Kernels

_REGISTRY: dict[tuple[str, str], type] = {}
CATEGORIES = ("embedding", "norm", "position", "mixer", "feed_forward", "block", "head")


def register_part(category: str, kind: str):
    if category not in CATEGORIES:
        raise ValueError(f"unknown part category {category!r}")

    def deco(cls):
        _REGISTRY[(category, kind)] = cls
        cls.category, cls.kind = category, kind
        return cls
    return deco


def build_part(category: str, spec: PartSpec, kernels: Kernels):
    try:
        cls = _REGISTRY[(category, spec.kind)]
    except KeyError:
        known = sorted(k for c, k in _REGISTRY if c == category)
        raise ValueError(f"no {category} part of kind {spec.kind!r}; registered: {known}") from None
    return cls(kernels=kernels, **spec.params)


@dataclass(frozen=True)
class ParamSpec:
    """A tensor a part needs from the weight files.

    ``init``: how the random-weights mode draws it: ("normal", std) or
    ("uniform", low, high).  ``keep_f32``: if the file stores it in 32-bit it
    stays so, whatever the compute type (norm weights may).
    """
    shape: tuple[int, ...]
    init: tuple = ("normal", 0.02)
    keep_f32: bool = False


# -------------------------------------------------------------------- caches
@dataclass(frozen=True)
class KVPagesSpec:
    """The mixer keeps keys and values of ``window`` (0: all) past positions in pages."""
    num_kv_heads: int
    head_dim: int
    window: int = 0


@dataclass(frozen=True)
class StateSlotSpec:
    """The mixer keeps a fixed-size state per request."""
    shape: tuple[int, ...]
    dtype: torch.dtype = torch.float32


@dataclass
class PagedKV:
    """What an attention-like mixer gets: its layer's pages and its group's index."""
    k: torch.Tensor        # [pages, kv heads, page, head_dim]
    v: torch.Tensor        # [pages, kv heads, head_dim, page]  (transposed)
    group: int
    page_size: int
    writable: bool = True  # False: the pages belong to an earlier execution; read only


@dataclass
class StateSlots:
    """What a mixer with state gets: one row per state slot."""
    state: torch.Tensor    # [slots, *shape]


@dataclass
class GroupTables:
    """Per cache group: where the step's tokens go and where each sequence's pages are."""
    slots: torch.Tensor         # int32 [T]: page * page_size + offset of every token
    block_table: torch.Tensor   # int32 [S, W]
    window: int


@dataclass
class HostStep:
    """One step as the host knows it: what parts may size launches and buffers by.

    ``frozen``: the step's launches are recorded for replay with other lengths, so
    their geometry must cover every key count up to ``k_len_bound`` (what the block
    tables can hold); otherwise ``k_len_bound`` is the largest of ``k_lens``.
    ``memo`` is a scratch pad for what a part derives from these lists, so that the
    layers of a model that share a part kind derive it once per step."""
    q_lens: list[int]           # tokens of each sequence in this step
    starts: list[int]           # position of each sequence's first token in this step
    k_lens: list[int]           # keys of each sequence once this step's tokens are stored
    state_slots: list[int]      # the state slot of each sequence
    k_len_bound: int
    frozen: bool = False
    memo: dict = field(default_factory=dict)


@dataclass
class StepContext:
    """Everything about one step that parts may need.  Device tensors are int32.

    ``inputs`` holds the per-step device arrays that parts asked for through
    ``Part.step_inputs`` (they travel in the step's one upload); ``workspace(n)``
    gives a float32 buffer of at least n elements whose contents do not outlive a
    part's forward (its size was announced through ``Part.workspace_floats``)."""
    kernels: Kernels
    num_tokens: int
    num_seqs: int
    positions: torch.Tensor      # [T]
    cu_q: torch.Tensor           # [S + 1]
    k_len: torch.Tensor          # [S]: keys of each sequence once this step's tokens are stored
    state_slots: torch.Tensor    # [S]: the state slot of each sequence
    groups: list[GroupTables]
    host: HostStep
    inputs: Mapping[str, torch.Tensor] = field(default_factory=dict)
    workspace: Callable[[int], torch.Tensor] | None = None

    # Host copies, for parts that loop over sequences on the host.
    @property
    def host_q_lens(self) -> list[int]:
        return self.host.q_lens

    @property
    def host_starts(self) -> list[int]:
        return self.host.starts

    @property
    def host_state_slots(self) -> list[int]:
        return self.host.state_slots


# ----------------------------------------------------------------- interfaces
class Part:
    category = kind = ""

    def __init__(self, kernels: Kernels):
        self.kernels = kernels

    def params(self) -> Mapping[str, ParamSpec]:
        """Tensors needed, by local name ("weight", "q_proj.weight", ...)."""
        return {}

    def load(self, tensors: Mapping[str, torch.Tensor]) -> None:
        """Receive the tensors named by ``params`` (on the GPU)."""

    def children(self) -> Mapping[str, "Part"]:
        """Sub-parts whose parameters live under ``<name>.`` of this part's names."""
        return {}

    # Per-step needs beyond the context's own fields.  Parts with the same ``step_inputs_key`` get one
    # shared set of arrays: the step function asks one of them and uploads the answer with the step.
    step_inputs_key: str | None = None

    def step_inputs(self, step: HostStep) -> Mapping[str, np.ndarray]:
        """int32 host arrays this part wants on the GPU for the step, by name (``ctx.inputs[name]``).
        Their shapes may depend on the number of sequences and tokens only when ``step.frozen``."""
        return {}

    def workspace_floats(self, step: HostStep) -> int:
        """float32 elements of ``ctx.workspace`` that this part's forward will ask for in this step."""
        return 0

    # False: the part's launches depend on the step's host numbers (``ctx.host_*``) and not only on the arrays
    # on the GPU, so a recorded step would repeat one step's numbers; a model with such a part is never recorded.
    replayable = True


class Norm(Part):
    def forward(self, x: torch.Tensor) -> torch.Tensor:
        raise NotImplementedError

    def forward_add(self, x: torch.Tensor, residual: torch.Tensor) -> torch.Tensor:
        """residual += x (in place); returns the norm of the sum."""
        raise NotImplementedError


class PositionEncoding(Part):
    def apply(self, q: torch.Tensor, k: torch.Tensor, positions: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
        """Encode positions into q [T, heads, d] and k [T, kv heads, d]."""
        raise NotImplementedError


class Mixer(Part):
    def cache_spec(self) -> KVPagesSpec | StateSlotSpec | None:
        return None

    def forward(self, x: torch.Tensor, ctx: StepContext, cache: PagedKV | StateSlots | None) -> torch.Tensor:
        raise NotImplementedError


class FeedForward(Part):
    def forward(self, x: torch.Tensor, ctx: StepContext) -> torch.Tensor:
        raise NotImplementedError


class Embedding(Part):
    def forward(self, ids: torch.Tensor) -> torch.Tensor:
        raise NotImplementedError


class Head(Part):
    def forward(self, x: torch.Tensor) -> torch.Tensor:
        raise NotImplementedError


class Block(Part):
    """The arrangement of a layer's parts.  It carries the pair (hidden,
    residual) of the reference's decoder (src/exec/dense_swiglu_decoder.rs:556-615)."""

    def forward(self, hidden: torch.Tensor, residual: torch.Tensor | None, ctx: StepContext,
                cache) -> tuple[torch.Tensor, torch.Tensor]:
        raise NotImplementedError
