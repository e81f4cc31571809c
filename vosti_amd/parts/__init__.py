from .base import (Block, Embedding, FeedForward, GroupTables, Head, HostStep, KVPagesSpec, Mixer, Norm, PagedKV, ParamSpec,
                   Part, PositionEncoding, StateSlotSpec, StateSlots, StepContext, build_part, register_part)
from . import standard  # registers the built-in parts

__all__ = ["Block", "Embedding", "FeedForward", "GroupTables", "Head", "HostStep", "KVPagesSpec", "Mixer", "Norm", "PagedKV",
           "ParamSpec", "Part", "PositionEncoding", "StateSlotSpec", "StateSlots", "StepContext", "build_part",
           "register_part", "standard"]
