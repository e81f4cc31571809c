"""Configuration of the Qwen3 dense decoder, read from config.json.

The key set and the rules are those of the reference's profile projection
(python/vosti_kernels/model_families/qwen3/profile.py:41-61 for the keys,
:129-164 for the rules; typed twin src/boundary/model_families/qwen3/config.rs:9-18
and src/model_config.rs:32-41).  The reference additionally demands equality
with one of two sealed profiles and fixes eps and theta
(qwen3/physical.py:29-32); here every valid geometry is admitted and both are
parameters.

The rules themselves are written once, in the native library
(csrc/host/qwen3.cpp: ``qwen3_config`` checks the keys, ``qwen3_model_spec``
describes the model as parts), which the native engine uses directly.  This
class is the typed face of the same thing for Python callers: ``from_dict``
hands the raw keys to the library and keeps the typed values it returns, and
``model_spec`` is the library's description turned into this package's
``ModelSpec``.
"""
from __future__ import annotations

from dataclasses import asdict, dataclass
from typing import Any, Mapping

from .registry import describe, register_architecture, spec_from_description
from .spec import ModelSpec


@register_architecture("Qwen3ForCausalLM", model_type="qwen3")
@dataclass(frozen=True)
class Qwen3Config:
    vocab_size: int
    hidden_size: int
    intermediate_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    max_position_embeddings: int
    rms_norm_eps: float
    rope_theta: float
    tie_word_embeddings: bool = False
    architecture: str = "Qwen3ForCausalLM"

    @classmethod
    def from_dict(cls, raw: Mapping[str, Any]) -> "Qwen3Config":
        """Checks the keys (``ConfigError`` names the one at fault) and returns the typed values, defaults
        filled in (kv heads, head size, the newer spelling of theta)."""
        return cls(**describe(dict(raw, architectures=["Qwen3ForCausalLM"]))["config"])

    def to_dict(self) -> dict[str, Any]:
        d = asdict(self)
        arch = d.pop("architecture")
        d.update({
            "architectures": [arch], "model_type": "qwen3", "hidden_act": "silu", "attention_bias": False,
            "attention_dropout": 0.0, "use_sliding_window": False, "sliding_window": None, "rope_scaling": None,
        })
        return d

    def model_spec(self) -> ModelSpec:
        """The decoder as data: pre-norm blocks of attention and SwiGLU
        (src/exec/dense_swiglu_decoder.rs:43-441), every layer alike, run once
        each in order (src/exec/dense_swiglu_model.rs:131-1041)."""
        spec = spec_from_description(describe(self.to_dict()))
        spec.validate()
        return spec
