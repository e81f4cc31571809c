"""Configuration of the Qwen3 dense decoder, read from config.json.

The key set and the rules are those of the reference's profile projection
(python/vosti_kernels/model_families/qwen3/profile.py:41-61 for the keys,
:129-164 for the rules; typed twin src/boundary/model_families/qwen3/config.rs:9-18
and src/model_config.rs:32-41).  The reference additionally demands equality
with one of two sealed profiles and fixes eps and theta
(qwen3/physical.py:29-32); here every valid geometry is admitted and both are
parameters.
"""
from __future__ import annotations

import math
from dataclasses import asdict, dataclass
from typing import Any, Mapping

from .registry import ConfigError, register_architecture
from .spec import LayerSpec, ModelSpec, PartSpec, ScheduleEntry

_MISSING = object()


def _get(raw: Mapping[str, Any], key: str, default: Any = _MISSING) -> Any:
    if key in raw and raw[key] is not None:
        return raw[key]
    if default is _MISSING:
        raise ConfigError(f"config.json: required key {key!r} is missing")
    return default


def _pos_int(raw: Mapping[str, Any], key: str, default: Any = _MISSING) -> int:
    v = _get(raw, key, default)
    if isinstance(v, bool) or not isinstance(v, int) or v <= 0:
        raise ConfigError(f"config.json: {key!r} must be a positive integer, got {v!r}")
    return v


def _pos_float(raw: Mapping[str, Any], key: str, default: Any = _MISSING) -> float:
    v = _get(raw, key, default)
    if isinstance(v, bool) or not isinstance(v, (int, float)) or not math.isfinite(float(v)) or v <= 0:
        raise ConfigError(f"config.json: {key!r} must be a finite positive number, got {v!r}")
    return float(v)


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

    # ------------------------------------------------------------- parsing
    @classmethod
    def from_dict(cls, raw: Mapping[str, Any]) -> "Qwen3Config":
        if raw.get("model_type", "qwen3") != "qwen3":
            raise ConfigError(f"config.json: 'model_type' is {raw.get('model_type')!r}, expected 'qwen3'")
        hidden = _pos_int(raw, "hidden_size")
        heads = _pos_int(raw, "num_attention_heads")
        kv_heads = _pos_int(raw, "num_key_value_heads", heads)
        if "head_dim" in raw and raw["head_dim"] is not None:
            head_dim = _pos_int(raw, "head_dim")
        else:
            if hidden % heads:
                raise ConfigError("config.json: 'head_dim' is absent and 'hidden_size' is not a multiple of 'num_attention_heads'")
            head_dim = hidden // heads
        if heads % kv_heads:
            raise ConfigError(f"config.json: 'num_attention_heads' ({heads}) must be a multiple of 'num_key_value_heads' ({kv_heads})")
        if head_dim % 2:
            raise ConfigError(f"config.json: 'head_dim' ({head_dim}) must be even")
        if _get(raw, "hidden_act", "silu") != "silu":
            raise ConfigError(f"config.json: 'hidden_act' is {raw['hidden_act']!r}; this architecture uses 'silu'")
        if _get(raw, "attention_bias", False) is not False:
            raise ConfigError("config.json: 'attention_bias' must be false")
        if float(_get(raw, "attention_dropout", 0.0)) != 0.0:
            raise ConfigError("config.json: 'attention_dropout' must be 0")
        if _get(raw, "use_sliding_window", False) is not False:
            raise ConfigError("config.json: 'use_sliding_window' must be false: this architecture attends to all keys")
        layer_types = raw.get("layer_types")
        if layer_types is not None and any(t != "full_attention" for t in layer_types):
            raise ConfigError("config.json: 'layer_types' must name 'full_attention' for every layer")
        rope_theta = raw.get("rope_theta")
        rope_params = raw.get("rope_parameters")
        scaling = raw.get("rope_scaling")
        if isinstance(rope_params, Mapping):
            if rope_theta is None:
                rope_theta = rope_params.get("rope_theta")
            if rope_params.get("rope_type", "default") != "default":
                scaling = rope_params
        if scaling is not None and not (isinstance(scaling, Mapping) and scaling.get("rope_type", scaling.get("type")) == "default"):
            raise ConfigError("config.json: 'rope_scaling' must be null: only the default rotary encoding is built")
        tie = _get(raw, "tie_word_embeddings", False)
        if not isinstance(tie, bool):
            raise ConfigError("config.json: 'tie_word_embeddings' must be true or false")
        # A model without layers is lm_head(rms_norm(embed)) (src/exec/dense_swiglu_model.rs:276-359).
        layers = _get(raw, "num_hidden_layers")
        if isinstance(layers, bool) or not isinstance(layers, int) or layers < 0:
            raise ConfigError(f"config.json: 'num_hidden_layers' must be an integer, zero or more, got {layers!r}")
        if layer_types is not None and len(layer_types) != layers:
            raise ConfigError("config.json: 'layer_types' must have one entry per layer")
        return cls(
            vocab_size=_pos_int(raw, "vocab_size"),
            hidden_size=hidden,
            intermediate_size=_pos_int(raw, "intermediate_size"),
            num_hidden_layers=layers,
            num_attention_heads=heads,
            num_key_value_heads=kv_heads,
            head_dim=head_dim,
            max_position_embeddings=_pos_int(raw, "max_position_embeddings"),
            rms_norm_eps=_pos_float(raw, "rms_norm_eps"),
            rope_theta=_pos_float({"rope_theta": rope_theta}, "rope_theta"),
            tie_word_embeddings=tie,
        )

    def to_dict(self) -> dict[str, Any]:
        d = asdict(self)
        arch = d.pop("architecture")
        d.update({
            "architectures": [arch], "model_type": "qwen3", "hidden_act": "silu", "attention_bias": False,
            "attention_dropout": 0.0, "use_sliding_window": False, "sliding_window": None, "rope_scaling": None,
        })
        return d

    # --------------------------------------------------------- description
    def model_spec(self) -> ModelSpec:
        """The decoder as data: pre-norm blocks of attention and SwiGLU
        (src/exec/dense_swiglu_decoder.rs:43-441), every layer alike, run once
        each in order (src/exec/dense_swiglu_model.rs:131-1041)."""
        norm = PartSpec("rmsnorm", {"size": self.hidden_size, "eps": self.rms_norm_eps})
        head_norm = PartSpec("rmsnorm", {"size": self.head_dim, "eps": self.rms_norm_eps})
        rope = PartSpec("rotary", {"head_dim": self.head_dim, "rotary_dim": self.head_dim, "theta": self.rope_theta,
                                    "max_positions": self.max_position_embeddings})
        mixer = PartSpec("attention", {
            "hidden_size": self.hidden_size, "num_heads": self.num_attention_heads,
            "num_kv_heads": self.num_key_value_heads, "head_dim": self.head_dim,
            "scale": self.head_dim ** -0.5, "window": 0, "q_norm": head_norm, "k_norm": head_norm, "position": rope,
        })
        ffn = PartSpec("swiglu", {"hidden_size": self.hidden_size, "intermediate_size": self.intermediate_size})
        layers = []
        for i in range(self.num_hidden_layers):
            p = f"model.layers.{i}."
            layers.append(LayerSpec(
                block="prenorm", mixer=mixer, feed_forward=ffn,
                norms={"input": norm, "post_mixer": norm},
                names={
                    "norms.input.weight": p + "input_layernorm.weight",
                    "norms.post_mixer.weight": p + "post_attention_layernorm.weight",
                    "mixer.q_proj.weight": p + "self_attn.q_proj.weight",
                    "mixer.k_proj.weight": p + "self_attn.k_proj.weight",
                    "mixer.v_proj.weight": p + "self_attn.v_proj.weight",
                    "mixer.o_proj.weight": p + "self_attn.o_proj.weight",
                    "mixer.q_norm.weight": p + "self_attn.q_norm.weight",
                    "mixer.k_norm.weight": p + "self_attn.k_norm.weight",
                    "feed_forward.gate_proj.weight": p + "mlp.gate_proj.weight",
                    "feed_forward.up_proj.weight": p + "mlp.up_proj.weight",
                    "feed_forward.down_proj.weight": p + "mlp.down_proj.weight",
                }))
        spec = ModelSpec(
            architecture=self.architecture,
            vocab_size=self.vocab_size,
            hidden_size=self.hidden_size,
            max_positions=self.max_position_embeddings,
            embedding=PartSpec("token_embedding", {"vocab_size": self.vocab_size, "hidden_size": self.hidden_size}),
            layers=tuple(layers),
            schedule=tuple(ScheduleEntry(i) for i in range(self.num_hidden_layers)),
            final_norm=norm,
            head=PartSpec("linear_head", {"vocab_size": self.vocab_size, "hidden_size": self.hidden_size,
                                          "tied": self.tie_word_embeddings}),
            # A tied head is the embedding table itself (python/vosti_kernels/model_families/qwen3/physical.py:131-134);
            # a checkpoint that stores an lm_head.weight beside it is tolerated.
            names={"embedding.weight": "model.embed_tokens.weight", "final_norm.weight": "model.norm.weight",
                   "head.weight": "model.embed_tokens.weight" if self.tie_word_embeddings else "lm_head.weight"},
            ignored_names=("lm_head.weight",) if self.tie_word_embeddings else (),
        )
        spec.validate()
        return spec
