"""Typed configuration of the Qwen3 dense decoder, read from config.json.

Reference: the twelve fields and their config.json keys are those of
src/models/qwen3/config.py:6-38; ``scale = 1/sqrt(head_dim)`` is derived as in
src/models/qwen3/config.py:46.  Unlike the reference no size has a default here:
a key that config.json lacks is an error, so that no model size stands in code.
"""
from __future__ import annotations

import json
import math
import os
from dataclasses import dataclass, asdict
from typing import Any, Dict, Tuple

from .spec import (AttentionSpec, LayerSpec, ModelSpec, RMSNormSpec, RopeSpec,
                   ScheduleEntry, SwiGLUSpec)

ARCHITECTURE = "Qwen3ForCausalLM"

_REQUIRED_INT = ("vocab_size", "hidden_size", "intermediate_size", "num_hidden_layers",
                 "num_attention_heads", "num_key_value_heads", "head_dim",
                 "max_position_embeddings")


class ConfigError(ValueError):
    """config.json lacks a key, or holds a value the engine does not model."""


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
    tie_word_embeddings: bool
    attention_bias: bool = False
    eos_token_ids: Tuple[int, ...] = ()
    architecture: str = ARCHITECTURE

    # ---- reading -------------------------------------------------------
    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> "Qwen3Config":
        missing = [k for k in _REQUIRED_INT + ("rms_norm_eps", "tie_word_embeddings") if k not in d]
        rope_parameters = d.get("rope_parameters") or {}
        # rope_parameters.rope_theta wins over rope_theta (src/models/qwen3/config.py:23,35)
        if "rope_theta" in rope_parameters:
            theta = rope_parameters["rope_theta"]
        elif "rope_theta" in d:
            theta = d["rope_theta"]
        else:
            theta = None
            missing.append("rope_theta")
        if missing:
            raise ConfigError("config.json lacks the keys: " + ", ".join(sorted(missing)))

        scaling = d.get("rope_scaling") or {}
        scaling_type = scaling.get("rope_type", scaling.get("type"))
        if scaling_type not in (None, "default"):
            raise ConfigError(f"rope scaling of type {scaling_type!r} is not modelled")
        rp_type = rope_parameters.get("rope_type", rope_parameters.get("type"))
        if rp_type not in (None, "default"):
            raise ConfigError(f"rope scaling of type {rp_type!r} is not modelled")
        if d.get("use_sliding_window", False):
            raise ConfigError("use_sliding_window=true is not modelled for Qwen3ForCausalLM")

        eos = d.get("eos_token_id", ())
        if eos is None:
            eos = ()
        elif isinstance(eos, int):
            eos = (eos,)
        cfg = cls(
            **{k: int(d[k]) for k in _REQUIRED_INT},
            rms_norm_eps=float(d["rms_norm_eps"]),
            rope_theta=float(theta),
            tie_word_embeddings=bool(d["tie_word_embeddings"]),
            attention_bias=bool(d.get("attention_bias", False)),
            eos_token_ids=tuple(int(e) for e in eos),
        )
        cfg.validate()
        return cfg

    @classmethod
    def from_folder(cls, folder: str) -> "Qwen3Config":
        with open(os.path.join(folder, "config.json")) as f:
            return cls.from_dict(json.load(f))

    def validate(self) -> None:
        for k in _REQUIRED_INT:
            if getattr(self, k) <= 0:
                raise ConfigError(f"{k} must be positive, got {getattr(self, k)}")
        if self.num_attention_heads % self.num_key_value_heads:
            raise ConfigError(
                f"num_attention_heads ({self.num_attention_heads}) is no multiple of "
                f"num_key_value_heads ({self.num_key_value_heads})")
        if self.head_dim % 2:
            raise ConfigError(f"head_dim ({self.head_dim}) must be even for the rotation")
        if not self.rms_norm_eps > 0:
            raise ConfigError("rms_norm_eps must be positive")
        if not self.rope_theta > 0:
            raise ConfigError("rope_theta must be positive")

    # ---- writing -------------------------------------------------------
    def to_dict(self) -> Dict[str, Any]:
        d = asdict(self)
        d.pop("architecture")
        eos = d.pop("eos_token_ids")
        d["architectures"] = [self.architecture]
        d["model_type"] = "qwen3"
        if eos:
            d["eos_token_id"] = eos[0] if len(eos) == 1 else list(eos)
        return d

    # ---- the model this configuration describes --------------------------
    def to_model_spec(self) -> ModelSpec:
        """Layers in the order of src/models/qwen3/model.py:278-298,349-359."""
        rope = RopeSpec(theta=self.rope_theta, rotary_dim=self.head_dim,
                        max_positions=self.max_position_embeddings)
        attention = AttentionSpec(
            num_heads=self.num_attention_heads,
            num_kv_heads=self.num_key_value_heads,
            head_dim=self.head_dim,
            scale=1.0 / math.sqrt(self.head_dim),
            qkv_bias=self.attention_bias,
            # per-head q/k norm exactly when there is no bias (src/models/qwen3/model.py:204-206)
            qk_norm_eps=None if self.attention_bias else self.rms_norm_eps,
            window=None,
            position=rope,
        )
        norm = RMSNormSpec(eps=self.rms_norm_eps)
        ffn = SwiGLUSpec(intermediate_size=self.intermediate_size)
        layers = tuple(
            LayerSpec(prefix=f"model.layers.{i}", mixer_norm=norm, mixer=attention,
                      ffn_norm=norm, ffn=ffn)
            for i in range(self.num_hidden_layers))
        spec = ModelSpec(
            architecture=self.architecture,
            vocab_size=self.vocab_size,
            hidden_size=self.hidden_size,
            layers=layers,
            schedule=tuple(ScheduleEntry(layer=i) for i in range(self.num_hidden_layers)),
            final_norm=norm,
            embed_name="model.embed_tokens.weight",
            final_norm_name="model.norm.weight",
            head_name="lm_head.weight",
            tie_head=self.tie_word_embeddings,
            max_positions=self.max_position_embeddings,
            eos_token_ids=self.eos_token_ids,
        )
        spec.validate()
        return spec
