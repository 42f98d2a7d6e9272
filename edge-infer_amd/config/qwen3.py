"""Typed configuration of the Qwen3 dense decoder, read from config.json keys.

Key names, required/optional status and admission checks follow the reference:
bindings/python/model_initializer.cpp:12-52,131-140 (keys, rejected options) and
runtime/include/models/qwen3_model.hpp:139-206 (value checks, default head_dim).
"""
from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Any, Mapping

from .specs import (AttentionSpec, GatedMLPSpec, LayerSpec, ModelSpec, NormSpec, PositionSpec,
                    default_schedule)

ARCHITECTURE = "Qwen3ForCausalLM"
_INT_MAX = 2**31 - 1


class ConfigError(ValueError):
    pass


def _positive_int(source: Mapping[str, Any], key: str) -> int:
    if key not in source:
        raise ConfigError(f"config.json lacks required key '{key}'")
    value = source[key]
    if isinstance(value, bool) or not isinstance(value, (int, float)):
        raise ConfigError(f"config.json key '{key}' must be a positive integer, got {value!r}")
    if not math.isfinite(value) or value < 1 or int(value) != value or value > _INT_MAX:
        raise ConfigError(f"config.json key '{key}' must be a positive integer, got {value!r}")
    return int(value)


def _token_id(source: Mapping[str, Any], key: str) -> int:
    if key not in source:
        raise ConfigError(f"config.json lacks required key '{key}'")
    value = source[key]
    if isinstance(value, bool) or not isinstance(value, (int, float)) or value < 0 \
            or int(value) != value or value > 2**32 - 1:
        raise ConfigError(f"config.json key '{key}' must be a token id, got {value!r}")
    return int(value)


def _positive_float(source: Mapping[str, Any], key: str) -> float:
    if key not in source:
        raise ConfigError(f"config.json lacks required key '{key}'")
    value = source[key]
    if isinstance(value, bool) or not isinstance(value, (int, float)) \
            or not math.isfinite(value) or value <= 0:
        raise ConfigError(f"config.json key '{key}' must be a positive finite number, got {value!r}")
    return float(value)


@dataclass(frozen=True)
class Qwen3Config:
    vocab_size: int
    hidden_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    intermediate_size: int
    max_position_embeddings: int
    bos_token_id: int
    eos_token_id: int
    rms_norm_eps: float
    rope_theta: float
    tie_word_embeddings: bool = False
    hidden_act: str = "silu"

    architecture = ARCHITECTURE

    @classmethod
    def from_dict(cls, source: Mapping[str, Any]) -> "Qwen3Config":
        # options the decoder does not implement are refused, never ignored
        if "hidden_act" in source and source["hidden_act"] != "silu":
            raise ConfigError("only SiLU-gated feed-forward layers are supported "
                              f"(hidden_act={source['hidden_act']!r})")
        scaling = source.get("rope_scaling")
        if scaling is not None and not (isinstance(scaling, dict) and len(scaling) == 0):
            raise ConfigError("scaled or multi-axis rotary encodings are not supported "
                              f"(rope_scaling={scaling!r})")
        sliding = bool(source.get("use_sliding_window", False)) if "use_sliding_window" in source \
            else (source.get("sliding_window") is not None and source.get("sliding_window", 0) > 0)
        if sliding:
            raise ConfigError("sliding-window attention is not part of this architecture's decoder")
        layer_types = source.get("layer_types")
        if layer_types is not None and any(t != "full_attention" for t in layer_types):
            raise ConfigError("only full-attention layers are supported "
                              f"(layer_types={layer_types!r})")
        tie = source.get("tie_word_embeddings", False)
        if not isinstance(tie, bool):
            raise ConfigError("tie_word_embeddings must be a boolean")

        hidden = _positive_int(source, "hidden_size")
        heads = _positive_int(source, "num_attention_heads")
        if "head_dim" in source and source["head_dim"] is not None:
            head_dim = _positive_int(source, "head_dim")
        else:
            if hidden % heads:
                raise ConfigError("hidden_size must be divisible by num_attention_heads "
                                  "when head_dim is absent")
            head_dim = hidden // heads
        config = cls(
            vocab_size=_positive_int(source, "vocab_size"),
            hidden_size=hidden,
            num_hidden_layers=_positive_int(source, "num_hidden_layers"),
            num_attention_heads=heads,
            num_key_value_heads=_positive_int(source, "num_key_value_heads"),
            head_dim=head_dim,
            intermediate_size=_positive_int(source, "intermediate_size"),
            max_position_embeddings=_positive_int(source, "max_position_embeddings"),
            bos_token_id=_token_id(source, "bos_token_id"),
            eos_token_id=_token_id(source, "eos_token_id"),
            rms_norm_eps=_positive_float(source, "rms_norm_eps"),
            rope_theta=_positive_float(source, "rope_theta"),
            tie_word_embeddings=tie,
        )
        config.validate()
        return config

    def validate(self) -> None:
        if self.num_attention_heads % self.num_key_value_heads:
            raise ConfigError("num_attention_heads must be a multiple of num_key_value_heads")
        if self.head_dim % 2:
            raise ConfigError("head_dim must be even for the rotary encoding")
        if self.num_attention_heads > 65535:
            raise ConfigError("num_attention_heads exceeds 65535")
        for name in ("num_attention_heads", "num_key_value_heads"):
            if getattr(self, name) * self.head_dim > _INT_MAX:
                raise ConfigError(f"{name} * head_dim exceeds the supported integer range")

    def to_dict(self) -> dict:
        """config.json content that `from_dict` reads back to an equal object."""
        return {
            "architectures": [ARCHITECTURE],
            "model_type": "qwen3",
            "vocab_size": self.vocab_size,
            "hidden_size": self.hidden_size,
            "num_hidden_layers": self.num_hidden_layers,
            "num_attention_heads": self.num_attention_heads,
            "num_key_value_heads": self.num_key_value_heads,
            "head_dim": self.head_dim,
            "intermediate_size": self.intermediate_size,
            "max_position_embeddings": self.max_position_embeddings,
            "bos_token_id": self.bos_token_id,
            "eos_token_id": self.eos_token_id,
            "rms_norm_eps": self.rms_norm_eps,
            "rope_theta": self.rope_theta,
            "tie_word_embeddings": self.tie_word_embeddings,
            "hidden_act": self.hidden_act,
        }

    # ------------------------------------------------------------------
    def model_spec(self) -> ModelSpec:
        """Every layer: pre-norm block of q/k-normed rotary GQA and a SwiGLU MLP.
        runtime/include/execution/decoder.hpp:119-169."""
        norm = NormSpec(kind="rmsnorm", eps=self.rms_norm_eps)
        position = PositionSpec(kind="rope", theta=self.rope_theta, dim=self.head_dim,
                                max_positions=self.max_position_embeddings)
        mixer = AttentionSpec(
            n_heads=self.num_attention_heads, n_kv_heads=self.num_key_value_heads,
            head_dim=self.head_dim, qk_norm=True, qk_norm_eps=self.rms_norm_eps,
            window=None, scale=None, position=position)
        ffn = GatedMLPSpec(intermediate_size=self.intermediate_size, activation=self.hidden_act)
        layer = LayerSpec(block="prenorm", norm=norm, mixer=mixer, feed_forward=ffn)
        spec = ModelSpec(
            architecture=ARCHITECTURE, vocab_size=self.vocab_size, hidden_size=self.hidden_size,
            layers=tuple(layer for _ in range(self.num_hidden_layers)),
            schedule=default_schedule(self.num_hidden_layers), final_norm=norm,
            tie_word_embeddings=self.tie_word_embeddings,
            max_position_embeddings=self.max_position_embeddings,
            bos_token_id=self.bos_token_id, eos_token_id=self.eos_token_id)
        spec.validate()
        return spec

    # ------------------------------------------------------------------
    @staticmethod
    def checkpoint_name(parameter: str) -> str:
        """Name of a model parameter in the checkpoint.
        bindings/python/include/decoder_weight_mapper.hpp:114-162 (read backwards)."""
        if parameter == "embed.weight":
            return "model.embed_tokens.weight"
        if parameter == "final_norm.weight":
            return "model.norm.weight"
        if parameter == "head.weight":
            return "lm_head.weight"
        if parameter == "head.bias":
            return "lm_head.bias"
        parts = parameter.split(".")
        if parts[0] == "layers" and len(parts) >= 4:
            prefix = f"model.layers.{parts[1]}."
            rest = ".".join(parts[2:])
            table = {
                "norm1.weight": "input_layernorm.weight",
                "norm2.weight": "post_attention_layernorm.weight",
                "mixer.q_proj.weight": "self_attn.q_proj.weight",
                "mixer.k_proj.weight": "self_attn.k_proj.weight",
                "mixer.v_proj.weight": "self_attn.v_proj.weight",
                "mixer.o_proj.weight": "self_attn.o_proj.weight",
                "mixer.q_norm.weight": "self_attn.q_norm.weight",
                "mixer.k_norm.weight": "self_attn.k_norm.weight",
                "ffn.gate_proj.weight": "mlp.gate_proj.weight",
                "ffn.up_proj.weight": "mlp.up_proj.weight",
                "ffn.down_proj.weight": "mlp.down_proj.weight",
            }
            for path, name in list(table.items()):      # the optional bias of each projection
                if "_proj." in path:
                    table[path[:-len("weight")] + "bias"] = name[:-len("weight")] + "bias"
            if rest in table:
                return prefix + table[rest]
        raise KeyError(f"Qwen3 has no checkpoint tensor for parameter '{parameter}'")

    # alternative checkpoint names that mean the same parameter
    checkpoint_aliases = {"model.lm_head.weight": "lm_head.weight",
                          "model.lm_head.bias": "lm_head.bias"}
