"""Qwen3 dense decoder configuration, read from the keys of its ``config.json``.

Keys and defaults follow what the reference reads (utils/architecture.py:72-107):
``head_dim`` defaults to ``hidden_size // num_attention_heads`` (line 88) and need not multiply
back to the hidden size; ``rope_theta`` may sit at top level or inside ``rope_parameters`` /
``rope_scaling`` and defaults to 10000.0 (lines 23-30); ``rms_norm_eps`` has no default (106);
``num_key_value_heads``, when the file leaves it out, is the number of query heads (plain multi-head attention).
The refusals are the reference's (72-86, utils/attention.py:186-187).
"""
from __future__ import annotations

import dataclasses
from typing import Any, ClassVar, Mapping

from .base import ConfigError, ModelConfig, UnsupportedModelError, field

SUPPORTED_ACTIVATIONS = ("silu", "swish")


@dataclasses.dataclass(frozen=True)
class Qwen3Config(ModelConfig):
    MODEL_TYPE: ClassVar[str] = "qwen3"

    vocab_size: int = field("vocab_size", int)
    hidden_size: int = field("hidden_size", int)
    intermediate_size: int = field("intermediate_size", int)
    num_hidden_layers: int = field("num_hidden_layers", int)
    num_attention_heads: int = field("num_attention_heads", int)
    rms_norm_eps: float = field("rms_norm_eps", float)
    num_key_value_heads: int = field("num_key_value_heads", int, 0)
    head_dim: int = field("head_dim", int, 0)
    rope_theta: float = field("rope_theta", float, 0.0)
    attention_bias: bool = field("attention_bias", bool, False)
    tie_word_embeddings: bool = field("tie_word_embeddings", bool, False)
    hidden_act: str = field("hidden_act", str, "silu")
    max_position_embeddings: int = field("max_position_embeddings", int, 0)
    bos_token_id: object = field("bos_token_id", object, None)
    eos_token_id: object = field("eos_token_id", object, None)
    pad_token_id: object = field("pad_token_id", object, None)

    def resolve(self, raw: Mapping[str, Any]) -> "Qwen3Config":
        changes = {}
        if self.head_dim == 0:
            if self.num_attention_heads <= 0:
                raise ConfigError("num_attention_heads must be positive")
            changes["head_dim"] = self.hidden_size // self.num_attention_heads
        if self.num_key_value_heads == 0:            # absent: every query head has keys and values of its own
            changes["num_key_value_heads"] = self.num_attention_heads
        if self.rope_theta == 0.0:
            parameters = raw.get("rope_scaling") or raw.get("rope_parameters") or {}
            changes["rope_theta"] = float(parameters.get("rope_theta", 10000.0))
        return dataclasses.replace(self, **changes) if changes else self

    @property
    def group_size(self) -> int:
        return self.num_attention_heads // self.num_key_value_heads

    def validate(self, raw: Mapping[str, Any]) -> None:
        def reject(reason: str):
            raise UnsupportedModelError(f"Model type {self.MODEL_TYPE!r} is not supported: {reason}")

        for name in ("vocab_size", "hidden_size", "intermediate_size", "num_hidden_layers",
                     "num_attention_heads", "num_key_value_heads", "head_dim"):
            if getattr(self, name) <= 0:
                raise ConfigError(f"{name} must be positive: {getattr(self, name)}")
        if self.rms_norm_eps <= 0.0:
            raise ConfigError(f"rms_norm_eps must be positive: {self.rms_norm_eps}")
        if self.rope_theta <= 0.0:
            raise ConfigError(f"rope_theta must be positive: {self.rope_theta}")
        if self.num_attention_heads % self.num_key_value_heads != 0:
            reject("number of query heads must be divisible by the number of KV heads: "
                   f"query heads: {self.num_attention_heads}, KV heads: {self.num_key_value_heads}")
        if self.head_dim % 2 != 0:
            reject(f"rotate-half position encoding needs an even head_dim: {self.head_dim}")
        if self.head_dim % 16 != 0 or not 16 <= self.head_dim <= 256:
            reject(f"the attention kernels take head sizes 16, 32, ..., 256; got {self.head_dim}")
        use_sliding = raw.get("use_sliding_window")
        if use_sliding is None:
            use_sliding = raw.get("sliding_window") is not None
        if use_sliding or "sliding_attention" in (raw.get("layer_types") or []):
            reject("sliding-window attention is not implemented")
        for attribute in ("attn_logit_softcapping", "final_logit_softcapping"):
            if raw.get(attribute):
                reject(f"{attribute} is not implemented")
        if raw.get("partial_rotary_factor", 1.0) not in (1.0, None):
            reject("partial rotary embeddings are not implemented")
        if self.hidden_act not in SUPPORTED_ACTIVATIONS:
            reject(f"activation {self.hidden_act!r} is not supported (supported: {sorted(SUPPORTED_ACTIVATIONS)})")
        parameters = raw.get("rope_scaling") or raw.get("rope_parameters") or {}
        rope_type = parameters.get("rope_type", parameters.get("type", "default"))
        if rope_type not in (None, "default"):
            reject(f"RoPE type {rope_type!r} is not supported (supported: default)")
        if raw.get("mlp_bias"):
            reject("a biased MLP is not part of this architecture")
