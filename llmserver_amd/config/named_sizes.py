"""Model sizes that the command lines know by name, for runs with random weights: each entry is a ``config.json`` in
small, ``model_type`` included, so whoever asks for a name gets a configuration of whatever architecture the entry
names.  The sizes are those of published checkpoints (their ``config.json`` files) and of the tests' tiny models."""
from __future__ import annotations

from typing import Optional

from .base import ModelConfig
from .registry import config_from_dict

NAMED_SIZES = {
    "tiny-a": dict(model_type="qwen3", num_hidden_layers=2, hidden_size=64, num_attention_heads=4, num_key_value_heads=2, head_dim=16,
                   intermediate_size=128, vocab_size=256, rope_theta=10000.0, rms_norm_eps=1e-6, tie_word_embeddings=True),
    "tiny-b": dict(model_type="qwen3", num_hidden_layers=3, hidden_size=96, num_attention_heads=8, num_key_value_heads=2, head_dim=32,
                   intermediate_size=224, vocab_size=384, rope_theta=1e6, rms_norm_eps=1e-5, attention_bias=True),
    "qwen3-0.6b": dict(model_type="qwen3", num_hidden_layers=28, hidden_size=1024, num_attention_heads=16, num_key_value_heads=8,
                       head_dim=128, intermediate_size=3072, vocab_size=151936, rope_theta=1e6, rms_norm_eps=1e-6,
                       tie_word_embeddings=True),
    "qwen3-1.7b": dict(model_type="qwen3", num_hidden_layers=28, hidden_size=2048, num_attention_heads=16, num_key_value_heads=8,
                       head_dim=128, intermediate_size=6144, vocab_size=151936, rope_theta=1e6, rms_norm_eps=1e-6,
                       tie_word_embeddings=True),
    "qwen3-4b": dict(model_type="qwen3", num_hidden_layers=36, hidden_size=2560, num_attention_heads=32, num_key_value_heads=8,
                     head_dim=128, intermediate_size=9728, vocab_size=151936, rope_theta=1e6, rms_norm_eps=1e-6,
                     tie_word_embeddings=True),
    "qwen3-8b": dict(model_type="qwen3", num_hidden_layers=36, hidden_size=4096, num_attention_heads=32, num_key_value_heads=8,
                     head_dim=128, intermediate_size=12288, vocab_size=151936, rope_theta=1e6, rms_norm_eps=1e-6),
    "qwen3-14b": dict(model_type="qwen3", num_hidden_layers=40, hidden_size=5120, num_attention_heads=40, num_key_value_heads=8,
                      head_dim=128, intermediate_size=17408, vocab_size=151936, rope_theta=1e6, rms_norm_eps=1e-6),
    "qwen3-32b": dict(model_type="qwen3", num_hidden_layers=64, hidden_size=5120, num_attention_heads=64, num_key_value_heads=8,
                      head_dim=128, intermediate_size=25600, vocab_size=151936, rope_theta=1e6, rms_norm_eps=1e-6),
}


def named_size(name: str) -> dict:
    """The entry's keys, a copy the caller may change (fewer layers, say)."""
    try:
        return dict(NAMED_SIZES[name])
    except KeyError:
        raise KeyError(f"no size is named {name!r}; known: {', '.join(sorted(NAMED_SIZES))}") from None


def named_config(name: str, layers: Optional[int] = None) -> ModelConfig:
    """The typed configuration of a named size, with at most ``layers`` layers if given (shapes do not depend on depth)."""
    raw = named_size(name)
    if layers:
        raw["num_hidden_layers"] = min(int(raw["num_hidden_layers"]), int(layers))
    return config_from_dict(raw)
