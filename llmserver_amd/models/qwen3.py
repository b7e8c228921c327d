"""Qwen3 dense decoder put together from parts, layer by layer, from its typed configuration.

Layer kinds and tensor names as the reference has them (/root/reference/utils/model.py:7-54,
/root/reference/utils/attention.py:33-39, /root/reference/utils/layers.py:188-191,
/root/reference/utils/model_loader.py:54-67): pre-norm blocks of grouped-query attention with
per-head q/k RMSNorm and rotate-half RoPE, and a SwiGLU feed-forward; one eps for every norm
(/root/reference/utils/model.py:10-12, /root/reference/utils/attention.py:38-39).
"""
from __future__ import annotations

from ..config.qwen3 import Qwen3Config
from ..config.registry import register_architecture
from ..parts import GatedMLP, GQAttention, Linear, PreNormBlock, RMSNorm, RotaryPosition, TokenEmbedding
from .decoder import DecoderModel


def build_qwen3(config: Qwen3Config) -> DecoderModel:
    position = RotaryPosition(config.head_dim, config.rope_theta)
    blocks = []
    for _ in range(config.num_hidden_layers):
        attention = GQAttention(config.hidden_size, config.num_attention_heads, config.num_key_value_heads,
                                config.head_dim, position, qk_norm_eps=config.rms_norm_eps,
                                bias=config.attention_bias)
        mlp = GatedMLP(config.hidden_size, config.intermediate_size, config.hidden_act)
        blocks.append(PreNormBlock(RMSNorm(config.hidden_size, config.rms_norm_eps), attention,
                                   RMSNorm(config.hidden_size, config.rms_norm_eps), mlp))
    head = Linear(config.hidden_size, ("lm_head",), (config.vocab_size,), bias=False, out_float32=True)
    return DecoderModel(config, TokenEmbedding(config.vocab_size, config.hidden_size), blocks,
                        RMSNorm(config.hidden_size, config.rms_norm_eps), head, tie_head=config.tie_word_embeddings)


register_architecture("qwen3", Qwen3Config, build_qwen3, replace=True)
