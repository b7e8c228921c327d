"""Qwen3 dense decoder put together from parts, layer by layer, from its typed configuration.

Layer kinds and tensor names as the reference has them (utils/model.py:7-54,
utils/attention.py:33-39, utils/layers.py:188-191,
utils/model_loader.py:54-67): pre-norm blocks of grouped-query attention with
per-head q/k RMSNorm and rotate-half RoPE, and a SwiGLU feed-forward; one eps for every norm
(utils/model.py:10-12, utils/attention.py:38-39).
"""
from __future__ import annotations

from ..config.qwen3 import Qwen3Config
from ..config.registry import register_architecture
from ..parts import (AttentionNames, GatedMLP, GatedMLPNames, GQAttention, Linear, PreNormBlock, RMSNorm, RotaryPosition,
                     TokenEmbedding)
from .decoder import DecoderModel

# The checkpoint's tensor names (utils/attention.py:33-39, utils/layers.py:188-191, utils/model.py:10-13,46-54 in the reference).
ATTENTION_NAMES = AttentionNames(qkv=("q_proj", "k_proj", "v_proj"), out="o_proj", q_norm="q_norm", k_norm="k_norm")
MLP_NAMES = GatedMLPNames(gate_up=("gate_proj", "up_proj"), down="down_proj")
BLOCK_NAMES = ("input_layernorm", "self_attn", "post_attention_layernorm", "mlp")
MODEL_NAMES = ("model.embed_tokens", "model.layers", "model.norm")
HEAD_NAME = "lm_head"


def build_qwen3(config: Qwen3Config) -> DecoderModel:
    position = RotaryPosition(config.head_dim, config.rope_theta)
    blocks = []
    for _ in range(config.num_hidden_layers):
        attention = GQAttention(config.hidden_size, config.num_attention_heads, config.num_key_value_heads,
                                config.head_dim, position, qk_norm_eps=config.rms_norm_eps,
                                bias=config.attention_bias, names=ATTENTION_NAMES)
        mlp = GatedMLP(config.hidden_size, config.intermediate_size, config.hidden_act, names=MLP_NAMES)
        blocks.append(PreNormBlock(RMSNorm(config.hidden_size, config.rms_norm_eps), attention,
                                   RMSNorm(config.hidden_size, config.rms_norm_eps), mlp, names=BLOCK_NAMES))
    head = Linear(config.hidden_size, (HEAD_NAME,), (config.vocab_size,), bias=False, out_float32=True)
    return DecoderModel(config, TokenEmbedding(config.vocab_size, config.hidden_size), blocks,
                        RMSNorm(config.hidden_size, config.rms_norm_eps), head, tie_head=config.tie_word_embeddings,
                        names=MODEL_NAMES)


register_architecture("qwen3", Qwen3Config, build_qwen3, replace=True)
