"""The tests' own small configurations of the architecture; they differ in every size and option."""
from __future__ import annotations

from llmserver_amd.config import Qwen3Config, config_from_dict
from llmserver_amd.weights import RandomInit

TINY_A = dict(model_type="qwen3", num_hidden_layers=2, hidden_size=64, num_attention_heads=4, num_key_value_heads=2,
              head_dim=16, intermediate_size=128, vocab_size=256, rope_theta=10000.0, rms_norm_eps=1e-6,
              attention_bias=False, tie_word_embeddings=True)
TINY_A_INIT = RandomInit(seed=11, std=0.02, norm_noise=0.1)
TINY_A_PAGE = 16

TINY_B = dict(model_type="qwen3", num_hidden_layers=3, hidden_size=96, num_attention_heads=8, num_key_value_heads=2,
              head_dim=32, intermediate_size=224, vocab_size=384, rope_theta=1e6, rms_norm_eps=1e-5,
              attention_bias=True, tie_word_embeddings=False)
TINY_B_INIT = RandomInit(seed=23, std=0.03, norm_noise=0.1, bias_std=0.01)
TINY_B_PAGE = 8

# A third shape for what A and B do not reach: group of three heads, head size 48, odd vocabulary and width.
TINY_C = dict(model_type="qwen3", num_hidden_layers=2, hidden_size=72, num_attention_heads=6, num_key_value_heads=2,
              head_dim=48, intermediate_size=100, vocab_size=301, rope_theta=50000.0, rms_norm_eps=3e-6,
              attention_bias=False, tie_word_embeddings=False)
TINY_C_INIT = RandomInit(seed=5, std=0.05, norm_noise=0.2)
TINY_C_PAGE = 12

# A head size that is a multiple of 64: in bfloat16 steps of single tokens the attention kernel then normalises, rotates and
# writes the new key and value itself.  One KV head for five query heads.
TINY_D = dict(model_type="qwen3", num_hidden_layers=2, hidden_size=80, num_attention_heads=5, num_key_value_heads=1,
              head_dim=64, intermediate_size=176, vocab_size=200, rope_theta=2e5, rms_norm_eps=2e-6,
              attention_bias=False, tie_word_embeddings=True)
TINY_D_INIT = RandomInit(seed=37, std=0.05, norm_noise=0.15)
TINY_D_PAGE = 16

CASES = {"A": (TINY_A, TINY_A_INIT, TINY_A_PAGE), "B": (TINY_B, TINY_B_INIT, TINY_B_PAGE), "C": (TINY_C, TINY_C_INIT, TINY_C_PAGE),
         "D": (TINY_D, TINY_D_INIT, TINY_D_PAGE)}


def make_config(raw) -> Qwen3Config:
    return config_from_dict(dict(raw))
