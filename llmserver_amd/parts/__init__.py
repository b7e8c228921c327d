from .attention import AttentionNames, AttentionPlan, AttentionTuning, GQAttention, TileLaunchCost, build_attention_plan, group_tiling
from .base import (INT_TABLE, MATRIX, VECTOR, Block, FeedForward, Mixer, Norm, PagedKVSpec, ParamSpec, Part,
                   PositionEncoding, StateSpec)
from .block import PreNormBlock
from .embedding import TokenEmbedding
from .kernel_namespace import KernelNamespace
from .linear import Linear
from .mlp import GatedMLP, GatedMLPNames
from .norm import RMSNorm
from .rope import NoPosition, RotaryPosition

__all__ = ["KernelNamespace", "AttentionNames", "AttentionTuning", "TileLaunchCost", "GatedMLPNames", "AttentionPlan", "GQAttention", "build_attention_plan", "group_tiling", "INT_TABLE", "MATRIX", "VECTOR",
           "Block", "FeedForward", "Mixer", "Norm", "PagedKVSpec", "ParamSpec", "Part", "PositionEncoding",
           "StateSpec", "PreNormBlock", "TokenEmbedding", "Linear", "GatedMLP", "RMSNorm", "NoPosition",
           "RotaryPosition"]
