"""Token embedding lookup ``h0 = E[ids]`` without scaling (utils/model.py:56-59,110)."""
from __future__ import annotations

from .base import MATRIX, ParamSpec, Part


class TokenEmbedding(Part):
    def __init__(self, vocab: int, width: int):
        self.vocab, self.width = vocab, width
        self.weight = None

    def param_specs(self):
        return {"weight": ParamSpec((self.vocab, self.width), MATRIX, "normal", share_per_token=0.0)}

    def assign(self, name, tensor):
        assert name == "weight"
        self.weight = tensor

    def forward(self, token_ids, ctx):
        out = ctx.empty((token_ids.shape[0], self.width))
        ctx.ops.embedding(self.weight, token_ids, out)
        return out
