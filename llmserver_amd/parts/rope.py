"""Rotate-half rotary position encoding over the full head.

``inv_freq_i = theta^(-2i/d)`` for ``i = 0..d/2-1``, ``angle = position * inv_freq`` in 32-bit,
``x' = x*cos + rotate_half(x)*sin`` with ``rotate_half(x) = cat(-x[d/2:], x[:d/2])``
(utils/layers.py:140-177).  Positions are absolute token positions
(utils/batch.py:30,80).  The table of inverse frequencies is made once on the
host with the reference's expression (utils/layers.py:158); the rotation itself
happens inside the mixer's fused kernel, which gets the table and the positions of the step's
tokens, so a position depends on nothing but the token's own index.
"""
from __future__ import annotations

import torch

from .base import PositionEncoding


class RotaryPosition(PositionEncoding):
    def __init__(self, rotary_dim: int, theta: float):
        if rotary_dim % 2:
            raise ValueError(f"rotary_dim must be even: {rotary_dim}")
        self.rotary_dim = rotary_dim
        self.theta = float(theta)
        self._tables = {}

    def inverse_frequencies(self) -> torch.Tensor:
        indices = torch.arange(0, self.rotary_dim, 2, dtype=torch.long)
        return 1.0 / (self.theta ** (indices.to(torch.float32) / self.rotary_dim))

    def rotary_table(self, device):
        key = str(device)
        if key not in self._tables:
            self._tables[key] = self.inverse_frequencies().to(device=device, dtype=torch.float32).contiguous()
        return self._tables[key]

    def cos_sin(self, ctx):
        """cos and sin of the step's tokens, float32 ``[T, rotary_dim]``: computed once a step, whatever
        the number of layers that rotate with this encoding."""
        return ctx.computed(("rotary", id(self)), lambda: ctx.ops.rotary_table(ctx.positions, self.rotary_table(ctx.device)))


class NoPosition(PositionEncoding):
    """Tokens enter the mixer unrotated."""
