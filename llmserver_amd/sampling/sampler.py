"""Greedy and temperature sampling over the step's float32 logits.

The reference's engine samples with ``argmax`` only (/root/reference/utils/engine.py:295-297).
Temperature sampling draws from ``softmax(logits / temperature)`` (computed in 32-bit) by
inverting the cumulative distribution at a uniform number; the numbers come from a generator
seeded per request, so a request's tokens do not depend on what shares its batch.
"""
from __future__ import annotations

import random
from typing import List, Sequence

import numpy as np
import torch


def request_uniform(seed: int, draw: int) -> float:
    """The ``draw``-th uniform number in [0, 1) of a request's own generator."""
    return random.Random(f"{seed}:{draw}").random()


class Sampler:
    def __init__(self, ops, device):
        self.ops, self.device = ops, torch.device(device)

    def sample(self, logits: torch.Tensor, temperatures: Sequence[float], uniforms: Sequence[float]) -> List[int]:
        """One token per row of ``logits [n, vocab]``; temperature 0 takes the first maximum."""
        if logits.shape[0] == 0:
            return []
        return self.launch(logits, temperatures, uniforms).tolist()

    def launch(self, logits: torch.Tensor, temperatures: Sequence[float], uniforms: Sequence[float]) -> torch.Tensor:
        """Start the sampling of one token per row and return the int32 device tensor they will be in: whoever reads
        it (``tolist()``) waits for the step; until then the host is free for other work."""
        n = logits.shape[0]
        host = np.empty((2, n), dtype=np.float32)
        host[0] = temperatures
        host[1] = uniforms
        both = torch.from_numpy(host).to(self.device, non_blocking=True)
        out = torch.empty(n, dtype=torch.int32, device=self.device)
        self.ops.sample(logits, both[0], both[1], out)
        return out
