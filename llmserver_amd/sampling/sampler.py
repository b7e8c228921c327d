"""Greedy and temperature sampling over the step's float32 logits.

The reference's engine samples with ``argmax`` only (utils/engine.py:295-297).
Temperature sampling draws from ``softmax(logits / temperature)`` (computed in 32-bit) by
inverting the cumulative distribution at a uniform number; the numbers come from a generator
seeded per request, so a request's tokens do not depend on what shares its batch.
"""
from __future__ import annotations

import random
from typing import List, Sequence

import torch


def request_uniform(seed: int, draw: int) -> float:
    """The ``draw``-th uniform number in [0, 1) of a request's own generator."""
    return random.Random(f"{seed}:{draw}").random()


class PendingTokens:
    """Sampled tokens on their way to the host: ``device`` is the int32 tensor the kernels write, and a copy into
    pinned host memory follows them in the stream.  :meth:`tolist` waits for that copy only, so work that is put
    into the stream afterwards (the next step, started ahead) does not hold the tokens back."""

    def __init__(self, device: torch.Tensor, host: torch.Tensor):
        self.device = device
        self._host = host[:device.shape[0]]
        self._host.copy_(device, non_blocking=True)
        self._copied = None
        if device.is_cuda:
            self._copied = torch.cuda.Event()
            self._copied.record()

    def tolist(self) -> List[int]:
        if self._copied is not None:
            self._copied.synchronize()
        return self._host.tolist()


class Sampler:
    def __init__(self, ops, device):
        self.ops, self.device = ops, torch.device(device)
        self._host_buffers = []          # pinned buffers (sampled tokens on their way back, temperatures on their way there), used in turn
        self._turn = 0
        self._greedy = {}                # rows -> zeros on the device for steps without a temperature

    def sample(self, logits: torch.Tensor, temperatures: Sequence[float], uniforms: Sequence[float]) -> List[int]:
        """One token per row of ``logits [n, vocab]``; temperature 0 takes the first maximum."""
        if logits.shape[0] == 0:
            return []
        return self.launch(logits, temperatures, uniforms).tolist()

    def _host_buffer(self, n: int) -> torch.Tensor:
        pinned = self.device.type == "cuda"
        if len(self._host_buffers) < 8:
            self._host_buffers.append(torch.empty(max(n, 256), dtype=torch.int32, pin_memory=pinned))
        self._turn = (self._turn + 1) % len(self._host_buffers)
        if self._host_buffers[self._turn].shape[0] < n:
            self._host_buffers[self._turn] = torch.empty(2 * n, dtype=torch.int32, pin_memory=pinned)
        return self._host_buffers[self._turn]

    def launch(self, logits: torch.Tensor, temperatures: Sequence[float], uniforms: Sequence[float]) -> PendingTokens:
        """Start the sampling of one token per row, and the copy of the tokens to the host behind it; whoever reads
        them (``tolist()``) waits for that copy; until then the host is free for other work."""
        n = logits.shape[0]
        if not any(temperatures):
            both = self._greedy.get(n)               # greedy rows read neither their temperature's inverse nor a number
            if both is None:
                both = self._greedy[n] = torch.zeros((2, n), dtype=torch.float32, device=self.device)
        else:
            # Through pinned memory: a copy from pageable memory would make the host wait for everything the stream
            # still has to do, the running step included.
            staged = self._host_buffer(2 * n).view(torch.float32)[:2 * n].view(2, n)
            staged[0] = torch.as_tensor(temperatures, dtype=torch.float32)
            staged[1] = torch.as_tensor(uniforms, dtype=torch.float32)
            both = staged.to(self.device, non_blocking=True)
        out = torch.empty(n, dtype=torch.int32, device=self.device)
        self.ops.sample(logits, both[0], both[1], out)
        return PendingTokens(out, self._host_buffer(n))
