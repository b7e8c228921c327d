"""What a step has to read and to multiply, summed over what the model's parts declare.

Nothing here knows an architecture: weights come from ``param_specs()`` of the embedding, the blocks, the final norm and
the head (each tensor with the share of it that one token uses, :class:`~llmserver_amd.parts.base.ParamSpec`), caches
from ``cache_specs()``, and what a mixer computes beyond its projections from ``Mixer.mixing_flops``.  The benchmark's
roofline figures are these sums over the model it runs, whatever that model is made of.
"""
from __future__ import annotations

import dataclasses
import math
from typing import Dict, Iterable, Sequence

import torch

from ..parts.base import MATRIX, PagedKVSpec, ParamSpec, StateSpec


@dataclasses.dataclass(frozen=True)
class StepRow:
    """One request's share of a step: ``new_tokens`` tokens that end at a context of ``context`` tokens, the logits of
    ``wanted`` of them asked for."""
    new_tokens: int
    context: int
    wanted: int = 1


def _element_bytes(spec: ParamSpec, compute_dtype: torch.dtype) -> int:
    return torch.empty((), dtype=compute_dtype).element_size() if spec.role == MATRIX else 4


def _bytes_read(spec: ParamSpec, rows: int, compute_dtype: torch.dtype) -> float:
    """Bytes of one tensor that ``rows`` tokens read together: all of it if every token uses all of it; the rows
    that are looked up if it is a table read by row; and if a token uses a share p of it (one of several experts),
    the expected share that at least one of the tokens uses, 1 - (1 - p)^rows."""
    if rows <= 0:
        return 0.0
    size = math.prod(spec.shape) * _element_bytes(spec, compute_dtype)
    if spec.share_per_token >= 1.0:
        return float(size)
    if spec.share_per_token <= 0.0:
        return float(min(rows, spec.shape[0]) * size // max(1, spec.shape[0]))
    return size * (1.0 - (1.0 - spec.share_per_token) ** rows)


def _flops(spec: ParamSpec, rows: int) -> float:
    """A multiply and an add for every element of a matrix that a token uses; vectors and tables count nothing."""
    if spec.role != MATRIX or len(spec.shape) < 2:
        return 0.0
    return 2.0 * rows * math.prod(spec.shape) * spec.share_per_token


def _weights(model) -> Dict[str, Iterable[ParamSpec]]:
    return {"embedding": model.embedding.param_specs().values(),
            "blocks": [spec for block in model.blocks for spec in block.param_specs().values()],
            "final_norm": model.final_norm.param_specs().values(), "head": model.head.param_specs().values()}


def cache_bytes(model, rows: Sequence[StepRow], dtype: torch.dtype) -> float:
    """What the step's rows read of their caches: the keys and values of a row's context (of its window, where the
    layer has one) for every call of the order that reads a paged cache, the state of a row for every call with one."""
    element = torch.empty((), dtype=dtype).element_size()
    total = 0.0
    for call in model.order:
        spec = model.blocks[call.block].mixer.cache_spec()
        if isinstance(spec, PagedKVSpec):
            keys = sum(min(row.context, spec.window) if spec.window else row.context for row in rows)
            total += 2.0 * spec.n_kv_heads * spec.head_dim * element * keys
        elif isinstance(spec, StateSpec):
            total += math.prod(spec.shape) * torch.empty((), dtype=getattr(torch, spec.dtype)).element_size() * len(rows)
    return total


def step_bytes(model, rows: Sequence[StepRow], dtype: torch.dtype) -> float:
    """Bytes that a step of these rows has to read at least: every weight it uses once (a block that the order calls
    twice is still read once), and the caches of its rows."""
    tokens = sum(row.new_tokens for row in rows)
    wanted = sum(row.wanted for row in rows)
    weights = _weights(model)
    total = sum(_bytes_read(spec, tokens, dtype) for part in ("embedding", "blocks") for spec in weights[part])
    total += sum(_bytes_read(spec, wanted, dtype) for part in ("final_norm", "head") for spec in weights[part])
    return total + cache_bytes(model, rows, dtype)


def step_flops(model, rows: Sequence[StepRow]) -> float:
    """Floating-point operations of a step of these rows: the matrices of every call of the order for every token, the
    head for the wanted places, and what the mixers compute between their projections."""
    tokens = sum(row.new_tokens for row in rows)
    wanted = sum(row.wanted for row in rows)
    total = sum(_flops(spec, wanted) for spec in model.head.param_specs().values())
    for call in model.order:
        block = model.blocks[call.block]
        total += sum(_flops(spec, tokens) for spec in block.param_specs().values())
        total += sum(block.mixer.mixing_flops(row.new_tokens, row.context) for row in rows)
    return total
