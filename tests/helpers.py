"""Shared helpers of the tests: model folders in temporary places, traces, comparisons."""
from __future__ import annotations

import functools
import os
import tempfile

import torch

import plain_qwen3 as plain
from llmserver_amd.weights import write_random_model
from tiny_configs import CASES, make_config

_FOLDERS = {}


def model_folder(case: str) -> str:
    """A temporary model folder of a tiny case (made once per test session, never in the tree)."""
    if case not in _FOLDERS:
        raw, init, _ = CASES[case]
        folder = tempfile.mkdtemp(prefix=f"llmserver_amd_test_{case}_")
        write_random_model(make_config(raw), folder, init)
        _FOLDERS[case] = folder
    return _FOLDERS[case]


@functools.lru_cache(maxsize=None)
def plain_model(case: str):
    return plain.read_folder(model_folder(case))


def random_tokens(vocab: int, count: int, seed: int):
    generator = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (count,), generator=generator).tolist()


@functools.lru_cache(maxsize=None)
def plain_logits(case: str, count: int, seed: int):
    config, tensors = plain_model(case)
    return plain.forward(config, tensors, random_tokens(config["vocab_size"], count, seed))


def portions(total: int, sizes):
    """Cut ``range(total)`` into consecutive pieces of the given sizes, the last one taking the rest."""
    cuts, start = [], 0
    for size in sizes:
        if start >= total:
            break
        end = min(total, start + size)
        cuts.append((start, end))
        start = end
    if start < total:
        cuts.append((start, total))
    return cuts
