"""Shared helpers of the tests: model folders in temporary places, traces, comparisons."""
from __future__ import annotations

import functools
import os
import tempfile

import numpy as np
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


BF16 = plain.rounding_to(torch.bfloat16)


@functools.lru_cache(maxsize=None)
def rounded_logits(case: str, count: int, seed: int):
    """The plain implementation with its intermediate results rounded to bfloat16 where the reference's kernels round."""
    config, tensors = plain_model(case)
    return plain.forward(config, tensors, random_tokens(config["vocab_size"], count, seed), r=BF16)


def relative_error(got, exact) -> float:
    """Largest difference of one position's logits, in units of those logits' own largest magnitude."""
    got, exact = np.asarray(got, dtype=np.float64), np.asarray(exact, dtype=np.float64)
    size = float(np.abs(exact).max())
    return float(np.abs(got - exact).max()) / (size if size > 0 else 1.0)


ROUNDING_FACTOR = 1.25       # measured over the suite's configurations: 0.85 to 1.0 (the engine rounds q, k and SwiGLU once
                             # where the reference's kernels round twice), the worst single place up to 1.04


def check_against_rounded_oracle(engine_errors, rounded_errors, what, factor=ROUNDING_FACTOR):
    """A bfloat16 run may lose what bfloat16 loses, not more: its errors against the exact oracle (one per position,
    :func:`relative_error`) are held against the errors of the oracle that rounds where the reference's kernels round,
    over the same sequences.  Position by position the two are different draws of one spread (another order of sums
    rounds another way), so the spreads are compared: the median and the 99th percentile within ``factor`` of the
    rounded oracle's, the worst place (one draw from the tail) within 1.2 times ``factor``.  Median and percentile need
    a few dozen places to mean anything."""
    engine, rounded = np.asarray(engine_errors, dtype=np.float64), np.asarray(rounded_errors, dtype=np.float64)
    assert np.isfinite(engine).all() and np.isfinite(rounded).all() and len(engine) and len(rounded), what
    figures = {"median": (np.median(engine), np.median(rounded)), "99th percentile": (np.quantile(engine, 0.99), np.quantile(rounded, 0.99)),
               "worst": (engine.max(), rounded.max())}
    print(f"  {what}: bfloat16 error / rounded oracle's: " +
          ", ".join(f"{name} {ours:.2e} / {theirs:.2e}" for name, (ours, theirs) in figures.items()), flush=True)
    for name, (ours, theirs) in figures.items():
        if name != "worst" and len(engine) < 48:
            continue
        allowed = factor * (1.2 if name == "worst" else 1.0)
        assert ours <= allowed * theirs, f"{what}: {name} error {ours:.3e} is more than {allowed} x the rounded oracle's {theirs:.3e}"


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
