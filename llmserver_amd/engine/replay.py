"""Trace replay: feeds given token ids through a model step by step and writes logits.

It samples nothing and has no forward pass, cache or loader of its own: it drives the model,
the step function, the cache manager and the kernels that generation uses.  Steps arrive as
JSON objects, one per line::

    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}

All entries of a step form one batch.  ``want`` lists the places among an entry's tokens whose
logits are asked for; they are written to ``<out>/<step>.f32`` as little-endian float32
``[wanted, vocab]`` in the order of the entries and of ``want``.  Requests named in ``end`` give
back what they hold after the step.
"""
from __future__ import annotations

import json
import os
import sys
from typing import Iterable, TextIO

import torch

from ..cache import CacheManager
from .batch import StepEntry
from .loading import load_model, parse_dtype
from .step import ModelRunner

MAX_LIVE_REQUESTS = 4


def make_runner(model_dir: str, dtype, max_tokens: int, page_size: int = 16, device="cuda", ops=None,
                max_live: int = MAX_LIVE_REQUESTS) -> ModelRunner:
    """Load the model and a cache pool for ``max_tokens`` tokens (rounded up to whole pages)."""
    dtype = parse_dtype(dtype)
    model = load_model(model_dir, device, dtype)
    if ops is None:
        from ..kernels import default_ops
        ops = default_ops()
    specs = model.cache_specs()
    head_dims = sorted({spec.head_dim for spec in specs.values() if hasattr(spec, "head_dim")})
    ops.preload(head_dims, dtype)
    pages = max(1, -(-max_tokens // page_size))
    cache = CacheManager(specs, page_size, pages, num_state_slots=max_live, device=model.device, dtype=dtype,
                         model_identity=model_dir)
    return ModelRunner(model, cache, ops)


def replay(runner: ModelRunner, lines: Iterable[str], out_dir: str, report: TextIO = sys.stdout) -> int:
    """Run every step of ``lines``; returns the number of steps run."""
    os.makedirs(out_dir, exist_ok=True)
    count = 0
    for line in lines:
        line = line.strip()
        if not line:
            continue
        record = json.loads(line)
        step = record["step"]
        entries = []
        for item in record.get("entries", []):
            if not runner.cache.has(item["id"]):
                runner.cache.open(item["id"])
            entries.append(StepEntry(item["id"], item["tokens"], item.get("want", [])))
        if entries:
            logits = runner.step(entries)
            if logits.shape[0]:
                array = logits.to(torch.float32).cpu().numpy().astype("<f4", copy=False)
                array.tofile(os.path.join(out_dir, f"{step}.f32"))
            elif runner.device.type == "cuda":
                torch.cuda.synchronize()
        for request_id in record.get("end", []):
            if runner.cache.has(request_id):
                runner.cache.close(request_id)
        print(f"done {step}", file=report, flush=True)
        count += 1
    return count
