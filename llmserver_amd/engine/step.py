"""The step function: a batch of (request, its next tokens) in, logits at the wanted places out.

It runs only the tokens it is given, as one flat batch, against the cache earlier steps left:
portions of prompts beside single decoded tokens, cut anywhere.  The reference runs two kinds of
forward per engine step, padded prefill batches and a decode batch
(/root/reference/utils/engine.py:437-443, /root/reference/utils/model.py:76-158); here there is
one pass, and one code path serves generation, the benchmark and trace replay.
"""
from __future__ import annotations

from typing import List, Sequence

import numpy as np
import torch

from ..cache.manager import CacheManager
from .batch import Staging, StepContext, StepEntry


class ModelRunner:
    def __init__(self, model, cache: CacheManager, ops=None):
        if ops is None:
            from ..kernels import default_ops
            ops = default_ops()
        self.model, self.cache, self.ops = model, cache, ops
        self.device, self.dtype = model.device, model.dtype
        self._staging = [Staging(self.device), Staging(self.device)]
        self._flip = 0
        self.vocab = model.head.out_features

    def build_context(self, entries: Sequence[StepEntry]) -> StepContext:
        """Check the entries against the cache, allocate their pages, lay out the flat batch."""
        if not entries:
            raise ValueError("a step needs at least one entry")
        seen = set()
        token_ids: List[int] = []
        positions: List[int] = []
        token_row: List[int] = []
        row_start, row_len, row_ctx, logit_idx, request_ids = [], [], [], [], []
        for row, entry in enumerate(entries):
            if entry.request_id in seen:
                raise ValueError(f"request {entry.request_id!r} appears twice in one step")
            seen.add(entry.request_id)
            tokens = list(entry.tokens)
            if not tokens:
                raise ValueError(f"request {entry.request_id!r} brings no tokens")
            for token in tokens:
                if not 0 <= token < self.vocab:
                    raise ValueError(f"token id {token} of request {entry.request_id!r} is outside the vocabulary of {self.vocab}")
            record = self.cache.record(entry.request_id)
            start = record.num_computed
            for place in entry.want:
                if not 0 <= place < len(tokens):
                    raise ValueError(f"wanted place {place} is outside the {len(tokens)} tokens of request {entry.request_id!r}")
                logit_idx.append(len(token_ids) + place)
            row_start.append(len(token_ids))
            row_len.append(len(tokens))
            row_ctx.append(start + len(tokens))
            request_ids.append(entry.request_id)
            token_ids.extend(tokens)
            positions.extend(range(start, start + len(tokens)))
            token_row.extend([row] * len(tokens))
        taken = []
        try:
            for entry, ctx_len in zip(entries, row_ctx):
                self.cache.ensure(entry.request_id, ctx_len)
                taken.append(entry.request_id)
        except Exception:
            raise
        tables = []
        for group in self.cache.groups:
            width = max(1, max(len(self.cache.record(rid).tables[group.index]) for rid in request_ids))
            table = np.full((len(entries), width), -1, dtype=np.int32)
            for row, rid in enumerate(request_ids):
                pages = self.cache.record(rid).tables[group.index]
                table[row, :len(pages)] = pages
            tables.append(table)
        slots = None
        if self.cache.state_specs:
            slots = np.asarray([self.cache.record(rid).state_slot for rid in request_ids], dtype=np.int32)
        self._flip ^= 1
        ctx = StepContext(self.ops, self.device, self.dtype, self._staging[self._flip])
        ctx.fill(token_ids, positions, token_row, row_start, row_len, row_ctx, logit_idx, tables, slots, request_ids)
        return ctx

    @torch.inference_mode()
    def step(self, entries: Sequence[StepEntry]) -> torch.Tensor:
        """Run one step; returns float32 logits ``[wanted, vocab]`` in the order of the entries and their ``want``."""
        ctx = self.build_context(entries)
        self.model.prepare(ctx)
        ctx.upload()
        logits = self.model.forward(ctx, self.cache)
        for rid, ctx_len in zip(ctx.request_ids, ctx.h_row_ctx):
            self.cache.advance(rid, int(ctx_len))
        return logits
