"""The flat batch of one step and everything the kernels need to know about it.

A step carries, for each request in it, the next tokens of that request: a portion of its
prompt or one decoded token, cut anywhere.  All of them are laid end to end as ``T`` tokens.
Per token: id, absolute position, request row.  Per row: where its tokens start, how many there
are, and the context length after the step.  Per cache group: the rows' block tables.  Every
integer array is staged in one pinned host buffer and reaches the GPU in one copy, the
reference's static-header idea (utils/cuda_graph.py:29-34, 86-95) extended to
mixed batches, which the reference never forms (utils/batch.py:4-81).
"""
from __future__ import annotations

import dataclasses
from typing import Dict, List, Optional, Sequence

import numpy as np
import torch


@dataclasses.dataclass
class StepEntry:
    """One request's share of a step: its next tokens and the places whose logits are wanted."""
    request_id: object
    tokens: Sequence[int]
    want: Sequence[int] = ()


class Staging:
    """One int32 buffer on the host (pinned where possible) mirrored on the device."""

    def __init__(self, device, capacity: int = 1 << 16):
        self.device = torch.device(device)
        self.capacity = 0
        self.used = 0
        self._copied = None       # event after the last upload: the host buffer is free again once it has passed
        self._grow(capacity)

    def _grow(self, capacity: int):
        on_gpu = self.device.type == "cuda"
        self.host = torch.empty(capacity, dtype=torch.int32, pin_memory=on_gpu)
        self.host_np = self.host.numpy()
        self.dev = torch.empty(capacity, dtype=torch.int32, device=self.device) if on_gpu else self.host
        self.capacity = capacity

    def reset(self, needed: int = 0, may_grow: bool = True):
        if self._copied is not None:
            self._copied.synchronize()
            self._copied = None
        self.used = 0
        if needed > self.capacity:
            if not may_grow:
                raise RuntimeError("staging buffer of a captured step is too small")
            self._grow(max(needed, 2 * self.capacity))

    def stage(self, array: np.ndarray) -> torch.Tensor:
        """Copy ``array`` into the host buffer; returns the device view (valid after upload)."""
        array = np.ascontiguousarray(array, dtype=np.int32)
        count = array.size
        start = self.used
        if start + count > self.capacity:
            raise RuntimeError("staging buffer too small; reset() it with the needed size")
        self.host_np[start:start + count] = array.reshape(-1)
        self.used = start + ((count + 3) // 4) * 4          # keep every array 16-byte aligned
        return self.dev[start:start + count].view(array.shape)

    def upload(self):
        if self.dev is not self.host and self.used:
            self.dev[:self.used].copy_(self.host[:self.used], non_blocking=True)
            self._copied = torch.cuda.Event()
            self._copied.record()


class StepContext:
    """What the parts see of a step."""

    def __init__(self, ops, device, dtype, staging: Staging):
        self.ops, self.device, self.dtype, self.staging = ops, torch.device(device), dtype, staging
        self._plans: Dict[object, dict] = {}
        self._computed: Dict[object, object] = {}
        self._tables: Dict[int, torch.Tensor] = {}
        self.static_max_keys: Optional[int] = None      # set when the step's array shapes must be fixed (graph capture)
        self.page_size = None                           # keys a page of the cache holds, if the maker of the step says

    # -- building ------------------------------------------------------------------------
    def fill(self, token_ids, positions, token_row, row_start, row_len, row_ctx, logit_idx, tables: List[np.ndarray],
             state_slots: Optional[np.ndarray], request_ids: List[object]):
        self.h_token_ids = np.asarray(token_ids, dtype=np.int32)
        self.h_positions = np.asarray(positions, dtype=np.int32)
        self.h_token_row = np.asarray(token_row, dtype=np.int32)
        self.h_row_start = np.asarray(row_start, dtype=np.int32)
        self.h_row_len = np.asarray(row_len, dtype=np.int32)
        self.h_row_ctx = np.asarray(row_ctx, dtype=np.int32)
        self.h_logit_idx = np.asarray(logit_idx, dtype=np.int32)
        self.h_tables = tables
        self.h_state_slots = state_slots
        self.request_ids = list(request_ids)
        self.n_tokens, self.n_rows, self.n_out = len(self.h_token_ids), len(self.h_row_len), len(self.h_logit_idx)

    def upload(self):
        """Stage every host array of the step (the batch's and the mixers' plans) and copy once."""
        self.stage()
        self.staging.upload()

    def set_token_ids(self, token_ids: np.ndarray) -> None:
        """Replace the token ids of a step that is staged but not yet copied (see ``ModelRunner.prepare_ahead``)."""
        if token_ids.shape != self.h_token_ids.shape:
            raise ValueError(f"{token_ids.shape[0]} token ids for a step of {self.h_token_ids.shape[0]} tokens")
        self.h_token_ids = np.ascontiguousarray(token_ids, dtype=np.int32)
        self.staging.host_np[self._token_ids_at:self._token_ids_at + self.h_token_ids.size] = self.h_token_ids

    def stage(self):
        """Lay every host array of the step out in the staging buffer; nothing is copied yet."""
        plan_arrays = [(plan, name) for plan in self._plans.values() for name, value in plan.items()
                       if isinstance(value, np.ndarray)]
        arrays = [self.h_token_ids, self.h_positions, self.h_token_row, self.h_row_start, self.h_row_len, self.h_row_ctx,
                  self.h_logit_idx, *self.h_tables]
        if self.h_state_slots is not None:
            arrays.append(self.h_state_slots)
        needed = sum(a.size + 4 for a in arrays) + sum(plan[name].size + 4 for plan, name in plan_arrays)
        self.staging.reset(needed, may_grow=self.static_max_keys is None)
        self.layout = tuple(a.shape for a in arrays) + tuple(plan[name].shape for plan, name in plan_arrays)
        stage = self.staging.stage
        self._token_ids_at = self.staging.used
        self.token_ids, self.positions, self.token_row = stage(self.h_token_ids), stage(self.h_positions), stage(self.h_token_row)
        self.row_start, self.row_len, self.row_ctx = stage(self.h_row_start), stage(self.h_row_len), stage(self.h_row_ctx)
        self.logit_idx = stage(self.h_logit_idx)
        self._tables = {group: stage(table) for group, table in enumerate(self.h_tables)}
        self.state_slots = stage(self.h_state_slots) if self.h_state_slots is not None else None
        for plan, name in plan_arrays:
            plan[name] = stage(plan[name])

    # -- used by the parts ---------------------------------------------------------------------
    def empty(self, shape, dtype=None):
        return torch.empty(shape, device=self.device, dtype=dtype or self.dtype)

    def block_table(self, group: int) -> torch.Tensor:
        return self._tables[group]

    def computed(self, key, make):
        """A value computed on the device once per run of the step's kernels (e.g. the rotation
        table of a position encoding), shared by all layers that ask for it under ``key``."""
        if key not in self._computed:
            self._computed[key] = make()
        return self._computed[key]

    def forget_computed(self):
        """Before the step's kernels are recorded again (graph capture after an eager run)."""
        self._computed.clear()

    def has_plan(self, key) -> bool:
        return key in self._plans

    def set_plan(self, key, plan: dict):
        self._plans[key] = plan

    def get_plan(self, key) -> dict:
        return self._plans[key]
