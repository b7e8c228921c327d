"""Fills a model's parts with checkpoint tensors, by tensor name.

Matrices follow the compute dtype (bfloat16 for serving, float32 on the 32-bit path); small
per-channel vectors are held in float32, which keeps a vector stored in 32-bit as it is and
widens a bfloat16 one without loss; integer tables become int32.  The reference loads each
module strictly, so a missing or unexpected name raises (utils/model_loader.py:
49-52); here every problem of the folder is collected first and reported in one error.  The
output head is tied to the embedding when the configuration says so or the checkpoint has no
head (utils/model_loader.py:56-59).
"""
from __future__ import annotations

import torch

from ..parts.base import INT_TABLE, MATRIX, VECTOR
from .reader import CheckpointReader


class WeightsError(ValueError):
    """The tensors of a model folder do not fit the model: lists missing, unexpected, misshapen."""

    def __init__(self, directory, missing, unexpected, wrong_shape):
        self.missing, self.unexpected, self.wrong_shape = list(missing), list(unexpected), list(wrong_shape)
        lines = [f"weights in {directory!r} do not fit the model:"]
        if self.missing:
            lines.append(f"  missing tensors ({len(self.missing)}): " + ", ".join(self.missing))
        if self.unexpected:
            lines.append(f"  unexpected tensors ({len(self.unexpected)}): " + ", ".join(self.unexpected))
        if self.wrong_shape:
            lines.append(f"  wrong shapes ({len(self.wrong_shape)}): " + ", ".join(
                f"{name}: file {tuple(found)} != model {tuple(wanted)}" for name, found, wanted in self.wrong_shape))
        super().__init__("\n".join(lines))


def stored_dtype(role: str, compute_dtype: torch.dtype) -> torch.dtype:
    if role == MATRIX:
        return compute_dtype
    if role == VECTOR:
        return torch.float32
    if role == INT_TABLE:
        return torch.int32
    raise ValueError(f"unknown tensor role {role!r}")


def check_names(model, reader: CheckpointReader):
    specs = model.param_specs()
    ignored = model.ignored_names()
    present = set(reader.names())
    missing = sorted(name for name, spec in specs.items() if name not in present and not spec.optional and name not in ignored)
    unexpected = sorted(name for name in present if name not in specs)
    wrong = []
    for name in sorted(present & set(specs)):
        if name in ignored:
            continue
        found = reader.shape(name)
        if tuple(found) != tuple(specs[name].shape):
            wrong.append((name, found, specs[name].shape))
    return missing, unexpected, wrong


def load_weights(model, model_dir: str, device, dtype: torch.dtype) -> None:
    reader = CheckpointReader(model_dir)
    try:
        missing, unexpected, wrong = check_names(model, reader)
        if missing or unexpected or wrong:
            raise WeightsError(model_dir, missing, unexpected, wrong)
        specs = model.param_specs()
        ignored = model.ignored_names()
        assigned = []
        for name, spec in specs.items():
            if name in ignored or not reader.has(name):
                continue
            tensor = reader.get(name).to(device=device, dtype=stored_dtype(spec.role, dtype)).contiguous()
            model.assign(name, tensor)
            assigned.append(name)
        model.finalize(assigned, device, dtype)
    finally:
        reader.close()
