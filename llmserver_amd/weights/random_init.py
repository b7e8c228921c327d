"""Seeded random weights: writes a model folder from a configuration and a seed.

The reference's loader has no such mode; its tests seed a generator and draw every parameter
from a normal distribution (tests/test_paged_decode.py:273-277).  Here each
tensor is drawn from a generator seeded by (seed, tensor name), so the values do not depend on
the order of tensors: matrices ``N(0, std)``, norm weights ``1 + N(0, norm_noise)``, biases
``N(0, bias_std)``.
"""
from __future__ import annotations

import dataclasses
import hashlib
import json
import os

import torch

from ..config.base import ModelConfig
from ..config.registry import resolve_architecture
from ..parts.base import INT_TABLE, ParamSpec
from .loader import stored_dtype


@dataclasses.dataclass(frozen=True)
class RandomInit:
    seed: int = 0
    std: float = 0.02
    norm_noise: float = 0.0
    bias_std: float = 0.01


def _generator(seed: int, name: str, device="cpu") -> torch.Generator:
    digest = hashlib.sha256(f"{seed}:{name}".encode()).digest()
    generator = torch.Generator(device=device)
    generator.manual_seed(int.from_bytes(digest[:8], "little") & 0x7FFFFFFFFFFFFFFF)
    return generator


def random_tensor(name: str, spec: ParamSpec, init: RandomInit, device="cpu") -> torch.Tensor:
    """The float32 (or int32) values of one tensor."""
    generator = _generator(init.seed, name, device)
    if spec.role == INT_TABLE:
        return torch.randint(0, 2 ** 15, spec.shape, generator=generator, device=device, dtype=torch.int32)
    values = torch.randn(spec.shape, generator=generator, device=device, dtype=torch.float32)
    if spec.init == "norm":
        return 1.0 + init.norm_noise * values
    if spec.init == "bias":
        return init.bias_std * values
    if spec.init == "zeros":
        return torch.zeros_like(values)
    return init.std * values


def build_model(config: ModelConfig):
    _, builder = resolve_architecture(config.MODEL_TYPE)
    return builder(config)


def write_random_model(config: ModelConfig, folder: str, init: RandomInit = RandomInit(),
                       dtype: torch.dtype = torch.bfloat16) -> str:
    """Write ``folder/config.json`` and ``folder/model.safetensors`` (all floats stored as ``dtype``)."""
    from safetensors.torch import save_file

    os.makedirs(folder, exist_ok=True)
    model = build_model(config)
    ignored = model.ignored_names()
    tensors = {}
    for name, spec in model.param_specs().items():
        if name in ignored:
            continue
        values = random_tensor(name, spec, init)
        tensors[name] = values if spec.role == INT_TABLE else values.to(dtype)
    save_file(tensors, os.path.join(folder, "model.safetensors"))
    os.chmod(os.path.join(folder, "model.safetensors"), 0o644)       # readable by whoever runs the model, as config.json is
    with open(os.path.join(folder, "config.json"), "w") as handle:
        json.dump(config.to_dict(), handle, indent=1)
    return folder


def random_model_on_device(config: ModelConfig, device, dtype: torch.dtype, init: RandomInit = RandomInit()):
    """A model whose tensors are drawn on the device itself (no file; for large benchmark sizes)."""
    model = build_model(config)
    ignored = model.ignored_names()
    assigned = []
    for name, spec in model.param_specs().items():
        if name in ignored:
            continue
        values = random_tensor(name, spec, init, device=device)
        model.assign(name, values.to(stored_dtype(spec.role, dtype)))
        assigned.append(name)
        del values
    model.finalize(assigned, device, dtype)
    return model
