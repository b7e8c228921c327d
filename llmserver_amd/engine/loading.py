"""From a model folder to a model on the device, in the reference's manner
(utils/model_loader.py:18-86): the configuration picks the architecture, the
architecture's builder assembles the parts, the weights are streamed in by name."""
from __future__ import annotations

import torch

from .. import models  # noqa: F401  (registers the architectures)
from ..config import load_config, resolve_architecture
from ..weights import load_weights

DTYPES = {"bfloat16": torch.bfloat16, "bf16": torch.bfloat16, "float32": torch.float32, "fp32": torch.float32}


def parse_dtype(dtype) -> torch.dtype:
    if isinstance(dtype, torch.dtype):
        if dtype not in (torch.bfloat16, torch.float32):
            raise ValueError(f"the engine computes in bfloat16 or float32, not {dtype}")
        return dtype
    try:
        return DTYPES[str(dtype)]
    except KeyError:
        raise ValueError(f"unknown dtype {dtype!r}; choose bfloat16 or float32") from None


def load_model(model_dir: str, device="cuda", dtype="bfloat16"):
    """Read ``model_dir`` (config.json + safetensors) into a model on ``device``."""
    config = load_config(model_dir)
    _, builder = resolve_architecture(config.MODEL_TYPE)
    model = builder(config)
    model.name = model_dir
    load_weights(model, model_dir, torch.device(device), parse_dtype(dtype))
    return model
