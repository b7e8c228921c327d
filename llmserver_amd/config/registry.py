"""One registry from an architecture's name to its configuration class and model builder.

The reference keeps a tuple of verified ``model_type`` strings and refuses the rest with a
message that says what is supported (utils/architecture.py:16,48-54).  Here the
name maps to ``(config class, builder)``; a builder takes the typed config and returns a model
assembled from parts.  Registering another architecture is one call and changes no file here.
"""
from __future__ import annotations

from typing import Callable, Dict, Tuple, Type

from .base import ModelConfig, UnsupportedModelError, read_config_json

_ARCHITECTURES: Dict[str, Tuple[Type[ModelConfig], Callable]] = {}


def register_architecture(name: str, config_class: Type[ModelConfig], builder: Callable, *, replace: bool = False) -> None:
    """Map ``config.json["model_type"] == name`` to a config class and a model builder."""
    if name in _ARCHITECTURES and not replace:
        raise ValueError(f"architecture {name!r} is already registered")
    _ARCHITECTURES[name] = (config_class, builder)


def unregister_architecture(name: str) -> None:
    _ARCHITECTURES.pop(name, None)


def registered_architectures() -> tuple:
    return tuple(sorted(_ARCHITECTURES))


def resolve_architecture(name: str) -> Tuple[Type[ModelConfig], Callable]:
    if name not in _ARCHITECTURES:
        raise UnsupportedModelError(
            f"Model type {name!r} is not supported: registered architectures are {', '.join(registered_architectures()) or '(none)'}")
    return _ARCHITECTURES[name]


def config_from_dict(raw: dict) -> ModelConfig:
    name = raw.get("model_type")
    if not isinstance(name, str):
        raise UnsupportedModelError("config.json has no 'model_type' string naming the architecture")
    config_class, _ = resolve_architecture(name)
    return config_class.from_dict(raw)


def load_config(model_dir: str) -> ModelConfig:
    """Read ``model_dir/config.json`` into the typed config of the architecture it names."""
    return config_from_dict(read_config_json(model_dir))
