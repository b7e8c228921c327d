"""Typed model configuration: the base class every architecture's config derives from.

A configuration is read from the architecture's own ``config.json`` keys and nothing else; no
size or constant that ``config.json`` gives is repeated in code.  The reference builds an untyped
kwargs dict from a library config object (utils/architecture.py:90-107); here the
file is parsed directly into a frozen dataclass whose ``validate`` gives every refusal a reason
(utils/architecture.py:50-86).
"""
from __future__ import annotations

import dataclasses
import json
import os
from typing import Any, ClassVar, Mapping


class UnsupportedModelError(ValueError):
    """A model folder describes something this engine does not implement.

    Same role as utils/architecture.py:19.
    """


class ConfigError(ValueError):
    """A ``config.json`` is malformed: a required key is missing or a value has the wrong type."""


_MISSING = object()


def field(key: str, kind: type, default: Any = _MISSING, doc: str = ""):
    """A dataclass field bound to one ``config.json`` key."""
    meta = {"key": key, "kind": kind, "doc": doc, "required": default is _MISSING}
    if default is _MISSING:
        return dataclasses.field(metadata=meta)
    return dataclasses.field(default=default, metadata=meta)


def _coerce(name: str, kind: type, value: Any) -> Any:
    if kind is float and isinstance(value, (int, float)) and not isinstance(value, bool):
        return float(value)
    if kind is int and isinstance(value, int) and not isinstance(value, bool):
        return value
    if kind is bool and isinstance(value, bool):
        return value
    if kind is str and isinstance(value, str):
        return value
    if kind is object:
        return value
    raise ConfigError(f"config key {name!r} must be {kind.__name__}, got {value!r}")


@dataclasses.dataclass(frozen=True)
class ModelConfig:
    """Base of all architecture configurations.

    Subclasses declare their keys with :func:`field` and implement :meth:`validate`.
    ``model_type`` names the architecture in the registry.
    """

    MODEL_TYPE: ClassVar[str] = ""

    @classmethod
    def from_dict(cls, raw: Mapping[str, Any]) -> "ModelConfig":
        values = {}
        for f in dataclasses.fields(cls):
            meta = f.metadata
            if "key" not in meta:
                continue
            key = meta["key"]
            if key in raw and raw[key] is not None:
                values[f.name] = _coerce(key, meta["kind"], raw[key])
            elif meta["required"]:
                raise ConfigError(f"config.json of a {cls.MODEL_TYPE!r} model must give {key!r}")
        config = cls(**values)
        config = config.resolve(raw)
        config.validate(raw)
        return config

    def resolve(self, raw: Mapping[str, Any]) -> "ModelConfig":
        """Fill fields whose default depends on other fields. Returns a (possibly new) config."""
        return self

    def validate(self, raw: Mapping[str, Any]) -> None:
        """Raise :class:`UnsupportedModelError` or :class:`ConfigError` with a reason."""

    def to_dict(self) -> dict:
        """The ``config.json`` content that reads back as this configuration."""
        out = {"model_type": self.MODEL_TYPE}
        for f in dataclasses.fields(self):
            if "key" in f.metadata:
                out[f.metadata["key"]] = getattr(self, f.name)
        return out


def read_config_json(model_dir: str) -> dict:
    path = os.path.join(model_dir, "config.json")
    if not os.path.isfile(path):
        raise FileNotFoundError(f"{model_dir!r} has no config.json")
    with open(path) as handle:
        raw = json.load(handle)
    if not isinstance(raw, dict):
        raise ConfigError(f"{path} must hold a JSON object")
    return raw
