"""Typed model configurations and the architecture registry.

A configuration is a frozen dataclass whose fields are the keys of the
architecture's own ``config.json``.  Nothing else in the package holds a model
size: parts receive their sizes from a configuration when a model is built.

The registry maps an architecture name (``config.json``'s ``architectures[0]``)
to a configuration class and a model builder.  The reference has a single
model type and never looks at ``architectures``
(crates/glassbox-core/src/model.rs:7-47); the registry is what lets a second
architecture be added here without touching the engine.
"""
from __future__ import annotations

import json
import os
from dataclasses import dataclass, fields, MISSING
from typing import Any, Callable, Dict, Tuple, Type


class ConfigError(ValueError):
    """config.json is missing a key, has a wrong type, or asks for something unsupported."""


@dataclass(frozen=True)
class ModelConfig:
    """Base of every architecture's configuration."""

    #: architecture name under which the subclass is registered
    architecture = ""

    @classmethod
    def from_dict(cls, raw: Dict[str, Any]) -> "ModelConfig":
        raise NotImplementedError

    def to_dict(self) -> Dict[str, Any]:
        out = {"architectures": [self.architecture]}
        for f in fields(self):
            v = getattr(self, f.name)
            if v is not None:
                out[f.name] = v
        return out

    def save(self, folder: str) -> None:
        with open(os.path.join(folder, "config.json"), "w") as fh:
            json.dump(self.to_dict(), fh, indent=2)
            fh.write("\n")


def read_typed(cls: Type[ModelConfig], raw: Dict[str, Any]) -> Dict[str, Any]:
    """Pick the dataclass fields of ``cls`` out of ``raw`` with type checks.

    Required fields (no default) that are absent raise one ConfigError naming
    all of them; unknown keys are ignored, as serde does for the reference.
    """
    out: Dict[str, Any] = {}
    missing = []
    for f in fields(cls):
        if f.name in raw and raw[f.name] is not None:
            v = raw[f.name]
            want = f.type if isinstance(f.type, str) else getattr(f.type, "__name__", str(f.type))
            want = want.replace("Optional[", "").rstrip("]")
            if want == "int":
                if isinstance(v, bool) or not isinstance(v, int):
                    if isinstance(v, float) and v == int(v):
                        v = int(v)
                    else:
                        raise ConfigError(f"config key {f.name!r} must be an integer, got {v!r}")
            elif want == "float":
                if isinstance(v, bool) or not isinstance(v, (int, float)):
                    raise ConfigError(f"config key {f.name!r} must be a number, got {v!r}")
                v = float(v)
            elif want == "bool":
                if not isinstance(v, bool):
                    raise ConfigError(f"config key {f.name!r} must be true or false, got {v!r}")
            out[f.name] = v
        elif f.default is MISSING and f.default_factory is MISSING:  # type: ignore[misc]
            missing.append(f.name)
    if missing:
        raise ConfigError(f"config.json of {cls.architecture} lacks required keys: {', '.join(missing)}")
    return out


Builder = Callable[..., Any]
_REGISTRY: Dict[str, Tuple[Type[ModelConfig], Builder]] = {}
_MODEL_TYPES: Dict[str, str] = {}


def register_architecture(name: str, config_cls: Type[ModelConfig], builder: Builder,
                          model_type: str | None = None) -> None:
    """Register ``name`` -> (configuration class, builder(config) -> model).

    ``model_type`` is the optional ``config.json`` ``model_type`` value that
    stands in when ``architectures`` is absent.
    """
    _REGISTRY[name] = (config_cls, builder)
    if model_type:
        _MODEL_TYPES[model_type] = name


def _register_builtin() -> None:
    from .. import models  # noqa: F401  (importing the package registers its architectures)


def known_architectures() -> list:
    _register_builtin()
    return sorted(_REGISTRY)


def lookup(name: str) -> Tuple[Type[ModelConfig], Builder]:
    _register_builtin()
    if name not in _REGISTRY:
        raise ConfigError(
            f"unknown architecture {name!r}; registered: {', '.join(known_architectures()) or '(none)'}")
    return _REGISTRY[name]


def architecture_of(raw: Dict[str, Any]) -> str:
    archs = raw.get("architectures")
    if isinstance(archs, list) and archs:
        return str(archs[0])
    mt = raw.get("model_type")
    _register_builtin()
    if mt in _MODEL_TYPES:
        return _MODEL_TYPES[mt]
    raise ConfigError(
        "config.json names no architecture (key 'architectures'); registered: "
        + ", ".join(known_architectures()))


def config_from_dict(raw: Dict[str, Any]) -> ModelConfig:
    cls, _ = lookup(architecture_of(raw))
    return cls.from_dict(raw)


def config_from_dir(folder: str) -> ModelConfig:
    path = os.path.join(folder, "config.json")
    try:
        with open(path) as fh:
            raw = json.load(fh)
    except FileNotFoundError:
        raise ConfigError(f"{path}: no such file") from None
    except json.JSONDecodeError as e:
        raise ConfigError(f"{path}: not valid JSON ({e})") from None
    if not isinstance(raw, dict):
        raise ConfigError(f"{path}: top level must be an object")
    return config_from_dict(raw)
