"""One registry from an architecture's name (``config.json: architectures[0]``) to
what builds it: a typed configuration class and a function from that
configuration to a ``ModelSpec``.

The reference picks model pieces by name in several places
(yalis/external/model.py:372-373 for the MLP class, yalis/external/config.py:238-257
for the norm, yalis/attention/registry.py:3-17 for the attention backend); here one
table keyed by the architecture name does it.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Callable, Dict, Type

from .reader import ConfigError, read_config_json
from .specs import ModelSpec


@dataclass(frozen=True)
class Architecture:
    name: str
    config_class: Type[Any]  # has from_dict(raw) and to_dict()
    build_spec: Callable[[Any], ModelSpec]


_ARCHITECTURES: Dict[str, Architecture] = {}


def register_architecture(name: str, config_class: Type[Any], build_spec: Callable[[Any], ModelSpec]) -> None:
    _ARCHITECTURES[name] = Architecture(name, config_class, build_spec)


def known_architectures():
    _ensure_builtin()
    return sorted(_ARCHITECTURES)


def _ensure_builtin() -> None:
    # Importing the models package registers the architectures it ships.
    from .. import models  # noqa: F401


def get_architecture(name: str) -> Architecture:
    _ensure_builtin()
    if name not in _ARCHITECTURES:
        raise ConfigError(
            f"unknown architecture {name!r}; known architectures: {sorted(_ARCHITECTURES)}"
        )
    return _ARCHITECTURES[name]


def architecture_of(raw: Dict[str, Any]) -> Architecture:
    archs = raw.get("architectures")
    if not isinstance(archs, list) or len(archs) < 1 or not isinstance(archs[0], str):
        raise ConfigError("config.json: 'architectures' must be a list holding the model class name")
    return get_architecture(archs[0])


def load_model_config(model_dir: str):
    """Read ``model_dir/config.json``; returns (architecture, typed config)."""
    raw = read_config_json(model_dir)
    arch = architecture_of(raw)
    return arch, arch.config_class.from_dict(raw)
