"""Typed reading of a model folder's ``config.json``.

``KeyReader`` hands out keys with a type check and remembers which were taken, so
that an architecture can name the keys it does not understand instead of silently
ignoring a setting that changes the arithmetic.
"""
from __future__ import annotations

import json
import os
import warnings
from typing import Any, Dict, Iterable, Optional, Sequence

_MISSING = object()

# Keys that describe provenance, training or the tokenizer and never change what
# the decoder computes.  Architectures may add their own.
HARMLESS_KEYS = frozenset(
    {
        "architectures",
        "model_type",
        "torch_dtype",
        "dtype",
        "transformers_version",
        "use_cache",
        "initializer_range",
        "attention_dropout",
        "bos_token_id",
        "pad_token_id",
        "pretraining_tp",
        "_name_or_path",
        "name_or_path",
        "auto_map",
        "is_decoder",
        "output_attentions",
        "output_hidden_states",
        "return_dict",
    }
)


class ConfigError(ValueError):
    """A config.json that this framework cannot run as written."""


class KeyReader:
    def __init__(self, raw: Dict[str, Any], where: str = "config.json"):
        self.raw = dict(raw)
        self.where = where
        self.taken = set()

    def _get(self, key: str, default: Any) -> Any:
        self.taken.add(key)
        if key in self.raw and self.raw[key] is not None:
            return self.raw[key]
        if default is _MISSING:
            raise ConfigError(f"{self.where}: required key '{key}' is missing")
        return default

    def integer(self, key: str, default: Any = _MISSING, minimum: Optional[int] = None) -> Any:
        v = self._get(key, default)
        if v is None:
            return None
        if isinstance(v, bool) or not isinstance(v, int):
            if isinstance(v, float) and v.is_integer():
                v = int(v)
            else:
                raise ConfigError(f"{self.where}: '{key}' must be an integer, got {v!r}")
        if minimum is not None and v < minimum:
            raise ConfigError(f"{self.where}: '{key}' must be >= {minimum}, got {v}")
        return v

    def number(self, key: str, default: Any = _MISSING, positive: bool = False) -> Any:
        v = self._get(key, default)
        if v is None:
            return None
        if isinstance(v, bool) or not isinstance(v, (int, float)):
            raise ConfigError(f"{self.where}: '{key}' must be a number, got {v!r}")
        v = float(v)
        if positive and not v > 0.0:
            raise ConfigError(f"{self.where}: '{key}' must be > 0, got {v}")
        return v

    def boolean(self, key: str, default: Any = _MISSING) -> Any:
        v = self._get(key, default)
        if v is None:
            return None
        if not isinstance(v, bool):
            raise ConfigError(f"{self.where}: '{key}' must be true or false, got {v!r}")
        return v

    def string(self, key: str, default: Any = _MISSING) -> Any:
        v = self._get(key, default)
        if v is None:
            return None
        if not isinstance(v, str):
            raise ConfigError(f"{self.where}: '{key}' must be a string, got {v!r}")
        return v

    def mapping(self, key: str, default: Any = _MISSING) -> Any:
        v = self._get(key, default)
        if v is None:
            return None
        if not isinstance(v, dict):
            raise ConfigError(f"{self.where}: '{key}' must be an object, got {v!r}")
        return v

    def raw_value(self, key: str, default: Any = None) -> Any:
        return self._get(key, default)

    def require_value(self, key: str, allowed: Sequence[Any], default: Any) -> Any:
        """A key this framework understands only for some values."""
        v = self._get(key, default)
        if v not in allowed:
            raise ConfigError(
                f"{self.where}: '{key}'={v!r} is not supported (supported: {list(allowed)})"
            )
        return v

    def finish(self, harmless: Iterable[str] = (), strict: bool = False) -> None:
        unknown = sorted(set(self.raw) - self.taken - HARMLESS_KEYS - set(harmless))
        if unknown:
            msg = f"{self.where}: keys not understood by this architecture: {unknown}"
            if strict:
                raise ConfigError(msg)
            warnings.warn(msg, stacklevel=3)


def read_config_json(model_dir: str) -> Dict[str, Any]:
    path = os.path.join(model_dir, "config.json")
    if not os.path.isfile(path):
        raise FileNotFoundError(f"no config.json in model folder {model_dir!r}")
    with open(path, "r", encoding="utf-8") as f:
        raw = json.load(f)
    if not isinstance(raw, dict):
        raise ConfigError(f"{path}: top level must be an object")
    return raw
