"""Typed reading of a model folder's ``config.json``.

Every architecture owns a dataclass whose fields are the keys of its own
``config.json``.  The helpers here read one key at a time, check its type and
range, and raise :class:`ConfigError` with the key's name in the message.  The
reference does the same with serde defaults per field
(infernum-llama/src/config.rs:19-102) and three error classes
(infernum/src/error.rs:44-57): I/O, JSON, unsupported model.
"""
from __future__ import annotations

import json
import os
from typing import Any, Mapping, Optional, Sequence


class ConfigError(ValueError):
    """A key of config.json is missing, of the wrong type or out of range."""


class UnsupportedModelError(ConfigError):
    """config.json names a ``model_type`` that no registered architecture takes."""


_MISSING = object()


class KeyReader:
    """Reads typed keys out of a parsed config.json and remembers which were read."""

    def __init__(self, raw: Mapping[str, Any], where: str = "config.json"):
        if not isinstance(raw, Mapping):
            raise ConfigError(f"{where}: top level must be a JSON object, got {type(raw).__name__}")
        self.raw = raw
        self.where = where
        self.read_keys: set[str] = set()

    def _get(self, key: str, default: Any) -> Any:
        self.read_keys.add(key)
        if key not in self.raw or self.raw[key] is None:
            if default is _MISSING:
                raise ConfigError(f"{self.where}: required key '{key}' is missing")
            return default
        return self.raw[key]

    def has(self, key: str) -> bool:
        return key in self.raw and self.raw[key] is not None

    def integer(self, key: str, default: Any = _MISSING, minimum: Optional[int] = None) -> Optional[int]:
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

    def number(self, key: str, default: Any = _MISSING, positive: bool = False) -> Optional[float]:
        v = self._get(key, default)
        if v is None:
            return None
        if isinstance(v, bool) or not isinstance(v, (int, float)):
            raise ConfigError(f"{self.where}: '{key}' must be a number, got {v!r}")
        v = float(v)
        if v != v or v in (float("inf"), float("-inf")):
            raise ConfigError(f"{self.where}: '{key}' must be finite, got {v!r}")
        if positive and v <= 0.0:
            raise ConfigError(f"{self.where}: '{key}' must be > 0, got {v}")
        return v

    def boolean(self, key: str, default: Any = _MISSING) -> Optional[bool]:
        v = self._get(key, default)
        if v is None:
            return None
        if not isinstance(v, bool):
            raise ConfigError(f"{self.where}: '{key}' must be true or false, got {v!r}")
        return v

    def string(self, key: str, default: Any = _MISSING, choices: Optional[Sequence[str]] = None) -> Optional[str]:
        v = self._get(key, default)
        if v is None:
            return None
        if not isinstance(v, str):
            raise ConfigError(f"{self.where}: '{key}' must be a string, got {v!r}")
        if choices is not None and v not in choices:
            raise ConfigError(f"{self.where}: '{key}' must be one of {list(choices)}, got {v!r}")
        return v

    def integer_or_first(self, key: str, default: Any = _MISSING) -> Optional[int]:
        """An integer, or the first element of a list of integers.

        ``eos_token_id`` may be a list in config.json; the reference takes its
        first element (infernum-llama/src/config.rs:64-68).
        """
        v = self._get(key, default)
        if v is None:
            return None
        if isinstance(v, list):
            if not v:
                raise ConfigError(f"{self.where}: '{key}' is an empty list")
            v = v[0]
        if isinstance(v, bool) or not isinstance(v, int):
            raise ConfigError(f"{self.where}: '{key}' must be an integer or a list of integers, got {v!r}")
        return v

    def obj(self, key: str) -> Optional["KeyReader"]:
        v = self._get(key, None)
        if v is None:
            return None
        if not isinstance(v, Mapping):
            raise ConfigError(f"{self.where}: '{key}' must be an object, got {v!r}")
        return KeyReader(v, f"{self.where}:{key}")


def read_config_json(model_dir_or_file: str) -> dict:
    """Parse ``config.json`` of a model folder (or the file itself)."""
    path = model_dir_or_file
    if os.path.isdir(path):
        path = os.path.join(path, "config.json")
    try:
        with open(path, "r", encoding="utf-8") as f:
            text = f.read()
    except OSError as e:
        raise ConfigError(f"cannot read {path}: {e}") from e
    try:
        raw = json.loads(text)
    except json.JSONDecodeError as e:
        raise ConfigError(f"{path}: not valid JSON: {e}") from e
    if not isinstance(raw, dict):
        raise ConfigError(f"{path}: top level must be a JSON object")
    return raw
