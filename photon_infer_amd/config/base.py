"""Helpers for typed configurations read from a model folder's config.json.

The reference has no config.json: its configuration is a 7-int header of the weight
file (include/photon/arch/config.hpp:16-24) validated in src/io/checkpoint.cpp:91-101
(every field positive, heads divisible by kv heads).  The same validations are kept;
the source of the values is the architecture's own config.json keys.
"""
from __future__ import annotations

import json
import os
from typing import Any, Mapping

from ..errors import ConfigError, ErrorCode

_MISSING = object()


class ConfigReader:
    """Typed access to a config.json mapping that names the key in every error."""

    def __init__(self, raw: Mapping[str, Any], where: str = "config.json"):
        if not isinstance(raw, Mapping):
            raise ConfigError(f"{where}: top level must be a JSON object")
        self.raw = raw
        self.where = where

    def _get(self, key: str, default: Any = _MISSING) -> Any:
        if key in self.raw and self.raw[key] is not None:
            return self.raw[key]
        if default is _MISSING:
            raise ConfigError(f"{self.where}: required key '{key}' is missing")
        return default

    def has(self, key: str) -> bool:
        return key in self.raw and self.raw[key] is not None

    def integer(self, key: str, default: Any = _MISSING, *, minimum: int | None = 1) -> int:
        v = self._get(key, default)
        if isinstance(v, bool) or not isinstance(v, int):
            if isinstance(v, float) and v.is_integer():
                v = int(v)
            else:
                raise ConfigError(f"{self.where}: '{key}' must be an integer, got {v!r}")
        if minimum is not None and v < minimum:
            raise ConfigError(f"{self.where}: '{key}' must be >= {minimum}, got {v}")
        return v

    def number(self, key: str, default: Any = _MISSING, *, positive: bool = True) -> float:
        v = self._get(key, default)
        if isinstance(v, bool) or not isinstance(v, (int, float)):
            raise ConfigError(f"{self.where}: '{key}' must be a number, got {v!r}")
        v = float(v)
        if positive and not v > 0.0:
            raise ConfigError(f"{self.where}: '{key}' must be > 0, got {v}")
        return v

    def boolean(self, key: str, default: Any = _MISSING) -> bool:
        v = self._get(key, default)
        if not isinstance(v, bool):
            raise ConfigError(f"{self.where}: '{key}' must be true or false, got {v!r}")
        return v

    def string(self, key: str, default: Any = _MISSING) -> str:
        v = self._get(key, default)
        if not isinstance(v, str):
            raise ConfigError(f"{self.where}: '{key}' must be a string, got {v!r}")
        return v

    def mapping(self, key: str) -> "ConfigReader | None":
        if not self.has(key):
            return None
        v = self.raw[key]
        if not isinstance(v, Mapping):
            raise ConfigError(f"{self.where}: '{key}' must be an object or null, got {v!r}")
        return ConfigReader(v, f"{self.where}:{key}")

    def int_or_list(self, key: str) -> tuple[int, ...]:
        if not self.has(key):
            return ()
        v = self.raw[key]
        items = v if isinstance(v, (list, tuple)) else [v]
        out = []
        for it in items:
            if isinstance(it, bool) or not isinstance(it, int):
                raise ConfigError(f"{self.where}: '{key}' must be an int or a list of ints, got {v!r}")
            out.append(int(it))
        return tuple(out)


def read_config_json(model_dir: str) -> dict:
    """Read ``<model_dir>/config.json``; FileNotFound / ModelParseError as in
    src/io/checkpoint.cpp:29-34 for a missing or malformed file."""
    path = os.path.join(model_dir, "config.json")
    if not os.path.isfile(path):
        raise ConfigError(f"no config.json in model folder '{model_dir}'", ErrorCode.FILE_NOT_FOUND)
    try:
        with open(path, "r", encoding="utf-8") as f:
            raw = json.load(f)
    except (OSError, ValueError) as e:
        raise ConfigError(f"{path}: cannot be read as JSON: {e}") from e
    if not isinstance(raw, dict):
        raise ConfigError(f"{path}: top level must be a JSON object")
    return raw


def architecture_name(raw: Mapping[str, Any], where: str = "config.json") -> str:
    archs = raw.get("architectures")
    if not isinstance(archs, (list, tuple)) or not archs or not isinstance(archs[0], str):
        raise ConfigError(f"{where}: 'architectures' must be a non-empty list of names")
    return archs[0]
