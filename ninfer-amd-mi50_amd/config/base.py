"""Typed reading of config.json keys.

The reference reads config.json with `j.at(key)` (throws when absent) and
`j.find(key)` with a default (src/models/config.cpp:17-32). `KeyReader` keeps
that split (`need` / `opt`), adds type checks, and names the key in every
error.
"""
from __future__ import annotations

import json
import os
from typing import Any, Dict, Iterable, List, Optional


class ConfigError(ValueError):
    """A config.json key is missing, of the wrong type or out of range."""


_MISSING = object()


class KeyReader:
    """Typed access to a config dictionary; remembers which keys were read."""

    def __init__(self, raw: Dict[str, Any], where: str = "config.json"):
        if not isinstance(raw, dict):
            raise ConfigError(f"{where}: top level must be an object")
        self.raw = raw
        self.where = where
        self.used: set = set()

    def _get(self, key: str, default: Any) -> Any:
        self.used.add(key)
        if key not in self.raw or self.raw[key] is None:
            if default is _MISSING:
                raise ConfigError(f"{self.where}: required key '{key}' is missing")
            return default
        return self.raw[key]

    def need_int(self, key: str, minimum: Optional[int] = None) -> int:
        return self._int(key, self._get(key, _MISSING), minimum)

    def opt_int(self, key: str, default: Optional[int], minimum: Optional[int] = None
                ) -> Optional[int]:
        v = self._get(key, default)
        return v if v is None else self._int(key, v, minimum)

    def _int(self, key: str, v: Any, minimum: Optional[int]) -> int:
        if isinstance(v, bool) or not isinstance(v, (int, float)) or int(v) != v:
            raise ConfigError(f"{self.where}: key '{key}' must be an integer, got {v!r}")
        v = int(v)
        if minimum is not None and v < minimum:
            raise ConfigError(f"{self.where}: key '{key}' must be >= {minimum}, got {v}")
        return v

    def need_float(self, key: str) -> float:
        return self._float(key, self._get(key, _MISSING))

    def opt_float(self, key: str, default: float) -> float:
        return self._float(key, self._get(key, default))

    def _float(self, key: str, v: Any) -> float:
        if isinstance(v, bool) or not isinstance(v, (int, float)):
            raise ConfigError(f"{self.where}: key '{key}' must be a number, got {v!r}")
        return float(v)

    def opt_bool(self, key: str, default: bool) -> bool:
        v = self._get(key, default)
        if not isinstance(v, bool):
            raise ConfigError(f"{self.where}: key '{key}' must be true or false, got {v!r}")
        return v

    def opt_str(self, key: str, default: Optional[str]) -> Optional[str]:
        v = self._get(key, default)
        if v is not None and not isinstance(v, str):
            raise ConfigError(f"{self.where}: key '{key}' must be a string, got {v!r}")
        return v

    def opt_int_list(self, key: str, default: Iterable[int]) -> List[int]:
        v = self._get(key, list(default))
        if not isinstance(v, list):
            raise ConfigError(f"{self.where}: key '{key}' must be a list of integers")
        return [self._int(f"{key}[{i}]", x, 0) for i, x in enumerate(v)]

    def opt_raw(self, key: str, default: Any = None) -> Any:
        return self._get(key, default)


def read_config_json(model_dir: str) -> Dict[str, Any]:
    path = os.path.join(model_dir, "config.json")
    if not os.path.isfile(path):
        raise ConfigError(f"{path}: no such file")
    with open(path, "r", encoding="utf-8") as f:
        try:
            return json.load(f)
        except json.JSONDecodeError as e:
            raise ConfigError(f"{path}: not valid JSON ({e})") from None


def architecture_name(raw: Dict[str, Any]) -> str:
    """`architectures[0]`, the key of the model registry
    (reference src/models/config.cpp:12-14 stores it; it has no registry)."""
    arch = raw.get("architectures")
    if not isinstance(arch, list) or not arch or not isinstance(arch[0], str):
        raise ConfigError("config.json: key 'architectures' must be a non-empty list of names")
    return arch[0]
