"""Reading typed configurations from a model folder's config.json.

A configuration class lists its keys once, with type, default and a check;
`ConfigReader` fetches them, remembers which keys were defaulted (the
reference prints its defaulted GGUF fields the same way,
ferrox-models/src/loader.rs:103-116, ferrox-cli/src/run.rs:520-528) and turns
every problem into one `ConfigError` that names the key.
"""
from __future__ import annotations

import json
import os
from typing import Any

_MISSING = object()


class ConfigError(ValueError):
    """A config.json that cannot be used: missing key, wrong type, unsupported value."""


class ConfigReader:
    def __init__(self, raw: dict, where: str = "config.json"):
        if not isinstance(raw, dict):
            raise ConfigError(f"{where}: top level must be a JSON object")
        self.raw = raw
        self.where = where
        self.defaulted: list[str] = []

    def _get(self, key: str, default: Any):
        if key in self.raw and self.raw[key] is not None:
            return self.raw[key]
        if default is _MISSING:
            raise ConfigError(f"{self.where}: required key '{key}' is missing")
        self.defaulted.append(key)
        return default

    def integer(self, key: str, default: Any = _MISSING, minimum: int | None = None) -> int:
        v = self._get(key, default)
        if isinstance(v, bool) or not isinstance(v, int):
            if isinstance(v, float) and float(v).is_integer():
                v = int(v)
            else:
                raise ConfigError(f"{self.where}: key '{key}' must be an integer, got {v!r}")
        if minimum is not None and v < minimum:
            raise ConfigError(f"{self.where}: key '{key}' must be >= {minimum}, got {v}")
        return v

    def optional_integer(self, key: str, minimum: int | None = None):
        if self.raw.get(key) is None:
            return None
        return self.integer(key, minimum=minimum)

    def number(self, key: str, default: Any = _MISSING, positive: bool = False) -> float:
        v = self._get(key, default)
        if isinstance(v, bool) or not isinstance(v, (int, float)):
            raise ConfigError(f"{self.where}: key '{key}' must be a number, got {v!r}")
        v = float(v)
        if positive and not v > 0.0:
            raise ConfigError(f"{self.where}: key '{key}' must be > 0, got {v}")
        return v

    def boolean(self, key: str, default: Any = _MISSING) -> bool:
        v = self._get(key, default)
        if not isinstance(v, bool):
            raise ConfigError(f"{self.where}: key '{key}' must be true or false, got {v!r}")
        return v

    def string(self, key: str, default: Any = _MISSING) -> str:
        v = self._get(key, default)
        if not isinstance(v, str):
            raise ConfigError(f"{self.where}: key '{key}' must be a string, got {v!r}")
        return v

    def int_list(self, key: str, default: Any = _MISSING) -> tuple:
        v = self._get(key, default)
        if not isinstance(v, (list, tuple)) or any(isinstance(i, bool) or not isinstance(i, int) for i in v):
            raise ConfigError(f"{self.where}: key '{key}' must be a list of integers, got {v!r}")
        return tuple(int(i) for i in v)


def read_config_json(folder_or_file: str) -> dict:
    path = folder_or_file
    if os.path.isdir(path):
        path = os.path.join(path, "config.json")
    if not os.path.isfile(path):
        raise ConfigError(f"no config.json at {path}")
    with open(path) as f:
        try:
            return json.load(f)
        except json.JSONDecodeError as e:
            raise ConfigError(f"{path}: not valid JSON ({e})") from e
