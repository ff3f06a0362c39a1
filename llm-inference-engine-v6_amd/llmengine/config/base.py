"""Typed access to the keys of a model's config.json.

Every size and constant of a model comes from here; model code holds none.
Reference: the key names and defaults follow src/weights.cpp:55-121 of the
reference, which reads the same file into its ModelConfig
(include/llmengine/config.hpp:9-31).
"""
from __future__ import annotations

import json
import os
from typing import Any, Mapping


class ConfigError(ValueError):
    """A config.json is missing a key, has a wrong type, or asks for an
    option this engine does not implement."""


_MISSING = object()


class KeyReader:
    """Reads typed values out of a config mapping and names the key on error."""

    def __init__(self, data: Mapping[str, Any], where: str = "config.json"):
        if not isinstance(data, Mapping):
            raise ConfigError(f"{where}: expected a JSON object, got {type(data).__name__}")
        self.data = data
        self.where = where

    def has(self, key: str) -> bool:
        return key in self.data and self.data[key] is not None

    def _get(self, key: str, default: Any) -> Any:
        if self.has(key):
            return self.data[key]
        if default is _MISSING:
            raise ConfigError(f"{self.where}: required key '{key}' is missing")
        return default

    def integer(self, key: str, default: Any = _MISSING, minimum: int | None = None) -> int:
        v = self._get(key, default)
        if isinstance(v, bool) or not isinstance(v, int):
            if isinstance(v, float) and v == int(v):
                v = int(v)
            else:
                raise ConfigError(f"{self.where}: key '{key}' must be an integer, got {v!r}")
        if minimum is not None and v < minimum:
            raise ConfigError(f"{self.where}: key '{key}' must be >= {minimum}, got {v}")
        return int(v)

    def number(self, key: str, default: Any = _MISSING) -> float:
        v = self._get(key, default)
        if isinstance(v, bool) or not isinstance(v, (int, float)):
            raise ConfigError(f"{self.where}: key '{key}' must be a number, got {v!r}")
        return float(v)

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

    def mapping(self, key: str) -> "KeyReader | None":
        if not self.has(key):
            return None
        v = self.data[key]
        if not isinstance(v, Mapping):
            raise ConfigError(f"{self.where}: key '{key}' must be an object, got {v!r}")
        return KeyReader(v, f"{self.where}:{key}")


def read_json(path: str) -> Any:
    with open(path, "r", encoding="utf-8") as f:
        try:
            return json.load(f)
        except json.JSONDecodeError as e:
            raise ConfigError(f"{path}: not valid JSON ({e})") from None


def read_model_json(model_dir: str) -> tuple[dict, dict | None]:
    """Returns (config.json, generation_config.json or None) of a model folder."""
    cfg_path = os.path.join(model_dir, "config.json")
    if not os.path.isfile(cfg_path):
        raise ConfigError(f"no config.json in {model_dir}")
    cfg = read_json(cfg_path)
    gen_path = os.path.join(model_dir, "generation_config.json")
    gen = read_json(gen_path) if os.path.isfile(gen_path) else None
    return cfg, gen
