"""Typed reading of a model folder's config.json.

The reference reads its model description through typed getters with defaults
(/root/reference/internal/gguf/gguf.go:117-181) and rejects an incomplete one
with a single error (/root/reference/internal/llm/model.go:95-97).  `KeyReader`
is the same idea over a JSON object: every access names a key, a type and an
optional default; all problems are collected and raised together.
"""
from __future__ import annotations

import json
import os
from typing import Any

_REQUIRED = object()


class ConfigError(ValueError):
    """config.json is missing keys, has keys of the wrong type or fails validation."""


class KeyReader:
    def __init__(self, data: dict, where: str = "config.json"):
        if not isinstance(data, dict):
            raise ConfigError(f"{where}: expected a JSON object, got {type(data).__name__}")
        self.data = data
        self.where = where
        self.problems: list[str] = []

    def _get(self, key: str, default: Any):
        if key not in self.data or self.data[key] is None:
            if default is _REQUIRED:
                self.problems.append(f"missing key {key!r}")
                return None
            return default
        return self.data[key]

    def int(self, key: str, default: Any = _REQUIRED):
        v = self._get(key, default)
        if v is None:
            return v
        if isinstance(v, bool) or not isinstance(v, int):
            if isinstance(v, float) and v.is_integer():
                return int(v)
            self.problems.append(f"key {key!r}: expected an integer, got {v!r}")
            return None
        return v

    def float(self, key: str, default: Any = _REQUIRED):
        v = self._get(key, default)
        if v is None:
            return v
        if isinstance(v, bool) or not isinstance(v, (int, float)):
            self.problems.append(f"key {key!r}: expected a number, got {v!r}")
            return None
        return float(v)

    def bool(self, key: str, default: Any = _REQUIRED):
        v = self._get(key, default)
        if v is None:
            return v
        if not isinstance(v, bool):
            self.problems.append(f"key {key!r}: expected true or false, got {v!r}")
            return None
        return v

    def str(self, key: str, default: Any = _REQUIRED):
        v = self._get(key, default)
        if v is None:
            return v
        if not isinstance(v, str):
            self.problems.append(f"key {key!r}: expected a string, got {v!r}")
            return None
        return v

    def object(self, key: str, default: Any = _REQUIRED):
        v = self._get(key, default)
        if v is None:
            return v
        if not isinstance(v, dict):
            self.problems.append(f"key {key!r}: expected an object, got {v!r}")
            return None
        return v

    def int_or_list(self, key: str, default: Any = _REQUIRED):
        """An id or a list of ids (eos_token_id is either)."""
        v = self._get(key, default)
        if v is None:
            return ()
        if isinstance(v, int) and not isinstance(v, bool):
            return (v,)
        if isinstance(v, list) and all(isinstance(i, int) and not isinstance(i, bool) for i in v):
            return tuple(v)
        self.problems.append(f"key {key!r}: expected an integer or a list of integers, got {v!r}")
        return ()

    def require(self, ok: bool, message: str):
        if not ok:
            self.problems.append(message)

    def finish(self):
        if self.problems:
            raise ConfigError(f"{self.where}: " + "; ".join(self.problems))


def read_config_json(model_dir: str) -> dict:
    path = os.path.join(model_dir, "config.json")
    if not os.path.isfile(path):
        raise ConfigError(f"{model_dir}: no config.json in the model folder")
    with open(path, "r", encoding="utf-8") as f:
        try:
            data = json.load(f)
        except json.JSONDecodeError as e:
            raise ConfigError(f"{path}: not valid JSON ({e})") from None
    if not isinstance(data, dict):
        raise ConfigError(f"{path}: expected a JSON object")
    return data
