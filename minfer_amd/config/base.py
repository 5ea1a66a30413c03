"""Typed configuration: helpers for reading an architecture's own config.json keys.

The reference reads typed hyper-parameters with defaults from its model file's metadata
(`HParams`, src/models/qwen2/loader.rs:11-29,97-147 of yusiwen/minfer); here the source is
config.json.  Every rejection names the key and the value it found.
"""
from __future__ import annotations

import json
import os
from typing import Any, Dict, Optional


class ConfigError(ValueError):
    """A config.json that cannot be turned into a model: the message names the key."""


_MISSING = object()


class KeyReader:
    """Reads keys of one config.json dict with type checks, and remembers which keys were
    looked at, so a model can report what it never used."""

    def __init__(self, raw: Dict[str, Any], where: str = "config.json"):
        if not isinstance(raw, dict):
            raise ConfigError(f"{where}: top level must be an object, found {type(raw).__name__}")
        self.raw = raw
        self.where = where
        self.seen = set()

    def _get(self, key: str, default: Any) -> Any:
        self.seen.add(key)
        if key not in self.raw or self.raw[key] is None:
            if default is _MISSING:
                raise ConfigError(f"{self.where}: required key '{key}' is missing")
            return default
        return self.raw[key]

    def integer(self, key: str, default: Any = _MISSING, minimum: Optional[int] = 1) -> Optional[int]:
        v = self._get(key, default)
        if v is None:
            return None
        if isinstance(v, bool) or not isinstance(v, int):
            if isinstance(v, float) and v == int(v):
                v = int(v)
            else:
                raise ConfigError(f"{self.where}: '{key}' must be an integer, found {v!r}")
        if minimum is not None and v < minimum:
            raise ConfigError(f"{self.where}: '{key}' must be >= {minimum}, found {v}")
        return v

    def number(self, key: str, default: Any = _MISSING, positive: bool = True) -> float:
        v = self._get(key, default)
        if isinstance(v, bool) or not isinstance(v, (int, float)):
            raise ConfigError(f"{self.where}: '{key}' must be a number, found {v!r}")
        v = float(v)
        if positive and not v > 0.0:
            raise ConfigError(f"{self.where}: '{key}' must be > 0, found {v}")
        return v

    def boolean(self, key: str, default: Any = _MISSING) -> bool:
        v = self._get(key, default)
        if not isinstance(v, bool):
            raise ConfigError(f"{self.where}: '{key}' must be true or false, found {v!r}")
        return v

    def string(self, key: str, default: Any = _MISSING) -> str:
        v = self._get(key, default)
        if not isinstance(v, str):
            raise ConfigError(f"{self.where}: '{key}' must be a string, found {v!r}")
        return v

    def raw_value(self, key: str, default: Any = None) -> Any:
        self.seen.add(key)
        return self.raw.get(key, default)

    def token_ids(self, key: str) -> tuple:
        """An id or a list of ids (eos_token_id may be either); absent -> empty."""
        v = self.raw_value(key)
        if v is None:
            return ()
        ids = v if isinstance(v, (list, tuple)) else [v]
        for t in ids:
            if isinstance(t, bool) or not isinstance(t, int) or t < 0:
                raise ConfigError(f"{self.where}: '{key}' must hold token ids, found {v!r}")
        return tuple(int(t) for t in ids)


def read_config_json(folder_or_file: str) -> Dict[str, Any]:
    path = folder_or_file
    if os.path.isdir(path):
        path = os.path.join(path, "config.json")
    try:
        with open(path) as f:
            raw = json.load(f)
    except FileNotFoundError:
        raise ConfigError(f"no config.json at {path}") from None
    except json.JSONDecodeError as e:
        raise ConfigError(f"{path}: not valid JSON ({e})") from None
    if not isinstance(raw, dict):
        raise ConfigError(f"{path}: top level must be an object")
    return raw


def architecture_name(raw: Dict[str, Any]) -> str:
    """The model class a config.json asks for: architectures[0]."""
    archs = raw.get("architectures")
    if isinstance(archs, str):
        return archs
    if isinstance(archs, (list, tuple)) and archs and isinstance(archs[0], str):
        return archs[0]
    raise ConfigError("config.json: 'architectures' must be a non-empty list of names, "
                      f"found {archs!r}")
