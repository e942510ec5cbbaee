"""Reading typed values out of a config.json, with errors that name the key."""
from __future__ import annotations

import json
import os
from typing import Any, Dict, Optional


class ConfigError(ValueError):
    """A config.json that cannot be used; the message names the key."""


_MISSING = object()


def read_config_json(folder: str) -> Dict[str, Any]:
    path = os.path.join(folder, "config.json")
    if not os.path.isfile(path):
        raise ConfigError(f"no config.json in model folder {folder!r}")
    with open(path) as f:
        try:
            data = json.load(f)
        except json.JSONDecodeError as e:
            raise ConfigError(f"{path}: not valid JSON: {e}") from None
    if not isinstance(data, dict):
        raise ConfigError(f"{path}: the top level must be an object")
    return data


class KeyReader:
    """Typed access to the keys of one config.json; every failure names the key."""

    def __init__(self, data: Dict[str, Any], where: str = "config.json"):
        self.data = data
        self.where = where

    def _get(self, key: str, default: Any):
        v = self.data.get(key, _MISSING)
        if v is _MISSING or v is None:
            if default is _MISSING:
                raise ConfigError(f"{self.where}: required key {key!r} is missing")
            return _MISSING
        return v

    def integer(self, key: str, default: Any = _MISSING, minimum: Optional[int] = 1) -> int:
        v = self._get(key, default)
        if v is _MISSING:
            return default
        if isinstance(v, bool) or not isinstance(v, int):
            raise ConfigError(f"{self.where}: key {key!r} must be an integer, got {v!r}")
        if minimum is not None and v < minimum:
            raise ConfigError(f"{self.where}: key {key!r} must be >= {minimum}, got {v}")
        return v

    def number(self, key: str, default: Any = _MISSING, positive: bool = True) -> float:
        v = self._get(key, default)
        if v is _MISSING:
            return default
        if isinstance(v, bool) or not isinstance(v, (int, float)):
            raise ConfigError(f"{self.where}: key {key!r} must be a number, got {v!r}")
        if positive and not v > 0:
            raise ConfigError(f"{self.where}: key {key!r} must be > 0, got {v}")
        return float(v)

    def boolean(self, key: str, default: Any = _MISSING) -> bool:
        v = self._get(key, default)
        if v is _MISSING:
            return default
        if not isinstance(v, bool):
            raise ConfigError(f"{self.where}: key {key!r} must be true or false, got {v!r}")
        return v

    def token_ids(self, key: str):
        """An optional token id, or a list of them (``eos_token_id`` may be either)."""
        v = self.data.get(key)
        if v is None:
            return ()
        items = v if isinstance(v, list) else [v]
        for i in items:
            if isinstance(i, bool) or not isinstance(i, int) or i < 0:
                raise ConfigError(f"{self.where}: key {key!r} must hold token ids, got {v!r}")
        return tuple(items)

    def absent_or(self, key: str, allowed, why: str):
        """Reject a key whose value would change the computation in a way this engine
        does not implement."""
        v = self.data.get(key)
        if v is None:
            return
        if v not in allowed:
            raise ConfigError(f"{self.where}: key {key!r} = {v!r} is not supported ({why})")
