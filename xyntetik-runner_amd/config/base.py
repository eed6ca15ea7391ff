"""Typed reading of ``config.json``.

A value of the wrong type, sign or range is an error that names the key; it is
never passed on as garbage.  The reference reads its hyper-parameters with typed
getters that fall back to a default on a wrong type, a negative or a NaN
(src/gguf.c:494-567) and then refuses bad geometry in one place
(src/model.c:2295-2329); here both steps raise ``ConfigError``.
"""
from __future__ import annotations

import json
import math
import os
from typing import Any, Mapping, Optional, Sequence

# Upper bound of every axis, as in src/model.c:2295-2329.
MAX_AXIS = 1 << 20
_MISSING = object()


class ConfigError(ValueError):
    """A config.json that cannot describe a model this engine can build."""


def read_config_json(model_dir: str) -> dict:
    path = os.path.join(model_dir, "config.json")
    try:
        with open(path, "r", encoding="utf-8") as f:
            raw = json.load(f)
    except FileNotFoundError:
        raise ConfigError(f"{path}: no config.json in the model folder") from None
    except json.JSONDecodeError as e:
        raise ConfigError(f"{path}: not valid JSON ({e})") from None
    if not isinstance(raw, dict):
        raise ConfigError(f"{path}: top level must be a JSON object")
    return raw


def architecture_name(raw: Mapping[str, Any]) -> str:
    archs = raw.get("architectures")
    if not isinstance(archs, list) or not archs or not isinstance(archs[0], str):
        raise ConfigError("config.json: 'architectures' must be a non-empty list of names")
    return archs[0]


class Fields:
    """Typed getters over a parsed config.json."""

    def __init__(self, raw: Mapping[str, Any], where: str = "config.json"):
        self.raw = raw
        self.where = where

    def _get(self, key: str, default: Any):
        v = self.raw.get(key, _MISSING)
        if v is _MISSING or v is None:
            if default is _MISSING:
                raise ConfigError(f"{self.where}: required key '{key}' is missing")
            return _MISSING
        return v

    def integer(self, key: str, default: Any = _MISSING, lo: int = 1, hi: int = MAX_AXIS) -> int:
        v = self._get(key, default)
        if v is _MISSING:
            return default
        if isinstance(v, bool) or not isinstance(v, int):
            if isinstance(v, float) and v.is_integer():
                v = int(v)
            else:
                raise ConfigError(f"{self.where}: '{key}' must be an integer, got {v!r}")
        if not (lo <= v <= hi):
            raise ConfigError(f"{self.where}: '{key}' = {v} is outside [{lo}, {hi}]")
        return v

    def number(self, key: str, default: Any = _MISSING, lo: float = -math.inf,
               hi: float = math.inf, lo_open: bool = False) -> float:
        v = self._get(key, default)
        if v is _MISSING:
            return default
        if isinstance(v, bool) or not isinstance(v, (int, float)):
            raise ConfigError(f"{self.where}: '{key}' must be a number, got {v!r}")
        v = float(v)
        if math.isnan(v) or math.isinf(v):
            raise ConfigError(f"{self.where}: '{key}' must be finite, got {v!r}")
        if v < lo or v > hi or (lo_open and v == lo):
            raise ConfigError(f"{self.where}: '{key}' = {v} is out of range")
        return v

    def boolean(self, key: str, default: Any = _MISSING) -> bool:
        v = self._get(key, default)
        if v is _MISSING:
            return default
        if not isinstance(v, bool):
            raise ConfigError(f"{self.where}: '{key}' must be true or false, got {v!r}")
        return v

    def string(self, key: str, default: Any = _MISSING, choices: Optional[Sequence[str]] = None) -> str:
        v = self._get(key, default)
        if v is _MISSING:
            return default
        if not isinstance(v, str):
            raise ConfigError(f"{self.where}: '{key}' must be a string, got {v!r}")
        if choices is not None and v not in choices:
            raise ConfigError(f"{self.where}: '{key}' = {v!r}, expected one of {list(choices)}")
        return v

    def int_or_list(self, key: str, default: Any = _MISSING) -> tuple:
        """An id or a list of ids (``eos_token_id`` may be either)."""
        v = self._get(key, default)
        if v is _MISSING:
            return tuple(default) if default is not None else ()
        items = v if isinstance(v, list) else [v]
        out = []
        for it in items:
            if isinstance(it, bool) or not isinstance(it, int) or it < 0:
                raise ConfigError(f"{self.where}: '{key}' must hold token ids, got {v!r}")
            out.append(it)
        return tuple(out)

    def mapping(self, key: str) -> Optional["Fields"]:
        v = self.raw.get(key)
        if v is None:
            return None
        if not isinstance(v, dict):
            raise ConfigError(f"{self.where}: '{key}' must be an object, got {v!r}")
        return Fields(v, f"{self.where}:{key}")
