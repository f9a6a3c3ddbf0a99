"""Helpers shared by typed architecture configurations.

A configuration class reads the keys of its architecture's own `config.json`
and nothing else: every size and constant the model needs comes from there.
"""
from __future__ import annotations

import json
import os
from typing import Any, Mapping


class ConfigError(ValueError):
    """A config.json that this framework cannot serve; the text names the key."""


_MISSING = object()


def take(d: Mapping[str, Any], key: str, kind, default: Any = _MISSING) -> Any:
    """Read `key` from `d` as `kind` (int, float, bool or str).

    Without a default the key is required.  A value of the wrong JSON type is an
    error and is never coerced silently (a bool is not an int, 3.5 is not an int).
    """
    if key not in d or d[key] is None:
        if default is _MISSING:
            raise ConfigError(f"config.json: required key '{key}' is missing")
        return default
    v = d[key]
    if kind is bool:
        if not isinstance(v, bool):
            raise ConfigError(f"config.json: '{key}' must be true or false, got {v!r}")
        return v
    if kind is int:
        if isinstance(v, bool) or not isinstance(v, (int, float)) or int(v) != v:
            raise ConfigError(f"config.json: '{key}' must be an integer, got {v!r}")
        return int(v)
    if kind is float:
        if isinstance(v, bool) or not isinstance(v, (int, float)):
            raise ConfigError(f"config.json: '{key}' must be a number, got {v!r}")
        return float(v)
    if kind is str:
        if not isinstance(v, str):
            raise ConfigError(f"config.json: '{key}' must be a string, got {v!r}")
        return v
    raise TypeError(kind)


def read_config_json(model_dir: str) -> dict:
    path = os.path.join(model_dir, "config.json")
    if not os.path.isfile(path):
        raise ConfigError(f"{path}: no config.json in the model folder")
    with open(path, "r", encoding="utf-8") as f:
        try:
            d = json.load(f)
        except json.JSONDecodeError as e:
            raise ConfigError(f"{path}: not valid JSON ({e})") from None
    if not isinstance(d, dict):
        raise ConfigError(f"{path}: top level must be a JSON object")
    return d
