"""What every typed configuration shares: the error, and reading a folder's
config.json.  A configuration reads the keys of its architecture's own
`config.json` and nothing else: every size and constant the model needs comes
from there.
"""
from __future__ import annotations

import json
import os

from ..native import ConfigError  # noqa: F401


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
