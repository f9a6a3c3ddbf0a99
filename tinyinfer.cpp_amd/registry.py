"""The registry from an architecture's name to its model.

An entry is a pair: the typed configuration class that reads the architecture's
`config.json`, and a builder from that configuration to a `ModelSpec`.  The
reference gates on one string (`general.architecture == "qwen3"`,
/root/reference/src/model.cpp:26-30); here that string compare is a table, and
an unknown name is an error that lists what is registered.
"""
from __future__ import annotations

from typing import Any, Callable, Dict, Mapping, Tuple

from .config.base import ConfigError

_ARCHITECTURES: Dict[str, Tuple[Callable[[Mapping[str, Any]], Any], Callable[[Any], Any]]] = {}


def register_architecture(names, read_config, build_spec) -> None:
    """`read_config(dict) -> config`, `build_spec(config) -> ModelSpec`.

    `names`: every spelling that may stand in config.json's `architectures[0]`
    or `model_type`.
    """
    if isinstance(names, str):
        names = (names,)
    for n in names:
        _ARCHITECTURES[n] = (read_config, build_spec)


def registered_architectures():
    return sorted(_ARCHITECTURES)


def resolve_architecture(config_dict: Mapping[str, Any]):
    """Pick the entry by `architectures[0]`, else by `model_type`."""
    candidates = []
    archs = config_dict.get("architectures")
    if isinstance(archs, (list, tuple)):
        candidates.extend(a for a in archs if isinstance(a, str))
    mt = config_dict.get("model_type")
    if isinstance(mt, str):
        candidates.append(mt)
    if not candidates:
        raise ConfigError("config.json: neither 'architectures' nor 'model_type' names the model; "
                          f"registered: {registered_architectures()}")
    for c in candidates:
        if c in _ARCHITECTURES:
            return c, _ARCHITECTURES[c]
    raise ConfigError(f"config.json: architecture {candidates!r} is not registered; "
                      f"registered: {registered_architectures()}")


def config_and_spec(config_dict: Mapping[str, Any]):
    """config.json's dict -> (typed configuration, ModelSpec)."""
    _, (read_config, build_spec) = resolve_architecture(config_dict)
    cfg = read_config(config_dict)
    return cfg, build_spec(cfg)
