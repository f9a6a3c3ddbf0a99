"""The registry from an architecture's name to its model.

An entry is a pair: a reader of the architecture's `config.json` into a typed
configuration, and a builder from that configuration to a `ModelSpec`.  The
reference gates on one string (`general.architecture == "qwen3"`,
/root/reference/src/model.cpp:26-30); here that string compare is a table, and
an unknown name is an error that lists what is registered.  The host library
has the table of the built-in architecture (config/config.cpp); architectures
registered from Python are kept here and looked up first.
"""
from __future__ import annotations

import json
from typing import Any, Callable, Dict, Mapping, Tuple

from . import native
from .config.base import ConfigError
from .config.qwen3 import Qwen3Config
from .spec import ModelSpec

_ARCHITECTURES: Dict[str, Tuple[Callable[[Mapping[str, Any]], Any], Callable[[Any], Any]]] = {}


def register_architecture(names, read_config, build_spec) -> None:
    """`read_config(dict) -> config`, `build_spec(config) -> ModelSpec`.  `names`: every spelling
    that may stand in config.json's `architectures[0]` or `model_type`."""
    if isinstance(names, str):
        names = (names,)
    for n in names:
        _ARCHITECTURES[n] = (read_config, build_spec)


def registered_architectures():
    return sorted(set(_ARCHITECTURES) | set(json.loads(native.text("ti_registered_architectures"))))


def _candidates(config_dict: Mapping[str, Any]):
    out = []
    archs = config_dict.get("architectures")
    if isinstance(archs, (list, tuple)):
        out.extend(a for a in archs if isinstance(a, str))
    mt = config_dict.get("model_type")
    if isinstance(mt, str):
        out.append(mt)
    return out


def config_and_spec(config_dict: Mapping[str, Any]):
    """config.json's dict -> (typed configuration, ModelSpec)."""
    for c in _candidates(config_dict):
        if c in _ARCHITECTURES:
            read_config, build_spec = _ARCHITECTURES[c]
            cfg = read_config(config_dict)
            return cfg, build_spec(cfg)
    # the library's table (its own architecture and whatever plugins registered); its error lists the names
    text = json.dumps(dict(config_dict)).encode()
    try:
        spec = ModelSpec.from_dict(json.loads(native.text("ti_spec_from_config", text)))
        typed = json.loads(native.text("ti_typed_config", text))
    except ConfigError as e:
        if "registered:" in str(e) and _ARCHITECTURES:
            raise ConfigError(str(e).split("registered:")[0] + f"registered: {registered_architectures()}") from None
        raise
    # the architecture's own typed configuration: a class of this package where there is one, else the
    # validated keys as the library wrote them back
    reader = _TYPED_CONFIGS.get(typed["architecture"], TypedConfig)
    return reader(typed["config"]), spec


class TypedConfig(dict):
    """The typed configuration of an architecture that has no class of its own here: its validated
    config.json keys, each also an attribute."""

    def __getattr__(self, name):
        try:
            return self[name]
        except KeyError:
            raise AttributeError(name) from None

    def to_dict(self) -> dict:
        return dict(self)


_TYPED_CONFIGS = {"Qwen3ForCausalLM": Qwen3Config.from_normalized, "qwen3": Qwen3Config.from_normalized}
