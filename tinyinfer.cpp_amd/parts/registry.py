"""Registry of parts by family and kind.

Families: "embedding", "norm", "pos", "mixer", "ffn", "block", "head".
A `PartSpec(kind, params)` is built by looking its kind up in its family: among
the kinds registered from Python first, then among the host library's own.
"""
from __future__ import annotations

from typing import Callable, Dict, Tuple

FAMILIES = ("embedding", "norm", "pos", "mixer", "ffn", "block", "head")
_PARTS: Dict[Tuple[str, str], Callable] = {}


def register_part(family: str, kind: str, factory: Callable) -> None:
    if family not in FAMILIES:
        raise ValueError(f"unknown part family {family!r}; families: {FAMILIES}")
    _PARTS[(family, kind)] = factory


def build_part(family: str, spec, prefix: str):
    """Instantiate `spec` (a PartSpec) of `family`; `prefix` starts its tensor names."""
    key = (family, spec.kind)
    if key not in _PARTS:
        have = sorted(k for f, k in _PARTS if f == family)
        raise KeyError(f"no {family} part of kind {spec.kind!r}; registered: {have}")
    return _PARTS[key](prefix=prefix, **spec.params)


def registered_parts(family: str):
    return sorted(k for f, k in _PARTS if f == family)
