"""Registry of parts by family and kind.

Families: "embedding", "norm", "pos", "mixer", "ffn", "block", "head".
There is one table, the host library's (parts/parts.cpp `register_part`).  A kind
registered from Python is entered there too, with a factory that calls back into
the Python class, so a `ModelSpec` that names it is built by the library like any
other; a kind the library itself (or a plugin loaded into it) registered needs
nothing here: `build_part` asks the library for it and hands back a view
(parts/builtin.py).
"""
from __future__ import annotations

import json
from typing import Callable, Dict, Tuple

from .. import native

FAMILIES = ("embedding", "norm", "pos", "mixer", "ffn", "block", "head")
_PARTS: Dict[Tuple[str, str], Callable] = {}


def register_part(family: str, kind: str, factory: Callable) -> None:
    """`factory(prefix=..., **params, **children)` makes the part (a subclass of `parts.Part`).  A block
    arrangement says which family each of its slots is built from in the factory's `slots` dict."""
    if family not in FAMILIES:
        raise ValueError(f"unknown part family {family!r}; families: {FAMILIES}")
    _PARTS[(family, kind)] = factory
    slots = getattr(factory, "slots", None) or {}
    native.call("ti_register_foreign_kind", family.encode(), kind.encode(), json.dumps(dict(slots)).encode())


def make_registered(family: str, kind: str, prefix: str, params: dict, children):
    """What the library calls when a spec comes to a kind registered from Python.  `children`: [(slot, handle)]
    of parts the library has built already (a block arrangement's)."""
    from ..spec import PartSpec
    from .builtin import adopt
    kids = {slot: adopt(ptr) for slot, ptr in children}          # (the handles are ours from here on)
    factory = _PARTS[(family, kind)]
    params = {k: (PartSpec.from_dict(v) if isinstance(v, dict) and "kind" in v and "params" in v else v)
              for k, v in params.items()}
    return factory(prefix=prefix, **params, **kids)


def build_part(family: str, spec, prefix: str):
    """Instantiate `spec` (a PartSpec) of `family`; `prefix` starts its tensor names.  A kind registered from
    Python gives that class's object, any other kind a view of the library's part."""
    from .builtin import adopt
    if family not in FAMILIES:
        raise ValueError(f"unknown part family {family!r}; families: {FAMILIES}")
    key = (family, spec.kind)
    if key in _PARTS and not getattr(_PARTS[key], "slots", None):
        return make_registered(family, spec.kind, prefix, dict(spec.params), ())
    params = spec.to_dict()["params"]
    return adopt(native.pointer("ti_part_create", family.encode(), spec.kind.encode(), prefix.encode(),
                                json.dumps(params).encode(), 0, None, None))


def registered_parts(family: str):
    """Every kind of `family` that a spec may name: the library's own, a plugin's, and those registered from Python."""
    return sorted(json.loads(native.text("ti_registered_parts", family.encode())))
