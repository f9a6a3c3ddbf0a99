"""A model put together from a `ModelSpec`: parts built through the part
registry, handed to the host library, which gathers their cache needs into
groups and keeps the run order (models/model.cpp)."""
from __future__ import annotations

import ctypes
import json
from typing import Dict, List, Tuple

from .. import native
from ..parts.base import join, part_handle
from ..parts.registry import _PARTS, build_part
from ..spec import ModelSpec, TensorNeed, cache_need_from_dict


class Model:
    def __init__(self, spec: ModelSpec):
        self.spec = spec
        self.vocab_size = spec.vocab_size
        self.hidden_size = spec.hidden_size
        self.embedding = build_part("embedding", spec.embedding, spec.embedding.name)
        self.blocks = []
        for ls in spec.layers:
            key = ("block", ls.block.kind)
            if key not in _PARTS:
                raise KeyError(f"no block arrangement of kind {ls.block.kind!r}")
            slots = getattr(_PARTS[key], "slots", None)
            if slots is None:
                raise TypeError(f"block arrangement {ls.block.kind!r} declares no `slots`")
            built = {}
            for slot, family in slots.items():
                if slot not in ls.parts:
                    raise KeyError(f"layer '{ls.prefix}': block '{ls.block.kind}' needs a '{slot}' part")
                ps = ls.parts[slot]
                built[slot] = build_part(family, ps, join(ls.prefix, ps.name))
            self.blocks.append(_PARTS[key](prefix=ls.prefix, **built, **ls.block.params))
        self.final_norm = build_part("norm", spec.final_norm, spec.final_norm.name)
        self.head = build_part("head", spec.lm_head, spec.lm_head.name)
        self.run_order = spec.run_order()
        for i in self.run_order:
            if not 0 <= i < len(self.blocks):
                raise ValueError(f"schedule names layer {i}, but there are {len(self.blocks)}")
        meta = {"architecture": spec.architecture, "vocab_size": spec.vocab_size, "hidden_size": spec.hidden_size,
                "schedule": spec.schedule, "eos_token_ids": list(spec.eos_token_ids),
                "max_position_embeddings": spec.max_position_embeddings,
                "cache_from": [ls.cache_from for ls in spec.layers]}
        handles = (ctypes.c_void_p * max(1, len(self.blocks)))(*[part_handle(b).ptr for b in self.blocks])
        try:
            self._ptr = native.pointer("ti_model_create", json.dumps(meta).encode(), part_handle(self.embedding).ptr,
                                       len(self.blocks), handles, part_handle(self.final_norm).ptr,
                                       part_handle(self.head).ptr)
        except native.ConfigError as e:
            raise ValueError(str(e)) from None
        # groups of cache layers with the same need, and per run: id(part) -> (group, cache layer)
        groups = json.loads(native.text("ti_model_cache_groups", self._ptr))
        self.cache_groups: List[Tuple[object, int]] = [(cache_need_from_dict(g["need"]), g["layers"]) for g in groups]
        by_identity = {part_handle(p).identity(): p for p in self.parts()}
        self.bindings: List[Dict[int, Tuple[int, int]]] = [
            {id(by_identity[ident]): (g, l) for ident, g, l in run}
            for run in json.loads(native.text("ti_model_bindings", self._ptr))]
        self.dtype = None

    def __del__(self):
        try:
            if native._lib is not None and getattr(self, "_ptr", None):
                native._lib.ti_model_release(self._ptr)
        except Exception:  # noqa: BLE001
            pass

    def parts(self):
        yield from self.embedding.walk()
        for b in self.blocks:
            yield from b.walk()
        yield from self.final_norm.walk()
        yield from self.head.walk()

    def tensors(self) -> Dict[str, TensorNeed]:
        """Every checkpoint tensor the model asks for, in a fixed order."""
        return {n: TensorNeed.from_dict(v) for n, v in json.loads(native.text("ti_model_tensors", self._ptr)).items()}
