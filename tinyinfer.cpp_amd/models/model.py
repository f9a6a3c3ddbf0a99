"""A model put together from a `ModelSpec` by the host library (models/model.cpp):
its parts are built through the one table of parts, their cache needs gathered
into groups, the run order kept as a list.  This class names the result."""
from __future__ import annotations

import ctypes
import json
from typing import Dict, List, Tuple

from .. import native
from ..parts.base import part_handle
from ..parts.builtin import adopt
from ..spec import ModelSpec, TensorNeed, cache_need_from_dict


class Model:
    def __init__(self, spec: ModelSpec):
        self.spec = spec
        self.vocab_size = spec.vocab_size
        self.hidden_size = spec.hidden_size
        self.run_order = spec.run_order()
        # the library builds every part through its table of parts (kinds registered from Python are made
        # by their Python classes on the way); what stands here afterwards are views of its parts
        try:
            self._ptr = native.pointer("ti_model_from_spec", json.dumps(spec.to_dict()).encode())
        except native.ConfigError as e:
            raise ValueError(str(e)) from None
        part = lambda which, i=0: adopt(native.pointer("ti_model_part", self._ptr, which, i))      # noqa: E731
        self.embedding = part(b"embedding")
        self.blocks = [part(b"block", i) for i in range(len(spec.layers))]
        self.final_norm = part(b"final_norm")
        self.head = part(b"head")
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
