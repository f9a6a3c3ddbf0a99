"""A model put together from a `ModelSpec`: parts built through the part
registry, cache needs gathered into groups, the run order kept as a list."""
from __future__ import annotations

from typing import Dict, List, Tuple

from ..spec import ModelSpec, TensorNeed
from ..parts.registry import build_part, _PARTS
from ..parts.base import join


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
        self._group_cache()

    # ------------------------------------------------------------------ parts
    def parts(self):
        yield from self.embedding.walk()
        for b in self.blocks:
            yield from b.walk()
        yield from self.final_norm.walk()
        yield from self.head.walk()

    def tensors(self) -> Dict[str, TensorNeed]:
        """Every checkpoint tensor the model asks for, in a fixed order.  A name
        asked for twice (a tied head) must be asked for with one shape; it is
        optional only if every asker says so."""
        out: Dict[str, TensorNeed] = {}
        for p in self.parts():
            for name, need in p.tensors().items():
                if name in out:
                    old = out[name]
                    if old.shape != need.shape or old.role != need.role:
                        raise ValueError(f"tensor '{name}' is asked for as {old.shape}/{old.role} "
                                         f"and as {need.shape}/{need.role}")
                    if old.optional and not need.optional:
                        out[name] = need
                else:
                    out[name] = need
        return out

    # ------------------------------------------------------------------ cache
    def _group_cache(self):
        """Give every run of a layer that keeps a cache a cache layer of its own,
        and gather cache layers with the same need into groups (one page id
        addresses a token's slot in every cache layer of its group).

        A layer named twice in the run order computes different keys and values
        each time, so each run has its own cache layer.  A layer with
        `cache_from = j` keeps none: it reads what the latest earlier run of
        layer j wrote (the first run of j if none came earlier).

        `self.bindings[r][id(part)] = (group, cache_layer)` for run r.
        """
        index: Dict[object, int] = {}
        counts: List[int] = []
        layers = self.spec.layers
        self.bindings: List[Dict[int, Tuple[int, int]]] = [dict() for _ in self.run_order]
        runs_of: Dict[int, List[int]] = {}
        for r, i in enumerate(self.run_order):
            runs_of.setdefault(i, []).append(r)
            if layers[i].cache_from is not None:
                continue
            for part in self.blocks[i].walk():
                need = part.cache_need()
                if need is None:
                    continue
                if need not in index:
                    index[need] = len(counts)
                    counts.append(0)
                g = index[need]
                self.bindings[r][id(part)] = (g, counts[g])
                counts[g] += 1
        for r, i in enumerate(self.run_order):
            j = layers[i].cache_from
            if j is None:
                continue
            if j not in runs_of or layers[j].cache_from is not None:
                raise ValueError(f"layer {i} reads the cache of layer {j}, which keeps none")
            earlier = [q for q in runs_of[j] if q < r]
            src = earlier[-1] if earlier else runs_of[j][0]
            theirs = [b for b in self.bindings[src].values()]
            mine = [p for p in self.blocks[i].walk() if p.cache_need() is not None]
            if len(theirs) != len(mine):
                raise ValueError(f"layer {i} cannot read the cache of layer {j}: "
                                 "they keep different numbers of caches")
            for part, b in zip(mine, theirs):
                self.bindings[r][id(part)] = b
        needs = sorted(index, key=lambda n: index[n])
        self.cache_groups: List[Tuple[object, int]] = [(n, counts[index[n]]) for n in needs]
