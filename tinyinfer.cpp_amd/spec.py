"""A model as data: which parts each layer is made of and in which order layers run.

Nothing here computes.  An architecture's builder turns its typed configuration
into a `ModelSpec`; the weight loader, the cache manager and the engine read
only the spec, so an architecture with other parts in some layers, a layer that
runs twice, or a layer that reads another layer's cache is a different list,
not different code.  The host library has the same records (include/inference.h);
a spec crosses as JSON.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional, Tuple


@dataclass
class PartSpec:
    """One part: its family's registered kind and every size/constant it needs.
    `name` is appended to the owner's tensor-name prefix ("self_attn", "mlp")."""
    kind: str
    params: Dict[str, Any] = field(default_factory=dict)
    name: str = ""

    def to_dict(self) -> dict:
        return {"kind": self.kind, "params": _plain(self.params), "name": self.name}

    @classmethod
    def from_dict(cls, d) -> "PartSpec":
        params = {k: (cls.from_dict(v) if isinstance(v, dict) and "kind" in v and "params" in v else v)
                  for k, v in (d.get("params") or {}).items()}
        return cls(d["kind"], params, d.get("name") or "")


def _plain(v):
    if isinstance(v, PartSpec):
        return v.to_dict()
    if isinstance(v, dict):
        return {k: _plain(x) for k, x in v.items()}
    if isinstance(v, (list, tuple)):
        return [_plain(x) for x in v]
    return v


@dataclass
class LayerSpec:
    """One layer: a block arrangement over named parts.  `prefix` starts the names of the
    layer's tensors in the checkpoint.  `cache_from` names another layer (by index into
    `ModelSpec.layers`) whose cache this layer's mixer reads instead of keeping one of its own."""
    prefix: str
    block: PartSpec
    parts: Dict[str, PartSpec]
    cache_from: Optional[int] = None


@dataclass
class ModelSpec:
    architecture: str
    vocab_size: int
    hidden_size: int
    embedding: PartSpec
    layers: List[LayerSpec]
    final_norm: PartSpec
    lm_head: PartSpec
    # order in which layers run: indices into `layers`; an index may appear twice
    schedule: Optional[List[int]] = None
    eos_token_ids: Tuple[int, ...] = ()
    max_position_embeddings: Optional[int] = None

    def run_order(self) -> List[int]:
        return list(range(len(self.layers))) if self.schedule is None else list(self.schedule)

    def to_dict(self) -> dict:
        return {"architecture": self.architecture, "vocab_size": self.vocab_size, "hidden_size": self.hidden_size,
                "embedding": self.embedding.to_dict(),
                "layers": [{"prefix": l.prefix, "block": l.block.to_dict(), "parts": {k: v.to_dict() for k, v in l.parts.items()},
                            "cache_from": l.cache_from} for l in self.layers],
                "final_norm": self.final_norm.to_dict(), "lm_head": self.lm_head.to_dict(),
                "schedule": None if self.schedule is None else list(self.schedule),
                "eos_token_ids": list(self.eos_token_ids), "max_position_embeddings": self.max_position_embeddings}

    @classmethod
    def from_dict(cls, d) -> "ModelSpec":
        layers = [LayerSpec(l["prefix"], PartSpec.from_dict(l["block"]),
                            {k: PartSpec.from_dict(v) for k, v in l["parts"].items()}, l.get("cache_from"))
                  for l in d["layers"]]
        return cls(d["architecture"], d["vocab_size"], d["hidden_size"], PartSpec.from_dict(d["embedding"]), layers,
                   PartSpec.from_dict(d["final_norm"]), PartSpec.from_dict(d["lm_head"]), d.get("schedule"),
                   tuple(d.get("eos_token_ids") or ()), d.get("max_position_embeddings"))


# ----------------------------------------------------------------- tensor needs
@dataclass(frozen=True)
class TensorNeed:
    """A checkpoint tensor a part asks for.

    role: "matrix"  — a matrix product operand, held in the engine's compute dtype
          "vector"  — a small vector used in 32-bit arithmetic, held in float32
          "table"   — an integer table, held in int32
    init: how the random-weights mode fills it: ("normal", mean, std), ("uniform", lo, hi), ("constant", v, 0)
    optional: absent from the checkpoint is allowed (the part copes)
    """
    shape: Tuple[int, ...]
    role: str = "matrix"
    init: Tuple[str, float, float] = ("normal", 0.0, 0.02)
    optional: bool = False

    def to_dict(self) -> dict:
        return {"shape": list(self.shape), "role": self.role, "init": self.init[0], "a": float(self.init[1]),
                "b": float(self.init[2]), "optional": self.optional}

    @classmethod
    def from_dict(cls, d) -> "TensorNeed":
        return cls(tuple(d["shape"]), d["role"], (d["init"], d["a"], d["b"]), d["optional"])


# -------------------------------------------------------------------- cache needs
@dataclass(frozen=True)
class PagedKVNeed:
    """Per-token keys and values in pages.  `window`: how many latest tokens are
    still read (None: all of them); pages wholly behind the window are given back."""
    kv_heads: int
    head_dim: int
    window: Optional[int] = None

    def to_dict(self) -> dict:
        return {"kind": "paged_kv", "kv_heads": self.kv_heads, "head_dim": self.head_dim, "window": self.window}


@dataclass(frozen=True)
class StateNeed:
    """Per-request state of fixed size (float32), zeroed when a request is admitted."""
    shape: Tuple[int, ...]

    def to_dict(self) -> dict:
        return {"kind": "state", "shape": list(self.shape)}


@dataclass(frozen=True)
class PagedRowsNeed:
    """Whatever a token keeps, `row_shape` elements per token and layer, in pages [page, row, ...] of
    the compute dtype (`float32`: of float32): a mixer with another kind of memory than keys and
    values.  `window` as for keys and values."""
    row_shape: Tuple[int, ...]
    float32: bool = False
    window: Optional[int] = None

    def to_dict(self) -> dict:
        return {"kind": "paged_rows", "row_shape": list(self.row_shape), "float32": self.float32, "window": self.window}


def cache_need_from_dict(d):
    if d is None:
        return None
    if d["kind"] == "state":
        return StateNeed(tuple(d["shape"]))
    if d["kind"] == "paged_rows":
        return PagedRowsNeed(tuple(d["row_shape"]), bool(d.get("float32")), d.get("window"))
    return PagedKVNeed(d["kv_heads"], d["head_dim"], d.get("window"))
