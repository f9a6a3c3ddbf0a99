"""A model as data: which parts each layer is made of and in which order layers run.

Nothing here computes.  An architecture's builder turns its typed configuration
into a `ModelSpec`; the weight loader, the cache manager and the engine read
only the spec, so an architecture with other parts in some layers, a layer that
runs twice, or a layer that reads another layer's cache is a different list,
not different code.
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


@dataclass
class LayerSpec:
    """One layer: a block arrangement over named parts.

    `prefix` starts the names of the layer's tensors in the checkpoint.
    `cache_from` names another layer (by index into `ModelSpec.layers`) whose
    cache this layer's mixer reads instead of keeping one of its own.
    """
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


# ----------------------------------------------------------------- tensor needs
@dataclass(frozen=True)
class TensorNeed:
    """A checkpoint tensor a part asks for.

    role: "matrix"  — a matrix product operand, held in the engine's compute dtype
          "vector"  — a small vector used in 32-bit arithmetic, held in float32
          "table"   — an integer table, held in int32
    init: how the random-weights mode fills it: ("normal", mean, std)
    optional: absent from the checkpoint is allowed (the part copes)
    """
    shape: Tuple[int, ...]
    role: str = "matrix"
    init: Tuple[str, float, float] = ("normal", 0.0, 0.02)
    optional: bool = False


# -------------------------------------------------------------------- cache needs
@dataclass(frozen=True)
class PagedKVNeed:
    """Per-token keys and values in pages.  `window`: how many latest tokens are
    still read (None: all of them); pages wholly behind the window are given back."""
    kv_heads: int
    head_dim: int
    window: Optional[int] = None


@dataclass(frozen=True)
class StateNeed:
    """Per-request state of fixed size (float32), zeroed when a request is admitted."""
    shape: Tuple[int, ...]
