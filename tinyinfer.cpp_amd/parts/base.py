"""What every part is: a holder of sizes, constants and weights that computes
through the kernels it is handed in the step context.  A part never looks at the
model it sits in; whatever it needs arrives as a constructor argument.

The built-in parts live in the host library (parts/parts.cpp); `NativePart`
(parts/builtin.py) names them from Python.  A part defined in Python subclasses
`Part`; the library then calls it through the step (native.py) with torch tensors
over the step's own memory.

Interfaces by family (M tokens in the step, H the residual width; `x` is the
32-bit residual stream [M, H], `h` an activation in the compute dtype):

  embedding  forward(ctx, tokens_i32[M], x)            fills x
  norm       forward(ctx, x, out=None, rows=None) -> h  (rows: gather these rows first)
  pos        apply(ctx, q, k)                           in place on 32-bit [M, heads, hd] views
  mixer      forward(ctx, h, x)                         adds its output into x
             cache_need() -> PagedKVNeed | StateNeed | None
  ffn        forward(ctx, h, x)                         adds its output into x
  block      forward(ctx, x)                            arranges its parts around x
  head       forward(ctx, h_rows) -> logits f32 [N, V]

What a part finds in `ctx` is listed in engine/context.py.  Before a part defined
in Python runs, the residual stream is complete (sums a product left for the next
norm are added), and `ctx.ops` completes it again before anything it launches.
"""
from __future__ import annotations

import ctypes
import json
from typing import Dict, List

from .. import native
from ..spec import TensorNeed


def join(prefix: str, name: str) -> str:
    if not prefix:
        return name
    if not name:
        return prefix
    return prefix + "." + name


class Handle:
    """A shared reference to a part of the host library."""

    def __init__(self, ptr: int):
        self.ptr = ptr

    def __del__(self):
        try:
            if self.ptr and native._lib is not None:
                native._lib.ti_part_release(self.ptr)
        except Exception:  # noqa: BLE001  (interpreter shutdown)
            pass

    def identity(self) -> int:
        return native.pointer("ti_part_pointer", self.ptr)


def children_arrays(children):
    """[(slot, part)] -> the C arrays of slot names and handles."""
    n = len(children)
    slots = (ctypes.c_char_p * max(1, n))(*[s.encode() for s, _ in children])
    handles = (ctypes.c_void_p * max(1, n))(*[part_handle(p).ptr for _, p in children])
    return n, slots, handles


def part_handle(part) -> Handle:
    """The library's part behind `part`: its own for a built-in part, else one that calls back into `part`."""
    h = getattr(part, "_ti_handle", None)
    if h is not None:
        return h
    description = {"tensors": {n: need.to_dict() for n, need in part.tensors().items()}}
    need = part.cache_need()
    if need is not None:
        description["cache_need"] = need.to_dict()
    kids = [(str(i), c) for i, c in enumerate(part.children())]
    n, slots, handles = children_arrays(kids)
    ptr = native.pointer("ti_part_create_foreign", part.family.encode(), native.register_foreign(part),
                         part.prefix.encode(), json.dumps(description).encode(), n, slots, handles)
    part._ti_handle = Handle(ptr)
    return part._ti_handle


class Part:
    family = ""

    def __init__(self, prefix: str = ""):
        self.prefix = prefix

    def tensors(self) -> Dict[str, TensorNeed]:
        """Checkpoint tensors of this part itself (children report their own)."""
        return {}

    def load(self, tensors) -> None:
        """Take the tensors named in `tensors()` (already on the device, already
        in the dtype their role asks for).  Absent optional tensors are missing keys."""

    def children(self) -> List["Part"]:
        return []

    def walk(self):
        yield self
        for c in self.children():
            yield from c.walk()

    def cache_need(self):
        return None
