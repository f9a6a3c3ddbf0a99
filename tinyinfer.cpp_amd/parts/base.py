"""What every part is: a holder of sizes, constants and weights that computes
through the kernels it is handed in the step context.  A part never looks at the
model it sits in; whatever it needs arrives as a constructor argument.

Interfaces by family (M tokens in the step, H the residual width; `x` is the
32-bit residual stream [M, H], `h` an activation in the compute dtype):

  embedding  forward(ctx, tokens_i32[M], x)            fills x
  norm       forward(ctx, x, out=None, rows=None) -> h  (rows: gather these rows first)
  pos        fused_rotation() -> dict or None          arguments for the fused q/k kernel
             apply(ctx, q, k)                           in place on 32-bit [M, heads, hd] views
  mixer      forward(ctx, h, x)                         adds its output into x
             cache_need() -> PagedKVNeed | StateNeed | None
  ffn        forward(ctx, h, x)                         adds its output into x
  block      forward(ctx, x)                            arranges its parts around x
  head       forward(ctx, h_rows) -> logits f32 [N, V]

Optional, for fewer kernels when a step has few tokens: a norm with the class
attribute `can_be_lazy` takes `forward(..., lazy=True)` and may then return its
rows not yet computed (`ops.kernels.NormedRows`); a block passes `lazy=True` only
for a consumer with the class attribute `takes_lazy_norm`, which promises to hand
h to exactly one `ctx.ops.linear` and to use nothing of it but its `shape`.
"""
from __future__ import annotations

from typing import Dict, List

from ..spec import TensorNeed


def join(prefix: str, name: str) -> str:
    if not prefix:
        return name
    if not name:
        return prefix
    return prefix + "." + name


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
