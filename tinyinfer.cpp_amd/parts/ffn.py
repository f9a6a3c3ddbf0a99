"""SwiGLU feed-forward: y = silu(h Wg^T) * (h Wu^T); out = y Wd^T, no biases
(/root/reference/src/inference.cu:60-65; src/cuda/ffn.cu:13-15).  Gate and up
rows are held as one matrix [2F, H] so one product yields both
(src/inference.cu:155-160) and the SwiGLU runs in its epilogue."""
from __future__ import annotations

import torch

from .base import Part, join
from .registry import register_part
from ..spec import TensorNeed


class SwiGLU(Part):
    family = "ffn"
    takes_lazy_norm = True      # h goes into one product and nowhere else

    def __init__(self, prefix: str, hidden: int, intermediate: int):
        super().__init__(prefix)
        self.hidden = int(hidden)
        self.intermediate = int(intermediate)
        self.w_gate_up = None
        self.w_down = None

    def tensors(self):
        H, F = self.hidden, self.intermediate
        return {
            join(self.prefix, "gate_proj.weight"): TensorNeed((F, H)),
            join(self.prefix, "up_proj.weight"): TensorNeed((F, H)),
            join(self.prefix, "down_proj.weight"): TensorNeed((H, F)),
        }

    def load(self, tensors):
        g = tensors[join(self.prefix, "gate_proj.weight")]
        u = tensors[join(self.prefix, "up_proj.weight")]
        self.w_gate_up = torch.cat([g, u], dim=0).contiguous()
        self.w_down = tensors[join(self.prefix, "down_proj.weight")].contiguous()

    def forward(self, ctx, h, x):
        M = h.shape[0]
        y = ctx.buf("ffn.y", (M, self.intermediate), ctx.act_dtype)
        ctx.ops.linear(h, self.w_gate_up, y, "swiglu")
        ctx.ops.linear(y, self.w_down, x, "add", may_defer=True)


register_part("ffn", "swiglu", SwiGLU)
