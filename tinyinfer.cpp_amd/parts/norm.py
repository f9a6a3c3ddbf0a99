"""RMSNorm.  y = x * rsqrt(mean(x^2) + eps) * w, all in 32-bit; the weight
multiplies directly and eps sits inside the root
(/root/reference/src/cuda/rms_norm.cu:15-25)."""
from __future__ import annotations

from .base import Part, join
from .registry import register_part
from ..spec import TensorNeed
from ..ops.kernels import NormedRows


class RMSNorm(Part):
    family = "norm"
    can_be_lazy = True

    def __init__(self, prefix: str, dim: int, eps: float):
        super().__init__(prefix)
        self.dim = int(dim)
        self.eps = float(eps)
        self.weight = None

    def tensors(self):
        return {join(self.prefix, "weight"): TensorNeed((self.dim,), "vector", ("normal", 1.0, 0.1))}

    def load(self, tensors):
        self.weight = tensors[join(self.prefix, "weight")]

    def forward(self, ctx, x, out=None, rows=None, lazy=False):
        """x: f32 [M, dim].  Returns the normed rows in the compute dtype; with
        `rows` (i32 [N]) only those rows of x are read, in that order.  `lazy`: the
        caller's consumer feeds the result to one `ops.linear` and nothing else, so
        where a kernel can take the norm in, the rows come back not yet computed."""
        n = x.shape[0] if rows is None else rows.shape[0]
        if out is None:
            out = ctx.buf("norm.out", (n, self.dim), ctx.act_dtype)
        if lazy and rows is None and ctx.ops.can_fuse_norm(n, out.dtype):
            return NormedRows(x, self.weight, self.eps, out)
        ctx.ops.rmsnorm(x, self.weight, self.eps, out, rows)
        return out


register_part("norm", "rmsnorm", RMSNorm)
