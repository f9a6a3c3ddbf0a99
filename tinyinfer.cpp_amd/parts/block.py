"""Arrangements of parts around the residual stream.

`pre_norm`: x += mixer(norm1(x)); x += ffn(norm2(x))
(/root/reference/src/inference.cu:35-66).  The mixer and the feed-forward add
into x themselves, so the residual sum happens in 32-bit in their last kernel.
The framework's own mixers and feed-forwards let that kernel leave part of the sum
to the norm that reads x next (`ops.linear(..., may_defer=True)`); a part that reads
x other than through `ctx.ops` calls `ctx.ops.flush()` first.
"""
from __future__ import annotations

from .base import Part
from .registry import register_part


class PreNormBlock(Part):
    family = "block"
    # which family each named slot of this arrangement is built from
    slots = {"norm1": "norm", "mixer": "mixer", "norm2": "norm", "ffn": "ffn"}

    def __init__(self, prefix: str, norm1, mixer, norm2, ffn):
        super().__init__(prefix)
        self.norm1, self.mixer, self.norm2, self.ffn = norm1, mixer, norm2, ffn

    def children(self):
        return [self.norm1, self.mixer, self.norm2, self.ffn]

    @staticmethod
    def _normed(ctx, norm, consumer, x):
        # a consumer that feeds h to exactly one `ops.linear` says so (`takes_lazy_norm`);
        # a norm that can hand its rows over uncomputed takes the `lazy` argument
        if getattr(consumer, "takes_lazy_norm", False) and getattr(norm, "can_be_lazy", False):
            return norm.forward(ctx, x, lazy=True)
        return norm.forward(ctx, x)

    def forward(self, ctx, x):
        h = self._normed(ctx, self.norm1, self.mixer, x)
        self.mixer.forward(ctx, h, x)
        h = self._normed(ctx, self.norm2, self.ffn, x)
        self.ffn.forward(ctx, h, x)


register_part("block", "pre_norm", PreNormBlock)
