"""Arrangements of parts around the residual stream.

`pre_norm`: x += mixer(norm1(x)); x += ffn(norm2(x))
(/root/reference/src/inference.cu:35-66).  The mixer and the feed-forward add
into x themselves, so the residual sum happens in 32-bit in their last kernel.
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

    def forward(self, ctx, x):
        h = self.norm1.forward(ctx, x)
        self.mixer.forward(ctx, h, x)
        h = self.norm2.forward(ctx, x)
        self.ffn.forward(ctx, h, x)


register_part("block", "pre_norm", PreNormBlock)
