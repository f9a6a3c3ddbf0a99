"""Token embedding x[m, :] = float(E[tok[m], :]), no scaling
(/root/reference/src/inference.cu:14-24), and the output head
logits = h E_out^T with E_out the embedding itself or a matrix of its own
(/root/reference/src/cuda/lm_head.cu:5-10; the reference is always tied,
src/model.h:42)."""
from __future__ import annotations

from .base import Part, join
from .registry import register_part
from ..spec import TensorNeed


class Embedding(Part):
    family = "embedding"

    def __init__(self, prefix: str, vocab: int, dim: int):
        super().__init__(prefix)
        self.vocab = int(vocab)
        self.dim = int(dim)
        self.weight = None

    def tensors(self):
        return {join(self.prefix, "weight"): TensorNeed((self.vocab, self.dim))}

    def load(self, tensors):
        self.weight = tensors[join(self.prefix, "weight")]

    def forward(self, ctx, tokens, x):
        ctx.ops.embed(self.weight, tokens, x)


class LMHead(Part):
    """`tied`: True reads `tied_to`; False reads its own `weight`; None takes
    its own weight if the checkpoint holds one and `tied_to` otherwise."""
    family = "head"

    def __init__(self, prefix: str, vocab: int, dim: int, tied, tied_to: str):
        super().__init__(prefix)
        self.vocab = int(vocab)
        self.dim = int(dim)
        self.tied = tied
        self.tied_to = tied_to
        self.weight = None

    def tensors(self):
        own = join(self.prefix, "weight")
        shape = (self.vocab, self.dim)
        if self.tied is True:
            # a checkpoint that still carries the duplicate is accepted
            return {self.tied_to: TensorNeed(shape), own: TensorNeed(shape, optional=True)}
        if self.tied is False:
            return {own: TensorNeed(shape)}
        return {self.tied_to: TensorNeed(shape), own: TensorNeed(shape, optional=True)}

    def load(self, tensors):
        own = join(self.prefix, "weight")
        if self.tied is False or (self.tied is None and own in tensors):
            self.weight = tensors[own]
        else:
            self.weight = tensors[self.tied_to]

    def forward(self, ctx, h_rows):
        n = h_rows.shape[0]
        logits = ctx.buf("head.logits", (n, self.vocab), ctx.f32)
        ctx.ops.linear(h_rows, self.weight, logits, "store")
        return logits


register_part("embedding", "table", Embedding)
register_part("head", "linear", LMHead)
