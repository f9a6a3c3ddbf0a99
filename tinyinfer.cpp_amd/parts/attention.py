"""Causal grouped-query attention over the paged cache.

Per token: q, k, v = h Wqkv^T (one fused matrix, no bias); every q head and
every k head is RMS-normed over head_dim with a weight shared by all heads
(before rotation; v is left alone); q and k are rotated by the position
encoding; k and v go into the cache page of the token's position; head h reads
kv head h // (heads / kv_heads), keys of its own request up to its own position
(and not older than `window`, if given), scores scaled by `scale`; the output
projection adds into the residual stream.
(/root/reference/src/inference.cu:41-55; src/cuda/attention.cu:12-87,107-198.)
"""
from __future__ import annotations

import math
from typing import Optional

import torch

from .base import Part, join
from .registry import register_part, build_part
from ..spec import TensorNeed, PagedKVNeed


class Attention(Part):
    family = "mixer"
    takes_lazy_norm = True      # h goes into one product and nowhere else

    def __init__(self, prefix: str, hidden: int, heads: int, kv_heads: int, head_dim: int,
                 qk_norm: bool = True, eps: float = 1e-6, window: Optional[int] = None,
                 scale: Optional[float] = None, pos=None, shares_kv: bool = False):
        super().__init__(prefix)
        if heads % kv_heads:
            raise ValueError(f"attention: heads {heads} not a multiple of kv_heads {kv_heads}")
        self.hidden, self.heads, self.kv_heads, self.head_dim = int(hidden), int(heads), int(kv_heads), int(head_dim)
        self.qk_norm = bool(qk_norm)
        self.eps = float(eps)
        self.window = None if window is None else int(window)
        self.scale = float(scale) if scale is not None else 1.0 / math.sqrt(self.head_dim)
        # a layer that reads another layer's keys and values projects only q
        self.shares_kv = bool(shares_kv)
        self.pos = build_part("pos", pos, prefix) if pos is not None else None
        self.nq = self.heads * self.head_dim
        self.nk = 0 if self.shares_kv else self.kv_heads * self.head_dim
        self.w_qkv = None
        self.w_o = None
        self.q_norm_w = None
        self.k_norm_w = None

    # ------------------------------------------------------------------ weights
    def tensors(self):
        H, hd = self.hidden, self.head_dim
        t = {join(self.prefix, "q_proj.weight"): TensorNeed((self.nq, H)),
             join(self.prefix, "o_proj.weight"): TensorNeed((H, self.nq))}
        if not self.shares_kv:
            t[join(self.prefix, "k_proj.weight")] = TensorNeed((self.nk, H))
            t[join(self.prefix, "v_proj.weight")] = TensorNeed((self.nk, H))
        if self.qk_norm:
            t[join(self.prefix, "q_norm.weight")] = TensorNeed((hd,), "vector", ("normal", 1.0, 0.1))
            if not self.shares_kv:
                t[join(self.prefix, "k_norm.weight")] = TensorNeed((hd,), "vector", ("normal", 1.0, 0.1))
        return t

    def load(self, tensors):
        names = ["q_proj.weight"] + ([] if self.shares_kv else ["k_proj.weight", "v_proj.weight"])
        self.w_qkv = torch.cat([tensors[join(self.prefix, n)] for n in names], dim=0).contiguous()
        self.w_o = tensors[join(self.prefix, "o_proj.weight")].contiguous()
        if self.qk_norm:
            self.q_norm_w = tensors[join(self.prefix, "q_norm.weight")]
            if not self.shares_kv:
                self.k_norm_w = tensors[join(self.prefix, "k_norm.weight")]
        if self.pos is not None and hasattr(self.pos, "to"):
            self.pos.to(self.w_o.device)

    def children(self):
        return [self.pos] if self.pos is not None else []

    # -------------------------------------------------------------------- cache
    def cache_need(self):
        return PagedKVNeed(self.kv_heads, self.head_dim, self.window)

    # ------------------------------------------------------------------ forward
    def forward(self, ctx, h, x):
        M = h.shape[0]
        width = self.nq + 2 * self.nk
        q = ctx.buf("attn.q", (M, self.nq), ctx.act_dtype)
        group, layer = ctx.binding(self)
        pool = ctx.kv_pool(group, layer)
        view = ctx.cache_view(group)
        rot = self.pos.fused_rotation() if self.pos is not None and hasattr(self.pos, "fused_rotation") else None
        a = ctx.buf("attn.out", (M, self.nq), ctx.act_dtype)
        fusable = self.pos is None or rot is not None     # a position encoding without a fused form needs qkv
        if fusable and not ctx.decode_only and ctx.ops.qkv_prepared(
                h, self.w_qkv, self.q_norm_w, self.k_norm_w, self.eps,
                None if rot is None else rot["inv_freq"], None if rot is None else rot.get("table"),
                ctx.positions, ctx.slots, view, pool, q, self.heads,
                0 if self.shares_kv else self.kv_heads, self.head_dim):
            # a step of many tokens: the projection's epilogue prepared q and wrote the cache
            ctx.ops.attention(ctx, view, q, pool, a, self.heads, self.kv_heads, self.head_dim, self.scale, self.window)
            ctx.ops.linear(a, self.w_o, x, "add", may_defer=True)
            return
        qkv = ctx.buf("attn.qkv", (M, width), ctx.f32)
        ctx.ops.linear(h, self.w_qkv, qkv, "store")
        if fusable and ctx.ops.attention_from_projections(
                ctx, view, qkv, self.q_norm_w, self.k_norm_w, self.eps,
                None if rot is None else rot["inv_freq"], None if rot is None else rot.get("table"),
                pool, not self.shares_kv, a, self.heads, self.kv_heads, self.head_dim, self.scale, self.window):
            # a step of single tokens: one kernel did it all
            ctx.ops.linear(a, self.w_o, x, "add", may_defer=True)
            return
        q_w, k_w = self.q_norm_w, self.k_norm_w
        if self.pos is not None and rot is None:
            # a position encoding without a fused form works on the 32-bit projections, after the
            # per-head norm (as in the fused order: norm, then position)
            n_k = 0 if self.shares_kv else self.kv_heads
            if q_w is not None or k_w is not None:
                ctx.ops.qk_norm_inplace(qkv, q_w, k_w, self.eps, self.heads, n_k, self.head_dim)
                q_w = k_w = None
            qv = qkv[:, :self.nq].unflatten(1, (self.heads, self.head_dim))
            kv = None if self.shares_kv else qkv[:, self.nq:self.nq + self.nk].unflatten(1, (self.kv_heads, self.head_dim))
            self.pos.apply(ctx, qv, kv)
        ctx.ops.qk_norm_rope_kv_write(
            qkv, q_w, k_w, self.eps,
            None if rot is None else rot["inv_freq"],
            ctx.positions, ctx.slots, view, pool, q,
            self.heads, 0 if self.shares_kv else self.kv_heads, self.head_dim,
            None if rot is None else rot.get("table"))
        ctx.ops.attention(ctx, view, q, pool, a, self.heads, self.kv_heads, self.head_dim,
                          self.scale, self.window)
        ctx.ops.linear(a, self.w_o, x, "add", may_defer=True)


register_part("mixer", "attention", Attention)
