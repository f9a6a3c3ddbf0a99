"""Half-split ("NeoX") rotary position encoding over the whole head: pair
(k, k + hd/2) turns by pos * theta^(-2k/hd)
(/root/reference/src/cuda/attention.cu:38,64-74; src/cuda/rope.cu:20-28; the
adjacent-pair variant is the mistake listed in docs/report.md:91).

The inverse frequencies are built once on the host in double precision and
rounded to float; the angle pos * inv_freq[k] and its sine and cosine are 32-bit
on the device.  `prepare(n)` tabulates them for positions below n (with the same
device function a kernel would call for a position beyond the table).
"""
from __future__ import annotations

import torch

from .base import Part
from .registry import register_part


class RotaryNeox(Part):
    family = "pos"

    def __init__(self, prefix: str, head_dim: int, theta: float):
        super().__init__(prefix)
        if head_dim % 2:
            raise ValueError(f"rotary: head_dim {head_dim} must be even")
        self.head_dim = int(head_dim)
        self.theta = float(theta)
        half = self.head_dim // 2
        k = torch.arange(half, dtype=torch.float64)
        self._inv_freq_host = torch.pow(
            torch.tensor(self.theta, dtype=torch.float64), -2.0 * k / self.head_dim).to(torch.float32)
        self.inv_freq = None
        self.table = None

    def to(self, device):
        self.inv_freq = self._inv_freq_host.to(device)
        self.table = None
        return self

    def prepare(self, ops, max_positions: int):
        """Tabulate cos and sin for positions [0, max_positions)."""
        if self.inv_freq is not None and (self.table is None or self.table.shape[0] < max_positions):
            self.table = ops.rope_table(self.inv_freq, int(max_positions))

    def fused_rotation(self):
        """Arguments for the fused norm/rotate/cache-write kernel."""
        return {"inv_freq": self.inv_freq, "table": self.table}

    def apply(self, ctx, q, k):
        """In place on f32 [M, heads, hd] views (strided rows allowed)."""
        ctx.ops.rope_neox(q, ctx.positions, self.inv_freq)
        if k is not None:
            ctx.ops.rope_neox(k, ctx.positions, self.inv_freq)


register_part("pos", "rope_neox", RotaryNeox)
