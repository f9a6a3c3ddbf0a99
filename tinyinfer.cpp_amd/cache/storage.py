"""The device tensors behind the cache manager: one pool of pages per paged
group, `[cache layer][page][K|V][kv head][...]`, and one block of state per
state group, `[cache layer][slot][...]`.  Within a page the keys of a kv head lie
`[row in page][head_dim]` (a score sums over head_dim) and the values transposed,
`[head_dim][row in page]` (the mix sums over rows): each is contiguous along the
dimension the matrix cores reduce over.  The tensor's nominal shape is
`[..., P, head_dim]` for both halves.

A page id addresses the same slot in every cache layer of its group.  At
Qwen3-0.6B sizes (8 kv heads x 128, 16 rows) a page is 64 KiB per layer in
bfloat16, and one kv head's rows of a page are 4 KiB contiguous: a flash
decoding workgroup streams whole pages.
"""
from __future__ import annotations

from typing import List

import torch

from .manager import CacheManager, PagedGroup
from ..spec import StateNeed


class CacheStorage:
    def __init__(self, manager: CacheManager, dtype: torch.dtype, device):
        self.manager = manager
        self.kv: List[torch.Tensor] = []
        self.state: List[torch.Tensor] = []
        for g, n_layers in zip(manager.groups, manager.group_layers):
            if isinstance(g, PagedGroup):
                self.kv.append(torch.empty(
                    (n_layers, g.pool.num_pages, 2, g.need.kv_heads, manager.page_size, g.need.head_dim),
                    dtype=dtype, device=device))
                self.state.append(None)
            elif isinstance(g, StateNeed):
                self.kv.append(None)
                self.state.append(torch.zeros((n_layers, manager.max_requests) + tuple(g.shape),
                                              dtype=torch.float32, device=device))

    def clear_slots(self, slots) -> None:
        """Zero the state of newly admitted requests (a fill kernel, not a memset)."""
        for s in self.state:
            if s is not None:
                for slot in slots:
                    s[:, slot].zero_()

    def bytes(self) -> int:
        return sum(t.numel() * t.element_size() for t in self.kv + self.state if t is not None)
