"""What a part defined in Python sees of a step: torch tensors over the step's own
memory, and the kernels.  The step itself is the host library's (`StepContext`,
include/inference.h); this object reads from it.

  ctx.ops                      the kernels (ops/kernels.py), launching where the step launches
  ctx.dtype / act_dtype / f32  the engine's compute dtype (name and torch dtype), and float32
  ctx.M                        tokens in the step
  ctx.tokens / positions / slots   int32 [M]: ids, positions, and each token's entry (row of the block tables)
  ctx.entries                  per entry: (first row, tokens, start position, state slot)
  ctx.decode_only              every entry is a single token
  ctx.buf(name, shape, dtype)  scratch memory, the same for the same name in every layer and step
  ctx.binding(part)            (group, cache layer) of the part's cache in this run of its layer
  ctx.kv_pool(group, layer)    [pages, 2, kv heads, P, head_dim]
  ctx.page_pool(group, layer)  [pages, P, ...]: the pages of a part that keeps rows of its own per token
  ctx.cache_view(group)        .table int32 [entries, pages per request], .page_size
  ctx.state(group, layer)      float32 [slots, ...]; index with an entry's state slot
"""
from __future__ import annotations

import ctypes
import json

from .. import native
from ..parts.base import part_handle


class CacheView:
    """The block-table rows of the step's entries, `table[entry][page index] -> page id`."""

    def __init__(self, table, page_size: int):
        self.table = table
        self.page_size = page_size


class StepContext:
    def __init__(self, ptr: int):
        from ..ops.kernels import Ops
        t = native.torch()
        self._native = ptr
        self._keep = []
        info = json.loads(native.text("ti_ctx_info", ptr))
        self.M = info["M"]
        self.decode_only = info["decode_only"]
        self.max_context = info["max_context"]
        self.dtype = info["dtype"]
        self.act_dtype = t.bfloat16 if self.dtype == "bfloat16" else t.float32
        self.f32 = t.float32
        self.device = t.device("cuda")
        self.entries = [tuple(e) for e in info["entries"]]
        self.ops = Ops(_borrowed=native.pointer("ti_ctx_ops", ptr))
        tok, pos, slot = ctypes.c_void_p(), ctypes.c_void_p(), ctypes.c_void_p()
        native.call("ti_ctx_pointers", ptr, ctypes.byref(tok), ctypes.byref(pos), ctypes.byref(slot))
        self.tokens, self.positions, self.slots = (self._ints(p.value, self.M) for p in (tok, pos, slot))

    @staticmethod
    def _ints(p, n):
        if not p:
            return None
        d = native.ti_tensor()
        d.data, d.dtype, d.ndim = p, 2, 1
        d.shape[0], d.stride[0] = n, 1
        return native.wrap(d)

    @property
    def run(self) -> int:
        return json.loads(native.text("ti_ctx_info", self._native))["run"]

    def buf(self, name: str, shape, dtype):
        shape = tuple(int(s) for s in shape)
        out = native.ti_tensor()
        native.call("ti_ctx_buf", self._native, name.encode(), native.dtype_code(dtype), len(shape),
                    (ctypes.c_int64 * max(1, len(shape)))(*shape), ctypes.byref(out))
        return native.wrap(out)

    def binding(self, part):
        g, l = ctypes.c_int(), ctypes.c_int()
        native.call("ti_ctx_binding", self._native, part_handle(part).ptr, ctypes.byref(g), ctypes.byref(l))
        return g.value, l.value

    def kv_pool(self, group: int, layer: int):
        out = native.ti_tensor()
        native.call("ti_ctx_kv_pool", self._native, group, layer, ctypes.byref(out))
        t = native.wrap(out)
        return t.view(t.shape[0], 2, t.shape[1] // 2, t.shape[2], t.shape[3])

    def page_pool(self, group: int, layer: int):
        """The pages of one cache layer as the library lays them out: [pages, P, ...] for a need of rows of
        its own (`PagedRowsNeed`), [pages, 2 x kv heads, P, head_dim] for keys and values."""
        out = native.ti_tensor()
        native.call("ti_ctx_kv_pool", self._native, group, layer, ctypes.byref(out))
        return native.wrap(out)

    def cache_view(self, group: int) -> CacheView:
        out, page = native.ti_tensor(), ctypes.c_int()
        native.call("ti_ctx_cache_view", self._native, group, ctypes.byref(out), ctypes.byref(page))
        return CacheView(native.wrap(out), page.value)

    def state(self, group: int, layer: int):
        """[slots, ...] float32 state of one cache layer; index with an entry's state slot."""
        out = native.ti_tensor()
        native.call("ti_ctx_state", self._native, group, layer, ctypes.byref(out))
        return native.wrap(out)
