"""The cache manager, named from Python: keys and values in pages with a block
table per request, one pool of pages per group of layers with the same need, and
slots for per-request state of fixed size.  The bookkeeping is the host
library's (cache/cache_manager.cpp, where the policy is described); an engine
owns one, and one can be made on its own (no GPU is needed).

Requests are named by any hashable value here; the library knows them by
64-bit numbers.
"""
from __future__ import annotations

import ctypes
import json
from typing import Dict, Hashable, List, Optional, Sequence, Tuple

from .. import native
from ..native import CacheError, OutOfPages  # noqa: F401
from ..spec import cache_need_from_dict


class PagePool:
    """Page ids 0..num_pages-1 with a LIFO free list (see the library's PagePool)."""

    def __init__(self, num_pages: int, scatter_window: int = 0, _borrowed: Optional[Tuple["CacheManager", int]] = None):
        self._borrowed = _borrowed
        self._ptr = None if _borrowed else native.pointer("ti_pool_create", int(num_pages), int(scatter_window))

    def __del__(self):
        try:
            if self._ptr and native._lib is not None:
                native._lib.ti_pool_release(self._ptr)
        except Exception:  # noqa: BLE001
            pass

    def _call(self, op: str, a: int = 0) -> int:
        out = ctypes.c_int64()
        if self._borrowed:
            manager, group = self._borrowed
            native.call("ti_cache_call", manager._ptr, ("pool_" + op).encode(), 0, group, a, ctypes.byref(out))
        else:
            native.call("ti_pool_call", self._ptr, op.encode(), a, ctypes.byref(out))
        return out.value

    num_free = property(lambda self: self._call("num_free"))
    num_pages = property(lambda self: self._call("num_pages"))
    high_water = property(lambda self: self._call("high_water"))
    taken_total = property(lambda self: self._call("taken_total"))

    def take(self) -> int:
        return self._call("take")

    def give_back(self, page: int) -> None:
        self._call("give_back", int(page))

    def free_list(self) -> List[int]:
        """The free pages; the last one is handed out next."""
        return json.loads(native.text("ti_pool_free_list", self._ptr))


class PagedGroup:
    """What the manager shows of one paged group."""

    def __init__(self, manager: "CacheManager", index: int, need, n_layers: int):
        self.need, self.n_layers, self.index = need, n_layers, index
        self.pool = PagePool(0, _borrowed=(manager, index))


class CacheManager:
    """groups: [(need, n_layers)] as `Model.cache_groups` lists them.  num_pages: pages in each paged
    group's pool."""

    def __init__(self, groups: Sequence[Tuple[object, int]] = (), page_size: int = 16, num_pages: int = 0,
                 max_requests: int = 64, max_seq: int = 0, scatter_window: int = 0, _borrowed: Optional[int] = None,
                 _owner=None):
        self._ids: Dict[Hashable, int] = {}
        self._names: Dict[int, Hashable] = {}
        self._next = 1
        self._owner = _owner                  # the engine whose manager this is (kept alive)
        self._own = _borrowed is None
        if _borrowed is None:
            spec = [{"need": need.to_dict(), "layers": n} for need, n in groups]
            self._ptr = native.pointer("ti_cache_create", json.dumps(spec).encode(), int(page_size), int(num_pages),
                                       int(max_requests), int(max_seq), int(scatter_window))
        else:
            self._ptr = _borrowed
        d = self.dump()
        self.page_size, self.max_requests, self.max_seq = d["page_size"], d["max_requests"], d["max_seq"]
        self.max_pages_per_request = d["table_width"]
        self.groups: List[object] = []
        for i, g in enumerate(d["groups"]):
            need = cache_need_from_dict(g["need"])
            self.groups.append(PagedGroup(self, i, need, g["layers"]) if g["paged"] else need)
        self.group_layers = [g["layers"] for g in d["groups"]]

    def __del__(self):
        try:
            if self._own and native._lib is not None:
                native._lib.ti_cache_release(self._ptr)
        except Exception:  # noqa: BLE001
            pass

    # ------------------------------------------------------------------ names
    def key(self, req: Hashable) -> int:
        """The library's number for `req` (a request the scheduler made is known by its own number)."""
        if isinstance(req, tuple) and len(req) == 2 and req[0] == "req#":
            return int(req[1])
        k = self._ids.get(req)
        if k is None:
            k = self._ids[req] = self._next
            self._names[k] = req
            self._next += 1
        return k

    def _name(self, k: int) -> Hashable:
        return self._names.get(k, ("req#", k))

    def _call(self, op: str, req: Optional[Hashable] = None, a: int = 0, b: int = 0) -> int:
        out = ctypes.c_int64()
        native.call("ti_cache_call", self._ptr, op.encode(), 0 if req is None else self.key(req), int(a), int(b),
                    ctypes.byref(out))
        return out.value

    # ---------------------------------------------------------------- queries
    def dump(self) -> dict:
        return json.loads(native.text("ti_cache_dump", self._ptr))

    def paged_groups(self):
        return [(i, g) for i, g in enumerate(self.groups) if isinstance(g, PagedGroup)]

    def state_groups(self):
        return [(i, g) for i, g in enumerate(self.groups) if not isinstance(g, PagedGroup)]

    def has(self, req: Hashable) -> bool:
        return bool(self._call("has", req))

    def live_requests(self):
        return [self._name(k) for k in self.dump()["live"]]

    def length(self, req: Hashable) -> int:
        return self._call("length", req)

    def slot(self, req: Hashable) -> int:
        return self._call("slot", req)

    def num_free_slots(self) -> int:
        return self._call("num_free_slots")

    def num_free_pages(self) -> int:
        """Free pages of the tightest group."""
        return self._call("num_free_pages")

    def table(self, group: int, req: Hashable) -> List[int]:
        return json.loads(native.text("ti_cache_table", self._ptr, int(group), self.key(req)))

    def can_reserve(self, req: Hashable, n_tokens: int) -> bool:
        return bool(self._call("can_reserve", req, n_tokens))

    @property
    def slots_to_clear(self) -> List[int]:
        """Slots whose state must be zeroed before their next use (the engine does it at its next step)."""
        return self.dump()["slots_to_clear"]

    def forget_slots_to_clear(self) -> None:
        self._call("clear_slots_list")

    # ---------------------------------------------------------------- actions
    def admit(self, req: Hashable) -> int:
        return self._call("admit", req)

    def reserve(self, req: Hashable, n_tokens: int) -> None:
        self._call("reserve", req, n_tokens)

    def commit(self, req: Hashable, n_tokens: int) -> None:
        self._call("commit", req, n_tokens)

    def rollback(self, req: Hashable) -> None:
        self._call("rollback", req)

    def _many(self, op: str, reqs: Sequence[Hashable]):
        for q in reqs:
            if q not in self._ids and not (isinstance(q, tuple) and len(q) == 2 and q[0] == "req#"):
                raise CacheError(f"request {q!r} is not admitted")
        ids = (ctypes.c_int64 * max(1, len(reqs)))(*[self.key(q) for q in reqs])
        return json.loads(native.text("ti_cache_many", self._ptr, op.encode(), len(reqs), ids))

    def reserve_one_each(self, reqs: Sequence[Hashable]) -> List[int]:
        return self._many("reserve_one_each", reqs)

    def commit_one_each(self, reqs: Sequence[Hashable]) -> None:
        self._many("commit_one_each", reqs)

    def release(self, req: Hashable) -> None:
        self._call("release", req)
        k = self._ids.pop(req, None)
        if k is not None:
            self._names.pop(k, None)

    def check(self) -> None:
        """No page lost, held twice or free while held; tables cover what they must (raises CacheError)."""
        self._call("check")
