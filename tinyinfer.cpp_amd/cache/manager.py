"""The cache manager: keys and values in pages with a block table per request,
one pool of pages per group of layers with the same need, and slots for
per-request state of fixed size.

The reference keeps one slab `[layer][sequence][K/V][kv head][max_seq][head_dim]`
that is allocated once for `max_batch x max_seq` tokens and never given back
per request (/root/reference/src/inference.cu:146-148,174-176).  Here a token
at position `pos` of a request lives in page `table[pos // P]` at row `pos % P`;
pages come from a LIFO free list (a page given back is the next one handed
out), are given back when the request ends, and, in a group whose layers read
only a window of keys, as soon as the window has passed them.  Page contents
are never cleared: a request reads only rows it has written itself.

Everything in this file is host bookkeeping; the tensors that hold the pages
and the state live in `CacheStorage`.
"""
from __future__ import annotations

import random

import numpy as np
from dataclasses import dataclass
from typing import Dict, Hashable, List, Optional, Sequence, Tuple

from ..spec import PagedKVNeed, StateNeed


class CacheError(RuntimeError):
    pass


class OutOfPages(CacheError):
    """A reservation that the free pages cannot cover.  Nothing was taken."""


class PagePool:
    """Page ids 0..num_pages-1 with a LIFO free list.

    `scatter_window` > 0: the pages are first handed out in a fixed pseudo-random order within
    windows of that many pages (window after window) instead of 0, 1, 2, ...  Requests that
    are filled one after the other then do not lie at equal distances in memory; at equal
    distances the attention kernels, which walk all requests in step, keep hitting the same
    memory channels (measured on MI355X, a decode step of 64 requests of 2,048 tokens: 5.49 ms
    in order, 5.03 ms shuffled within windows of 512 pages or over the whole pool, 5.58 ms within
    windows of 64; a step of 8 requests is 1 % faster in order or in windows of 512 than
    shuffled over the whole pool)."""

    def __init__(self, num_pages: int, scatter_window: int = 0):
        if num_pages <= 0:
            raise CacheError(f"a page pool needs at least one page, got {num_pages}")
        self.num_pages = int(num_pages)
        order = list(range(self.num_pages))
        if scatter_window > 1:
            rnd = random.Random(self.num_pages)
            for i in range(0, self.num_pages, scatter_window):
                chunk = order[i:i + scatter_window]
                rnd.shuffle(chunk)
                order[i:i + scatter_window] = chunk
        self._free: List[int] = order[::-1]                                # pop() gives order[0] first
        self._held = [False] * self.num_pages
        self.high_water = 0
        self.taken_total = 0          # pages handed out so far, counting a page again each time

    @property
    def num_free(self) -> int:
        return len(self._free)

    def take(self) -> int:
        if not self._free:
            raise OutOfPages("no free page")
        p = self._free.pop()
        assert not self._held[p], f"page {p} handed out twice"
        self._held[p] = True
        self.taken_total += 1
        self.high_water = max(self.high_water, self.num_pages - len(self._free))
        return p

    def give_back(self, p: int) -> None:
        if not (0 <= p < self.num_pages) or not self._held[p]:
            raise CacheError(f"page {p} given back but not held")
        self._held[p] = False
        self._free.append(p)


@dataclass
class _Request:
    slot: int
    length: int = 0            # tokens committed
    reserved: int = 0          # tokens that have pages (>= length)


class PagedGroup:
    """Pages and block tables of one group of layers."""

    def __init__(self, need: PagedKVNeed, n_layers: int, page_size: int, num_pages: int, table_width: int,
                 scatter_window: int = 0):
        self.need = need
        self.n_layers = n_layers
        self.page_size = page_size
        self.pool = PagePool(num_pages, scatter_window)
        self.tables: Dict[Hashable, List[int]] = {}      # -1: given back (behind the window)
        # the same as rows of `table_width` int32 (-1 where there is no page), ready to be
        # copied into a step's metadata
        self.table_width = table_width
        self.rows: Dict[Hashable, np.ndarray] = {}

    def new_table(self, req: Hashable) -> None:
        self.tables[req] = []
        self.rows[req] = np.full(self.table_width, -1, dtype=np.int32)

    def append_page(self, req: Hashable) -> None:
        t = self.tables[req]
        page = self.pool.take()
        self.rows[req][len(t)] = page
        t.append(page)

    def give_back_page(self, req: Hashable, index: int) -> None:
        t = self.tables[req]
        self.pool.give_back(t[index])
        t[index] = -1
        self.rows[req][index] = -1

    def drop_table(self, req: Hashable) -> None:
        t = self.tables.pop(req)
        del self.rows[req]
        for p in reversed(t):              # so the lowest page is handed out next
            if p >= 0:
                self.pool.give_back(p)

    def first_needed_page(self, next_pos: int) -> int:
        """Index of the first page that a query at `next_pos` or later still reads."""
        if self.need.window is None:
            return 0
        return max(0, next_pos - self.need.window + 1) // self.page_size

    def pages_to_cover(self, req: Hashable, upto: int) -> int:
        have = len(self.tables.get(req, ()))
        want = -(-upto // self.page_size)
        return max(0, want - have)


class CacheManager:
    """Admits requests, reserves pages for their next tokens in every group at
    once, advances their length, gives pages and slots back.

    groups: [(need, n_layers)] as `Model.cache_groups` lists them.
    num_pages: pages in each paged group's pool.
    """

    def __init__(self, groups: Sequence[Tuple[object, int]], page_size: int, num_pages: int,
                 max_requests: int, max_seq: int, scatter_window: int = 0):
        if page_size <= 0:
            raise CacheError("page_size must be positive")
        self.page_size = int(page_size)
        self.max_requests = int(max_requests)
        self.max_seq = int(max_seq)
        self.max_pages_per_request = -(-self.max_seq // self.page_size)
        self.groups: List[object] = []
        for need, n_layers in groups:
            if isinstance(need, PagedKVNeed):
                self.groups.append(PagedGroup(need, n_layers, self.page_size, num_pages,
                                              self.max_pages_per_request, scatter_window))
            elif isinstance(need, StateNeed):
                self.groups.append(need)
            else:
                raise CacheError(f"unknown cache need {need!r}")
        self.group_layers = [n for _, n in groups]
        self._paged = [(i, g) for i, g in enumerate(self.groups) if isinstance(g, PagedGroup)]
        self._requests: Dict[Hashable, _Request] = {}
        self._free_slots: List[int] = list(range(self.max_requests - 1, -1, -1))
        # slots whose state tensors must be zeroed before their next use
        self.slots_to_clear: List[int] = []

    # ---------------------------------------------------------------- queries
    def paged_groups(self):
        return self._paged

    def state_groups(self):
        return [(i, g) for i, g in enumerate(self.groups) if isinstance(g, StateNeed)]

    def has(self, req: Hashable) -> bool:
        return req in self._requests

    def live_requests(self):
        return list(self._requests)

    def length(self, req: Hashable) -> int:
        return self._requests[req].length

    def slot(self, req: Hashable) -> int:
        return self._requests[req].slot

    def num_free_slots(self) -> int:
        return len(self._free_slots)

    def num_free_pages(self) -> int:
        """Free pages of the tightest group."""
        paged = self.paged_groups()
        return min((g.pool.num_free for _, g in paged), default=1 << 30)

    def table(self, group: int, req: Hashable) -> List[int]:
        return self.groups[group].tables[req]

    def pages_needed(self, req: Optional[Hashable], n_tokens: int, length: Optional[int] = None) -> int:
        """Most pages any group must newly take for `n_tokens` more tokens of
        `req` (`req` None: a request not admitted yet, of `length` 0)."""
        r = self._requests.get(req) if req is not None else None
        base = (r.reserved if r else 0) if length is None else length
        worst = 0
        for _, g in self.paged_groups():
            worst = max(worst, g.pages_to_cover(req, base + n_tokens))
        return worst

    def can_reserve(self, req: Optional[Hashable], n_tokens: int) -> bool:
        r = self._requests.get(req) if req is not None else None
        base = r.reserved if r else 0
        if base + n_tokens > self.max_seq:
            return False
        for _, g in self.paged_groups():
            if g.pages_to_cover(req, base + n_tokens) > g.pool.num_free:
                return False
        return True

    # ---------------------------------------------------------------- actions
    def admit(self, req: Hashable) -> int:
        """Give `req` a state slot (its state is cleared before first use) and
        empty block tables.  Returns the slot."""
        if req in self._requests:
            raise CacheError(f"request {req!r} is already admitted")
        if not self._free_slots:
            raise CacheError(f"no free request slot (max_requests = {self.max_requests})")
        slot = self._free_slots.pop()
        self._requests[req] = _Request(slot)
        for _, g in self.paged_groups():
            g.new_table(req)
        self.slots_to_clear.append(slot)
        return slot

    def reserve(self, req: Hashable, n_tokens: int) -> None:
        """Make positions [reserved, reserved + n_tokens) writable in every paged
        group, or raise OutOfPages and take nothing."""
        r = self._requests[req]
        upto = r.reserved + n_tokens
        if upto > self.max_seq:
            raise CacheError(f"request {req!r}: {upto} tokens exceed max_seq = {self.max_seq}")
        for _, g in self.paged_groups():
            need = g.pages_to_cover(req, upto)
            if need > g.pool.num_free:
                raise OutOfPages(f"request {req!r} needs {need} more pages for {n_tokens} tokens, "
                                 f"{g.pool.num_free} are free")
        for _, g in self.paged_groups():
            for _ in range(g.pages_to_cover(req, upto)):
                g.append_page(req)
        r.reserved = upto

    def commit(self, req: Hashable, n_tokens: int) -> None:
        """The step wrote `n_tokens` more tokens of `req`.  Pages that every
        later query's window has passed are given back."""
        r = self._requests[req]
        if r.length + n_tokens > r.reserved:
            raise CacheError(f"request {req!r}: committing {n_tokens} tokens beyond its reservation")
        r.length += n_tokens
        for _, g in self.paged_groups():
            first = g.first_needed_page(r.length)
            if first == 0:
                continue
            t = g.tables[req]
            for i in range(min(first, len(t))):
                if t[i] >= 0:
                    g.give_back_page(req, i)

    # ---- a decode step: one token for each of several admitted requests.  The same as `reserve`
    # (for all of them or for none) and `commit` per request, without their per-request overhead.
    def reserve_one_each(self, reqs: Sequence[Hashable]) -> List[int]:
        """Make one more position writable for every request of `reqs` (all admitted, each
        once), or raise OutOfPages and take nothing.  Returns their lengths (the positions
        the new tokens take)."""
        try:
            rs = [self._requests[q] for q in reqs]
        except KeyError as e:
            raise CacheError(f"request {e.args[0]!r} is not admitted") from None
        P = self.page_size
        starts = []
        for r, q in zip(rs, reqs):
            if r.reserved != r.length:
                raise CacheError(f"request {q!r} has a reservation that was not committed")
            if r.reserved + 1 > self.max_seq:
                raise CacheError(f"request {q!r}: {r.reserved + 1} tokens exceed max_seq = {self.max_seq}")
            starts.append(r.length)
        todo = []
        for _, g in self._paged:
            tables = g.tables
            short = [q for r, q in zip(rs, reqs) if len(tables[q]) * P <= r.reserved]
            if len(short) > g.pool.num_free:
                raise OutOfPages(f"the step needs {len(short)} new pages, {g.pool.num_free} are free")
            if short:
                todo.append((g, short))
        for g, short in todo:
            for q in short:
                g.append_page(q)
        for r in rs:
            r.reserved += 1
        return starts

    def commit_one_each(self, reqs: Sequence[Hashable]) -> None:
        """The step wrote one more token of every request of `reqs` (see `commit`)."""
        P = self.page_size
        windowed = [g for _, g in self._paged if g.need.window is not None]
        for q in reqs:
            r = self._requests[q]
            if r.length + 1 > r.reserved:
                raise CacheError(f"request {q!r}: committing a token beyond its reservation")
            r.length += 1
            for g in windowed:
                # a page falls behind the window only when the window's first position enters a new page
                lo = r.length - g.need.window + 1
                if lo > 0 and lo % P == 0:
                    t = g.tables[q]
                    for i in range(min(lo // P, len(t))):
                        if t[i] >= 0:
                            g.give_back_page(q, i)

    def release(self, req: Hashable) -> None:
        """The request is over (finished, aborted or preempted): every page and
        its slot go back."""
        r = self._requests.pop(req, None)
        if r is None:
            raise CacheError(f"request {req!r} released but not admitted")
        for _, g in self.paged_groups():
            g.drop_table(req)
        self._free_slots.append(r.slot)

    # ------------------------------------------------------------- invariants
    def check(self) -> None:
        """No page lost, held twice or free while held; tables cover what they must."""
        for gi, g in self.paged_groups():
            held = []
            for req, t in g.tables.items():
                r = self._requests[req]
                assert len(t) * self.page_size >= r.reserved, (gi, req, "table shorter than reservation")
                row = g.rows[req]
                assert list(row[:len(t)]) == t and (row[len(t):] == -1).all(), (gi, req, "the table's row differs")
                first = g.first_needed_page(r.length)
                for i, p in enumerate(t):
                    if i >= first:
                        assert p >= 0, (gi, req, i, "a page still read was given back")
                    if p >= 0:
                        held.append(p)
            assert len(held) == len(set(held)), (gi, "a page is in two places")
            free = list(g.pool._free)
            assert len(free) == len(set(free)), (gi, "a page is free twice")
            assert not (set(free) & set(held)), (gi, "a page is free and held")
            assert len(free) + len(held) == g.pool.num_pages, (gi, "a page is lost")
        slots = [r.slot for r in self._requests.values()]
        assert len(slots) == len(set(slots)), "a slot is held twice"
        assert sorted(slots + self._free_slots) == list(range(self.max_requests)), "a slot is lost"
