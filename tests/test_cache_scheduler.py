"""The cache manager and the scheduler's decisions (host only, no GPU)."""
import random

import pytest

from tinyinfer_amd.cache import CacheError, CacheManager, OutOfPages
from tinyinfer_amd.engine.scheduler import Scheduler, SchedulerError
from tinyinfer_amd.sampling import SamplingParams, uniform
from tinyinfer_amd.spec import PagedKVNeed, PagedRowsNeed, StateNeed

FULL = PagedKVNeed(2, 16, None)
WIN = PagedKVNeed(2, 16, 10)


def manager(groups=((FULL, 2),), page_size=4, pages=12, slots=4, max_seq=64):
    return CacheManager(list(groups), page_size, pages, slots, max_seq)


def test_pages_are_taken_in_order_and_reused_lifo():
    m = manager()
    m.admit("a")
    m.reserve("a", 9)                                  # 3 pages
    assert m.table(0, "a") == [0, 1, 2]
    m.commit("a", 9)
    m.admit("b")
    m.reserve("b", 4)
    assert m.table(0, "b") == [3]
    m.release("a")
    m.admit("c")
    m.reserve("c", 5)
    assert m.table(0, "c") == [0, 1]                   # a's pages are handed out again, lowest first
    m.check()


def test_pages_scattered_within_windows_are_a_permutation():
    """With a scatter window every page is still handed out exactly once, each from the window
    that is due, in an order that is not 0, 1, 2, ...; released pages come back LIFO as before."""
    from tinyinfer_amd.cache.manager import PagePool
    pool = PagePool(70, scatter_window=16)
    taken = [pool.take() for _ in range(70)]
    assert sorted(taken) == list(range(70))
    for i in range(0, 70, 16):
        assert sorted(taken[i:i + 16]) == list(range(i, min(i + 16, 70)))
    assert taken != list(range(70))
    assert PagePool(70, scatter_window=16).free_list() == PagePool(70, scatter_window=16).free_list()   # a fixed order
    with pytest.raises(OutOfPages):
        pool.take()
    pool.give_back(taken[3])
    pool.give_back(taken[40])
    assert pool.take() == taken[40] and pool.take() == taken[3]
    m = CacheManager([(FULL, 1)], page_size=4, num_pages=64, max_requests=2, max_seq=128, scatter_window=8)
    m.admit("a")
    m.reserve("a", 100)
    m.commit("a", 100)
    m.check()
    m.release("a")
    m.check()
    assert m.num_free_pages() == 64


def test_reserve_is_all_or_nothing():
    m = manager(pages=3)
    m.admit("a")
    m.reserve("a", 8)
    with pytest.raises(OutOfPages):
        m.reserve("a", 9)                              # needs 3 more, 1 is free
    assert m.num_free_pages() == 1 and m.table(0, "a") == [0, 1]
    assert not m.can_reserve("a", 9) and m.can_reserve("a", 4)
    with pytest.raises(CacheError):
        m.reserve("a", 100)                            # beyond max_seq
    with pytest.raises(CacheError):
        m.commit("a", 9)                               # more than was reserved
    m.check()


def test_double_free_and_unknown_requests_are_errors():
    m = manager()
    m.admit("a")
    m.reserve("a", 3)
    m.release("a")
    with pytest.raises(CacheError):
        m.release("a")
    with pytest.raises(CacheError):
        m.groups[0].pool.give_back(0)                             # a page that is not held
    for r in "abcd":
        m.admit(r)
    with pytest.raises(CacheError):
        m.admit("e")                                   # no slot left
    with pytest.raises(CacheError):
        m.admit("a")
    m.check()


def test_window_group_gives_pages_back_as_the_window_passes():
    m = manager(groups=((FULL, 1), (WIN, 1)), page_size=4, pages=20)
    m.admit("a")
    for _ in range(30):
        m.reserve("a", 1)
        m.commit("a", 1)
        m.check()
    full, win = m.table(0, "a"), m.table(1, "a")
    assert all(p >= 0 for p in full) and len(full) == 8
    # the next query is position 30: it reads keys 21..30, so pages 0..4 (keys 0..19) are gone
    assert [p >= 0 for p in win] == [False] * 5 + [True] * 3
    assert m.groups[1].pool.num_free == 20 - 3
    # a long portion needs all its pages at once, then gives most back
    m.admit("b")
    m.reserve("b", 33)
    assert len(m.table(1, "b")) == 9
    m.commit("b", 33)
    assert sum(p >= 0 for p in m.table(1, "b")) == 3      # keys 24..33 -> pages 6, 7, 8
    m.release("a")
    m.release("b")
    assert m.groups[0].pool.num_free == 20 and m.groups[1].pool.num_free == 20
    m.check()


def test_pages_of_rows_of_another_shape_are_a_group_of_their_own():
    """A part that keeps rows of its own per token (neither keys nor values) gets pages, block tables and the
    window rule like any other paged group, apart from groups of another need."""
    rows = PagedRowsNeed((24,), float32=True, window=6)
    m = manager(groups=((FULL, 1), (rows, 2), (PagedRowsNeed((24,), float32=True, window=6), 1), (PagedRowsNeed((24,)), 1)),
                page_size=4, pages=12)
    assert [type(g.need).__name__ for g in m.groups] == ["PagedKVNeed", "PagedRowsNeed", "PagedRowsNeed", "PagedRowsNeed"]
    assert m.groups[1].need == m.groups[2].need != m.groups[3].need
    m.admit("a")
    for _ in range(21):
        m.reserve("a", 1)
        m.commit("a", 1)
        m.check()
    assert sum(p >= 0 for p in m.table(0, "a")) == 6 and sum(p >= 0 for p in m.table(3, "a")) == 6
    # the next token is position 21 and reads rows 16..21: pages 0..3 are gone
    assert [p >= 0 for p in m.table(1, "a")] == [False] * 4 + [True] * 2
    assert m.groups[1].pool.num_free == 10
    m.release("a")
    assert all(g.pool.num_free == 12 for g in m.groups)
    m.check()


def test_state_slots_are_cleared_on_admission():
    m = manager(groups=((FULL, 1), (StateNeed((3, 5)), 2)), slots=2)
    s = m.admit("a")
    assert m.slots_to_clear == [s]
    m.forget_slots_to_clear()
    m.release("a")
    assert m.admit("b") == s and m.slots_to_clear == [s]      # the slot comes back and is cleared again
    assert [i for i, _ in m.state_groups()] == [1]


@pytest.mark.parametrize("seed", range(6))
def test_decode_steps_reserved_in_one_call_match_the_calls_per_request(seed):
    """`reserve_one_each` / `commit_one_each` leave the manager in the state that `reserve` and
    `commit` per request leave it in (tables, free pages, lengths), with a window group giving
    pages back, and take nothing when the pages do not suffice."""
    rng = random.Random(seed)
    a = manager(groups=((FULL, 2), (WIN, 1)), page_size=4, pages=30, slots=6, max_seq=80)
    b = manager(groups=((FULL, 2), (WIN, 1)), page_size=4, pages=30, slots=6, max_seq=80)
    live = []
    for n in range(5):
        k = rng.choice([1, 3, 4, 9, 17])
        for m in (a, b):
            m.admit(n)
            m.reserve(n, k)
            m.commit(n, k)
        live.append(n)
    for _ in range(70):
        some = [q for q in live if rng.random() < 0.7]
        if not some:
            continue
        if any(a.length(q) + 1 > 80 for q in some):
            with pytest.raises(CacheError):
                a.reserve_one_each(some)
            for q in [q for q in some if a.length(q) + 1 > 80]:
                a.release(q)
                b.release(q)
                live.remove(q)
            continue
        try:
            starts = a.reserve_one_each(some)
        except OutOfPages:
            free = a.num_free_pages()
            a.check()
            assert a.num_free_pages() == free
            q = rng.choice(live)                      # make room in both and go on
            a.release(q)
            b.release(q)
            live.remove(q)
            continue
        assert starts == [b.length(q) for q in some]
        for q in some:
            b.reserve(q, 1)
        a.commit_one_each(some)
        for q in some:
            b.commit(q, 1)
        a.check()
        b.check()
        for gi in (0, 1):
            for q in live:
                assert a.table(gi, q) == b.table(gi, q), (gi, q)
        assert a.num_free_pages() == b.num_free_pages()
    with pytest.raises(CacheError):
        a.reserve_one_each(["nobody"])


@pytest.mark.parametrize("seed", range(8))
def test_random_orders_lose_no_page(seed):
    """Admissions, portions, decoding, ends and failed reservations in random order:
    no page is lost, held twice or freed twice."""
    rng = random.Random(seed)
    m = manager(groups=((FULL, 2), (WIN, 1)), page_size=4, pages=20, slots=5, max_seq=60)
    live, n = [], 0
    for _ in range(600):
        op = rng.random()
        if op < 0.15 and m.num_free_slots():
            n += 1
            m.admit(n)
            live.append(n)
        elif op < 0.85 and live:
            r = rng.choice(live)
            k = rng.choice([1, 1, 1, 2, 5, 9])
            if m.length(r) + k > 60:
                m.release(r)
                live.remove(r)
            elif m.can_reserve(r, k):
                m.reserve(r, k)
                m.commit(r, k)
            else:
                free = m.num_free_pages()
                with pytest.raises(OutOfPages):
                    m.reserve(r, k)
                assert m.num_free_pages() == free
        elif live:
            r = rng.choice(live)
            m.release(r)
            live.remove(r)
        m.check()
    for r in live:
        m.release(r)
    m.check()
    assert all(g.pool.num_free == 20 for _, g in m.paged_groups())


# ------------------------------------------------------------------- scheduler
class Driver:
    """Runs plans against the real cache manager the way the engine does."""

    def __init__(self, sched, next_token=lambda req: 7):
        self.s, self.next_token = sched, next_token
        self.history = []

    def step(self):
        plan = self.s.plan()
        c = self.s.cache
        for e in plan.entries:
            if not c.has(e.request.key):
                c.admit(e.request.key)
            assert c.length(e.request.key) == e.start
            c.reserve(e.request.key, e.n_tokens)
        for e in plan.entries:
            c.commit(e.request.key, e.n_tokens)
        c.check()
        sampled = {e.request.number: self.next_token(e.request) for e in plan.entries if e.sample}
        for r in self.s.commit(plan, sampled):
            c.release(r.key)
        self.history.append(plan)
        return plan

    def run(self, limit=10000):
        while self.s.has_work():
            self.step()
            limit -= 1
            assert limit > 0, "the scheduler does not terminate"


def test_prompts_are_cut_under_the_budget_and_decodes_go_first():
    c = manager(pages=64, page_size=4, slots=4, max_seq=128)
    s = Scheduler(c, max_batched_tokens=16, chunk_size=7)
    a = s.add(list(range(5)), 6)
    b = s.add(list(range(17)), 6)
    d = Driver(s)
    p = d.step()
    assert [(e.request.number, e.start, e.n_tokens, e.sample) for e in p.entries] == \
        [(0, 0, 5, True), (1, 0, 7, False)]                 # a whole, b's first portion of 7
    p = d.step()
    assert [(e.request.number, e.start, e.n_tokens, e.sample) for e in p.entries] == \
        [(0, 5, 1, True), (1, 7, 7, False)]                 # a decodes beside b's next portion
    cc = s.add(list(range(33)), 6)
    p = d.step()                                            # a: 1, b: last 3, c: budget allows 7
    assert [(e.request.number, e.n_tokens, e.sample) for e in p.entries] == [(0, 1, True), (1, 3, True), (2, 7, False)]
    assert sum(e.n_tokens for e in p.entries) <= 16
    d.run()
    for r in (a, b, cc):
        assert r.finish_reason == "length" and len(r.generated) == 6
    assert all(sum(e.n_tokens for e in p.entries) <= 16 for p in d.history)
    assert not c.live_requests() and c.num_free_pages() == 64


def test_eos_ends_a_request_and_is_not_emitted():
    c = manager(pages=64, slots=2, max_seq=128)
    s = Scheduler(c)
    toks = iter([5, 6, 99, 1, 2])
    r = s.add([1, 2, 3], 10, eos_token_ids=(99,))
    Driver(s, lambda req: next(toks)).run()
    assert r.generated == [5, 6] and r.finish_reason == "eos"


def test_requests_that_can_never_run_are_refused():
    c = manager(pages=8, page_size=4, slots=2, max_seq=40)
    s = Scheduler(c)
    with pytest.raises(SchedulerError):
        s.add(list(range(35)), 10)                          # beyond max_seq
    with pytest.raises(SchedulerError):
        s.add(list(range(30)), 8)                           # 38 tokens = 10 pages > 8
    with pytest.raises(SchedulerError):
        s.add([], 3)
    s.add(list(range(20)), 12)                              # exactly 8 pages: accepted


def test_running_out_of_pages_preempts_the_youngest_and_recomputes():
    """12 pages of 4.  Two requests of 12 prompt tokens + 16 new each need 14 pages
    together at the end: the younger gives way, keeps its tokens, comes back."""
    c = manager(pages=12, page_size=4, slots=4, max_seq=48)
    s = Scheduler(c, max_batched_tokens=64, chunk_size=64)
    a = s.add(list(range(12)), 16)
    b = s.add(list(range(100, 112)), 16)
    d = Driver(s, lambda req: 1000 + req.number * 100 + len(req.generated))
    d.run()
    assert a.preemptions == 0 and b.preemptions >= 1        # the oldest is never preempted
    assert a.generated == [1000 + i for i in range(16)]
    assert b.generated == [1100 + i for i in range(16)]     # nothing lost, nothing drawn twice
    first = next(i for i, p in enumerate(d.history) if p.preempted)
    assert d.history[first].preempted == [b]
    assert all(e.request is not b for e in d.history[first].entries)
    # when b comes back it is fed from position 0 over its prompt and what it had generated
    back = next(p for p in d.history[first + 1:] if any(e.request is b for e in p.entries))
    e = next(e for e in back.entries if e.request is b)
    assert e.start == 0 and e.n_tokens > 12
    assert not c.live_requests() and c.num_free_pages() == 12


def test_a_pool_too_small_for_the_only_request_is_an_error():
    c = manager(pages=4, page_size=4, slots=2, max_seq=16)
    s = Scheduler(c, chunk_size=64, max_batched_tokens=64)
    s.add(list(range(10)), 6)                               # 16 tokens = 4 pages: fits exactly
    Driver(s).run()
    c2 = manager(groups=((FULL, 1),), pages=4, page_size=4, slots=2, max_seq=16)
    s2 = Scheduler(c2, chunk_size=64, max_batched_tokens=64)
    s2.add(list(range(8)), 4)
    c2.admit("squatter")
    c2.reserve("squatter", 12)                              # someone else holds 3 of the 4 pages
    with pytest.raises(SchedulerError):
        Driver(s2).run()


@pytest.mark.parametrize("seed", range(6))
def test_every_request_finishes_under_pressure(seed):
    rng = random.Random(seed)
    c = manager(groups=((FULL, 1), (WIN, 1)), pages=24, page_size=4, slots=3, max_seq=64)
    s = Scheduler(c, max_batched_tokens=rng.choice([8, 16, 40]), chunk_size=rng.choice([3, 7, 32]))
    reqs = [s.add([rng.randrange(50) for _ in range(rng.randrange(1, 30))], rng.randrange(1, 20)) for _ in range(12)]
    d = Driver(s, lambda req: req.number * 1000 + len(req.generated))
    d.run()
    for r in reqs:
        assert r.finish_reason == "length"
        assert r.generated == [r.number * 1000 + i for i in range(r.max_new_tokens)]
    assert not c.live_requests()
    for p in d.history:
        assert sum(e.n_tokens for e in p.entries) <= s.max_batched_tokens
        assert len(p.entries) <= 3


class AheadDriver(Driver):
    """The same with the step behind each step planned and run before that step's tokens are
    known, where the scheduler allows it: what `run_requests` does."""

    def __init__(self, sched, next_token=lambda req: 7):
        super().__init__(sched, next_token)
        self.ahead_steps = 0
        self.wasted_rows = 0

    def feed(self, plan):
        c = self.s.cache
        for e in plan.entries:
            if not c.has(e.request.key):
                c.admit(e.request.key)
            assert c.length(e.request.key) == e.start
            c.reserve(e.request.key, e.n_tokens)
        for e in plan.entries:
            c.commit(e.request.key, e.n_tokens)
        c.check()

    def run(self, limit=10000):
        c = self.s.cache
        flying = None
        while flying is not None or self.s.has_work():
            if flying is None:
                flying = self.s.plan()
                self.feed(flying)
            ahead = self.s.plan_ahead()
            if ahead.entries:
                self.feed(ahead)                      # launched before `flying`'s tokens are known
                self.ahead_steps += 1
            live = [e for e in flying.entries if not e.request.finish_reason]
            self.wasted_rows += len(flying.entries) - len(live)
            sampled = {e.request.number: self.next_token(e.request) for e in live if e.sample}
            for r in self.s.commit(flying, sampled):
                c.release(r.key)
            self.history.append(flying)
            flying = ahead if ahead.entries else None
            limit -= 1
            assert limit > 0, "the scheduler does not terminate"


def test_a_step_is_planned_ahead_only_when_it_cannot_depend_on_the_last():
    c = manager(pages=64, page_size=4, slots=4, max_seq=128)
    s = Scheduler(c, max_batched_tokens=16, chunk_size=7)
    a = s.add(list(range(5)), 4)
    b = s.add(list(range(9)), 6)
    d = AheadDriver(s)
    p = s.plan()                                     # a whole, b's first portion
    d.feed(p)
    assert s.plan_ahead().entries == []              # a portion of a prompt is in the step
    s.commit(p, {0: 7})
    p = s.plan()                                     # a decodes, b's last two tokens
    d.feed(p)
    assert s.plan_ahead().entries == []
    s.commit(p, {0: 7, 1: 7})
    p = s.plan()                                     # both decode: a has 2 of 4, b 1 of 6
    assert [(e.request.number, e.start, e.n_tokens) for e in p.entries] == [(0, 6, 1), (1, 9, 1)]
    d.feed(p)
    late = s.add([1, 2, 3], 2)
    assert s.plan_ahead().entries == []              # somebody waits: the next step may admit them
    s.abort(late)
    ahead = s.plan_ahead()
    assert [(e.request.number, e.start, e.n_tokens, e.sample) for e in ahead.entries] == [(0, 7, 1, True), (1, 10, 1, True)]
    d.feed(ahead)
    with pytest.raises(SchedulerError):
        s.plan()                                     # not while a step planned ahead waits
    s.commit(p, {0: 7, 1: 7})                        # a: 3 of 4, b: 2 of 6
    assert s.plan_ahead().entries == []              # the step in flight gives a its last token: it ends there
    assert s.commit(ahead, {0: 7, 1: 7}) == [a]
    assert a.generated == [7] * 4 and b.generated == [7] * 3 and b.n_fed == 11
    c.release(a.key)
    d.run()
    assert b.generated == [7] * 6 and not c.live_requests() and c.num_free_pages() == 64


def test_a_request_ended_by_the_last_step_is_dropped_from_the_step_planned_ahead():
    c = manager(pages=64, slots=2, max_seq=128)
    s = Scheduler(c)
    streams = {0: iter([5, 6, 99, 1, 2, 3, 4, 5, 6, 7]), 1: iter(range(100, 120))}
    r = s.add([1, 2, 3], 10, eos_token_ids=(99,))
    q = s.add([4, 5], 6, eos_token_ids=(99,))
    d = AheadDriver(s, lambda req: next(streams[req.number]))
    d.run()
    assert r.generated == [5, 6] and r.finish_reason == "eos"
    assert q.generated == list(range(100, 106)) and q.finish_reason == "length"
    assert d.ahead_steps >= 3 and d.wasted_rows == 1           # r ran one token behind its last
    assert not c.live_requests() and c.num_free_pages() == 64


def test_no_step_is_planned_ahead_without_pages_for_it():
    c = manager(groups=((FULL, 1),), pages=4, page_size=4, slots=2, max_seq=16)
    s = Scheduler(c, chunk_size=64, max_batched_tokens=64)
    a = s.add(list(range(6)), 10)
    d = AheadDriver(s)
    p = s.plan()
    d.feed(p)
    s.commit(p, {0: 7})
    p = s.plan()                                     # token 7 of 16: 2 pages held, 2 free
    d.feed(p)
    c.admit("squatter")
    c.reserve("squatter", 8)                         # takes the two free pages
    assert c.num_free_pages() == 0
    assert [e.start for e in s.plan_ahead().entries] == [7]     # position 7 lies in a page a holds
    s.commit(p, {0: 7})
    s.commit(None, {0: 7})
    p = s.plan_ahead()                               # position 8 needs a page
    assert p.entries == []
    c.release("squatter")


@pytest.mark.parametrize("seed", range(6))
def test_steps_planned_ahead_change_no_token(seed):
    rng = random.Random(seed)
    c = manager(groups=((FULL, 1), (WIN, 1)), pages=24, page_size=4, slots=3, max_seq=64)
    s = Scheduler(c, max_batched_tokens=rng.choice([8, 16, 40]), chunk_size=rng.choice([3, 7, 32]))
    eos = 999
    reqs = [s.add([rng.randrange(50) for _ in range(rng.randrange(1, 30))], rng.randrange(1, 20), eos_token_ids=(eos,))
            for _ in range(12)]
    stops = {r.number: rng.choice([None, rng.randrange(0, 12)]) for r in reqs}

    def token(req):
        return eos if stops[req.number] == len(req.generated) else req.number * 1000 + len(req.generated)

    d = AheadDriver(s, token)
    d.run()
    for r in reqs:
        n = r.max_new_tokens if stops[r.number] is None else min(r.max_new_tokens, stops[r.number])
        assert r.generated == [r.number * 1000 + i for i in range(n)]
        assert r.finish_reason == ("eos" if n < r.max_new_tokens else "length")
    assert not c.live_requests() and all(g.pool.num_free == 24 for _, g in c.paged_groups())
    assert d.ahead_steps > 0


def test_random_stream_is_keyed_by_seed_request_and_count():
    u = uniform(42, 3, 5)
    assert u == uniform(42, 3, 5) and 0.0 <= u < 1.0
    assert len({uniform(42, r, n) for r in range(20) for n in range(20)}) == 400
    assert uniform(43, 3, 5) != u
    xs = [uniform(1, r, n) for r in range(100) for n in range(100)]
    assert abs(sum(xs) / len(xs) - 0.5) < 0.01
    assert SamplingParams().effective_top_k() == 512 and SamplingParams(top_k=7).effective_top_k() == 7
