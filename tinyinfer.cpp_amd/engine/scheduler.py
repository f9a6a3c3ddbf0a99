"""The scheduler: which tokens of which requests the next step runs.

The reference has no scheduler: every prompt is prefilled whole in one batch and
then every unfinished sequence decodes one token per step, in a cache sized so
that nothing can run out (/root/reference/src/main.cpp:210-297).  Here requests
wait in a queue, are admitted while a request slot and pages for their first
portion are free, have their prompts cut into portions under a token budget,
decode beside the portions of others, and give everything back when they end.

Decisions, all taken in `plan()` from host bookkeeping only:
  * every running request feeds the tokens it has not fed yet: one token if it
    is decoding, else a portion of at most `chunk_size`; requests that decode go
    first (oldest first), then portions of running requests, then new admissions,
    until `max_batched_tokens` is used up;
  * a request's logits are wanted only at the last token it has, when the step
    feeds it (then its next token is sampled);
  * when the free pages cannot cover the step, the running request admitted last
    is preempted: its pages and slot go back, it keeps its tokens (prompt and
    what it generated) and goes to the front of the queue, to be fed again from
    position 0 later.  The oldest running request is never preempted; if it
    alone cannot be covered, that is an error;
  * a request whose prompt plus `max_new_tokens` exceeds `max_seq`, or needs more
    pages than the pool has, is refused when it is added.
The n-th token of a request is drawn from (seed, request number, n), so neither
batching nor preemption changes what is sampled.
"""
from __future__ import annotations

from collections import deque
from dataclasses import dataclass, field
from typing import Deque, Dict, List, Optional, Sequence, Tuple

from ..cache.manager import CacheManager
from ..sampling.sampler import SamplingParams


class SchedulerError(RuntimeError):
    pass


@dataclass
class Request:
    number: int                          # order of submission; keys the random stream
    prompt: List[int]
    max_new_tokens: int
    params: SamplingParams = field(default_factory=SamplingParams)
    eos_token_ids: Tuple[int, ...] = ()
    tokens: List[int] = field(default_factory=list)      # prompt + generated so far
    n_fed: int = 0                       # tokens whose keys and values are in the cache
    generated: List[int] = field(default_factory=list)
    finish_reason: Optional[str] = None  # "length", "eos", "abort"
    preemptions: int = 0
    admitted_at: int = -1                # admission counter; larger = admitted later

    @property
    def key(self):
        return ("req", self.number)

    @property
    def pending(self) -> int:
        return len(self.tokens) - self.n_fed


@dataclass
class PlannedEntry:
    request: Request
    start: int            # position of the first token fed
    n_tokens: int
    sample: bool          # the step feeds the request's last token: sample its next one


@dataclass
class Plan:
    entries: List[PlannedEntry]
    preempted: List[Request]


class Scheduler:
    def __init__(self, cache: CacheManager, max_batched_tokens: int = 2048, chunk_size: int = 512,
                 max_running: Optional[int] = None):
        if max_batched_tokens <= 0 or chunk_size <= 0:
            raise SchedulerError("max_batched_tokens and chunk_size must be positive")
        self.cache = cache
        self.max_batched_tokens = int(max_batched_tokens)
        self.chunk_size = int(chunk_size)
        self.max_running = min(cache.max_requests, max_running or cache.max_requests)
        self.waiting: Deque[Request] = deque()
        self.running: List[Request] = []
        self.finished: List[Request] = []
        self._submitted = 0
        self._admissions = 0

    # ------------------------------------------------------------------ adding
    def add(self, prompt: Sequence[int], max_new_tokens: int, params: Optional[SamplingParams] = None,
            eos_token_ids: Sequence[int] = ()) -> Request:
        """Queue a request.  One that can never run is refused here."""
        prompt = [int(t) for t in prompt]
        if not prompt:
            raise SchedulerError("a request needs at least one prompt token")
        if max_new_tokens < 1:
            raise SchedulerError("max_new_tokens must be at least 1")
        total = len(prompt) + max_new_tokens
        if total > self.cache.max_seq:
            raise SchedulerError(f"prompt ({len(prompt)}) + max_new_tokens ({max_new_tokens}) exceeds "
                                 f"max_seq = {self.cache.max_seq}")
        pages = -(-total // self.cache.page_size)
        for _, g in self.cache.paged_groups():
            if pages > g.pool.num_pages:
                raise SchedulerError(f"the request needs {pages} pages but the pool has {g.pool.num_pages}")
        req = Request(self._submitted, prompt, int(max_new_tokens), params or SamplingParams(),
                      tuple(int(e) for e in eos_token_ids), tokens=list(prompt))
        self._submitted += 1
        self.waiting.append(req)
        return req

    def has_work(self) -> bool:
        return bool(self.waiting or self.running)

    # ---------------------------------------------------------------- planning
    def _new_pages(self, batch: List[Tuple[Request, int]]) -> int:
        """Pages the tightest group lacks for `batch` = [(request, n_tokens)] (<= 0: it fits)."""
        short = -(1 << 30)
        for _, g in self.cache.paged_groups():
            need = 0
            for req, n in batch:
                admitted = self.cache.has(req.key)
                need += g.pages_to_cover(req.key if admitted else None, req.n_fed + n)
            short = max(short, need - g.pool.num_free)
        return short if self.cache.paged_groups() else 0

    def _preempt(self, req: Request, plan: Plan) -> None:
        self.running.remove(req)
        if self.cache.has(req.key):
            self.cache.release(req.key)
        req.n_fed = 0
        req.preemptions += 1
        self.waiting.appendleft(req)
        plan.preempted.append(req)

    def plan(self) -> Plan:
        plan = Plan([], [])
        # running requests: those that decode go first, oldest first within each kind.
        # If the free pages cannot cover them, the one admitted last gives way and
        # the step is planned again without it.
        while True:
            budget = self.max_batched_tokens
            batch: List[Tuple[Request, int]] = []
            for req in sorted(self.running, key=lambda r: (r.pending != 1, r.admitted_at)):
                if budget <= 0:
                    break
                n = min(req.pending, self.chunk_size, budget)
                batch.append((req, n))
                budget -= n
            if not batch or self._new_pages(batch) <= 0:
                break
            if len(self.running) == 1:
                req = self.running[0]
                raise SchedulerError(
                    f"request {req.number} cannot get pages for {batch[0][1]} more tokens although it is the "
                    "only one running: the cache pool is too small for it")
            self._preempt(max(self.running, key=lambda r: r.admitted_at), plan)

        # admissions: in queue order, while a slot and pages for the first portion are free
        while self.waiting and budget > 0 and len(self.running) < self.max_running:
            req = self.waiting[0]
            if any(req is p for p in plan.preempted):
                break                            # it has just given way: not in the same step
            new_in_batch = sum(1 for r, _ in batch if not self.cache.has(r.key))
            if self.cache.num_free_slots() - new_in_batch <= 0:
                break
            n = min(req.pending, self.chunk_size, budget)
            if self._new_pages(batch + [(req, n)]) > 0:
                break
            self.waiting.popleft()
            req.admitted_at = self._admissions
            self._admissions += 1
            self.running.append(req)
            batch.append((req, n))
            budget -= n
        for req, n in batch:
            plan.entries.append(PlannedEntry(req, req.n_fed, n, req.n_fed + n == len(req.tokens)))
        if not plan.entries and self.has_work():
            raise SchedulerError("nothing can run: the cache pool cannot take the next request's first portion")
        return plan

    # --------------------------------------------------------------- committing
    def commit(self, plan: Plan, sampled: Dict[int, int]) -> List[Request]:
        """The step ran.  `sampled[request.number]` is the token drawn for every
        entry that asked for one.  Returns the requests that finished; their
        pages and slots are to be given back by the caller (`on_finish`)."""
        done = []
        for e in plan.entries:
            req = e.request
            req.n_fed += e.n_tokens
            if not e.sample:
                continue
            tok = int(sampled[req.number])
            # the reference drops an end-of-generation token instead of emitting it
            # (/root/reference/src/main.cpp:255,287) and counts the first token from
            # the prefill step towards -n (main.cpp:258,284)
            if tok in req.eos_token_ids:
                req.finish_reason = "eos"
            else:
                req.generated.append(tok)
                req.tokens.append(tok)
                if len(req.generated) >= req.max_new_tokens:
                    req.finish_reason = "length"
            if req.finish_reason:
                done.append(req)
        for req in done:
            self.running.remove(req)
            self.finished.append(req)
        return done

    def abort(self, req: Request) -> None:
        if req in self.running:
            self.running.remove(req)
        elif req in self.waiting:
            self.waiting.remove(req)
        req.finish_reason = "abort"
        self.finished.append(req)
