"""The scheduler, named from Python: which tokens of which requests the next step
runs.  The decisions are the host library's (engine/scheduler.cpp, where the
policy is described: admission, portions under a token budget, decodes first,
preempt the youngest and recompute when pages run out); this class shows its
state.
"""
from __future__ import annotations

import ctypes
import json
from dataclasses import dataclass
from typing import Dict, List, Optional, Sequence

from .. import native
from ..cache.manager import CacheManager
from ..native import SchedulerError  # noqa: F401
from ..sampling.sampler import SamplingParams


class Request:
    """A request of the library's scheduler; its fields are read from there."""

    def __init__(self, scheduler: "Scheduler", number: int, params: SamplingParams):
        self._scheduler = scheduler
        self.number = number
        self.params = params

    def _field(self, name):
        return json.loads(native.text("ti_scheduler_request", self._scheduler._ptr, self.number))[name]

    key = property(lambda self: ("req#", self._field("key")))
    prompt = property(lambda self: self._field("prompt"))
    max_new_tokens = property(lambda self: self._field("max_new_tokens"))
    tokens = property(lambda self: self._field("tokens"))
    generated = property(lambda self: self._field("generated"))
    n_fed = property(lambda self: self._field("n_fed"))
    finish_reason = property(lambda self: self._field("finish_reason"))
    preemptions = property(lambda self: self._field("preemptions"))
    admitted_at = property(lambda self: self._field("admitted_at"))
    eos_token_ids = property(lambda self: tuple(self._field("eos_token_ids")))

    @property
    def pending(self) -> int:
        d = json.loads(native.text("ti_scheduler_request", self._scheduler._ptr, self.number))
        return len(d["tokens"]) - d["n_fed"]

    def __repr__(self):
        return f"Request({self.number})"


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
        self.cache = cache
        self._ptr = native.pointer("ti_scheduler_create", cache._ptr, int(max_batched_tokens), int(chunk_size),
                                   int(max_running or 0))
        self.max_batched_tokens, self.chunk_size = int(max_batched_tokens), int(chunk_size)
        self._requests: Dict[int, Request] = {}

    def __del__(self):
        try:
            if native._lib is not None:
                native._lib.ti_scheduler_release(self._ptr)
        except Exception:  # noqa: BLE001
            pass

    def add(self, prompt: Sequence[int], max_new_tokens: int, params: Optional[SamplingParams] = None,
            eos_token_ids: Sequence[int] = ()) -> Request:
        """Queue a request.  One that can never run is refused here."""
        params = params or SamplingParams()
        prompt = [int(t) for t in prompt]
        eos = [int(e) for e in eos_token_ids]
        number = ctypes.c_int64()
        native.call("ti_scheduler_add", self._ptr, len(prompt), (ctypes.c_int * max(1, len(prompt)))(*prompt),
                    int(max_new_tokens), float(params.temperature), int(params.top_k), float(params.top_p),
                    int(params.seed) & ((1 << 64) - 1), len(eos), (ctypes.c_int * max(1, len(eos)))(*eos),
                    ctypes.byref(number))
        req = self._requests[number.value] = Request(self, number.value, params)
        return req

    def set_next_number(self, number: int) -> None:
        """The number the next request gets (it keys the request's random stream)."""
        native.call("ti_scheduler_set_next_number", self._ptr, int(number))

    def _state(self) -> dict:
        return json.loads(native.text("ti_scheduler_state", self._ptr))

    waiting = property(lambda self: [self._requests[n] for n in self._state()["waiting"]])
    running = property(lambda self: [self._requests[n] for n in self._state()["running"]])
    finished = property(lambda self: [self._requests[n] for n in self._state()["finished"]])

    def has_work(self) -> bool:
        s = self._state()
        return bool(s["waiting"] or s["running"])

    def plan(self) -> Plan:
        d = json.loads(native.text("ti_scheduler_plan", self._ptr))
        return Plan([PlannedEntry(self._requests[e["number"]], e["start"], e["n_tokens"], e["sample"]) for e in d["entries"]],
                    [self._requests[n] for n in d["preempted"]])

    def plan_ahead(self) -> Plan:
        """The step behind the last `plan()` (or `plan_ahead()`), before that one is committed: one
        more token of every running request, if all of them decode, nobody waits, none ends with the
        last step's token by its length and the pages are free; else an empty plan.  The next
        `commit` is for the earlier plan, the one after it for this one (without the requests that
        the earlier one ended)."""
        d = json.loads(native.text("ti_scheduler_plan_ahead", self._ptr))
        return Plan([PlannedEntry(self._requests[e["number"]], e["start"], e["n_tokens"], e["sample"]) for e in d["entries"]],
                    [])

    def commit(self, plan: Plan, sampled: Dict[int, int]) -> List[Request]:
        """The step of the last `plan()` ran.  `sampled[request.number]` is the token drawn for every
        entry that asked for one.  Returns the requests that finished; their pages and slots are to be
        given back by the caller."""
        numbers = list(sampled)
        n = len(numbers)
        done = json.loads(native.text("ti_scheduler_commit", self._ptr, n, (ctypes.c_int64 * max(1, n))(*numbers),
                                      (ctypes.c_int * max(1, n))(*[int(sampled[k]) for k in numbers])))
        return [self._requests[k] for k in done]

    def abort(self, req: Request) -> None:
        """Take the request out, wherever it is; its pages and slot go back."""
        native.call("ti_scheduler_abort", self._ptr, req.number)
