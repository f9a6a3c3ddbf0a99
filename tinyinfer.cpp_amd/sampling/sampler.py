"""Sampling parameters, the counter-based random stream, and the device sampler,
named from Python (sampling/sampler.cpp has them, and what the reference does:
/root/reference/src/main.cpp:23-84).
"""
from __future__ import annotations

import ctypes
from dataclasses import dataclass
from typing import List, Sequence

from .. import native

DEFAULT_TOP_K = 512          # the reference's cut when --top-k is 0: src/main.cpp:47-48


@dataclass(frozen=True)
class SamplingParams:
    temperature: float = 0.0     # <= 0: greedy (src/main.cpp:24,31-38)
    top_k: int = 0               # 0: the reference's default of 512
    top_p: float = 1.0
    seed: int = 42               # src/main.cpp:27

    def effective_top_k(self) -> int:
        return self.top_k if self.top_k > 0 else DEFAULT_TOP_K


def uniform(seed: int, request: int, n_generated: int) -> float:
    """A number in [0, 1) with 24 random bits (exact in float32), a pure function of its three keys."""
    mask = (1 << 64) - 1
    return float(native.lib().ti_uniform(seed & mask, request & mask, n_generated & mask))


class Sampler:
    """Draws one token per row of logits on the device."""

    def __init__(self, ops, device=None):
        self.ops = ops
        self._ptr = native.pointer("ti_sampler_create", ops._ptr)

    def __del__(self):
        try:
            if native._lib is not None:
                native._lib.ti_sampler_release(self._ptr)
        except Exception:  # noqa: BLE001
            pass

    @staticmethod
    def _arguments(n, params, requests, counters):
        mask = (1 << 64) - 1
        return ((ctypes.c_float * n)(*[p.temperature for p in params]), (ctypes.c_int * n)(*[p.top_k for p in params]),
                (ctypes.c_float * n)(*[p.top_p for p in params]), (ctypes.c_uint64 * n)(*[p.seed & mask for p in params]),
                (ctypes.c_int64 * n)(*requests), (ctypes.c_int64 * n)(*counters))

    def sample(self, logits, params: Sequence[SamplingParams], requests: Sequence[int], counters: Sequence[int]) -> List[int]:
        """logits f32 [n, V]; row i belongs to request number `requests[i]`, which has generated
        `counters[i]` tokens so far."""
        n = logits.shape[0]
        native.ensure_kernels(["sampling"])
        out = (ctypes.c_int * n)()
        native.call("ti_sampler_sample", self._ptr, native.describe_many([logits]), n,
                    *self._arguments(n, params, requests, counters), out)
        return list(out)

    def sample_async(self, logits, params: Sequence[SamplingParams], requests: Sequence[int], counters: Sequence[int],
                     feed=None):
        """The same without waiting: returns a ticket for `collect`.  `feed`: an engine whose token
        feedback receives the ids too, so that its next step can name them with
        `token_from_feedback(row)` before they are read.  At most two calls may be under way."""
        n = logits.shape[0]
        native.ensure_kernels(["sampling"])
        ticket = ctypes.c_uint64()
        native.call("ti_sampler_sample_async", self._ptr, native.describe_many([logits]), n,
                    *self._arguments(n, params, requests, counters), feed._ptr if feed is not None else None,
                    ctypes.byref(ticket))
        return (ticket.value, n)

    def collect(self, ticket) -> List[int]:
        """Wait for the ids of a `sample_async` call."""
        number, n = ticket
        out = (ctypes.c_int * n)()
        native.call("ti_sampler_collect", self._ptr, number, n, out)
        return list(out)
