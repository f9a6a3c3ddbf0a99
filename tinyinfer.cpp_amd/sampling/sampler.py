"""Sampling parameters, the counter-based random stream, and the device sampler.

The reference samples on the host: greedy argmax when the temperature is 0, else
the K largest logits (K = --top-k, or 512 when that is 0), weights exp(l/T - max),
an optional top-p cut, and one draw from a process-wide mt19937 shared by all
sequences in turn (/root/reference/src/main.cpp:23-84).  Here the same options
run on the device (`csrc/sampling.hip`), and the random stream is keyed by
(seed, request number, index of the generated token): what a request draws does
not depend on which other requests share its steps, nor on being preempted.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import List, Sequence

import torch

DEFAULT_TOP_K = 512          # the reference's cut when --top-k is 0: src/main.cpp:47-48


@dataclass(frozen=True)
class SamplingParams:
    temperature: float = 0.0     # <= 0: greedy (src/main.cpp:24,31-38)
    top_k: int = 0               # 0: the reference's default of 512
    top_p: float = 1.0
    seed: int = 42               # src/main.cpp:27

    def effective_top_k(self) -> int:
        return self.top_k if self.top_k > 0 else DEFAULT_TOP_K


_MASK = (1 << 64) - 1


def _mix(z: int) -> int:
    """splitmix64's output function."""
    z = (z + 0x9E3779B97F4A7C15) & _MASK
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & _MASK
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & _MASK
    return z ^ (z >> 31)


def uniform(seed: int, request: int, n_generated: int) -> float:
    """A number in [0, 1) with 24 random bits (exact in float32), a pure function
    of its three keys."""
    z = _mix(seed & _MASK)
    z = _mix(z ^ (request & _MASK))
    z = _mix(z ^ (n_generated & _MASK))
    return (z >> 40) / float(1 << 24)


class Sampler:
    """Draws one token per row of logits on the device."""

    def __init__(self, ops, device):
        self.ops = ops
        self.device = device
        self._cap = 0

    def _buffers(self, n: int):
        if n > self._cap:
            cap = max(64, 2 * n)
            self._f_host = torch.empty(3 * cap, dtype=torch.float32, pin_memory=True)
            self._i_host = torch.empty(cap, dtype=torch.int32, pin_memory=True)
            self._f_dev = torch.empty(3 * cap, dtype=torch.float32, device=self.device)
            self._i_dev = torch.empty(cap, dtype=torch.int32, device=self.device)
            self._out = torch.empty(cap, dtype=torch.int32, device=self.device)
            self._cap = cap

    def sample(self, logits: torch.Tensor, params: Sequence[SamplingParams], requests: Sequence[int],
               counters: Sequence[int]) -> List[int]:
        """logits f32 [n, V]; row i belongs to request number `requests[i]`, which
        has generated `counters[i]` tokens so far."""
        n = logits.shape[0]
        self._buffers(n)
        out = self._out[:n]
        if all(p.temperature <= 0.0 for p in params):
            self.ops.argmax(logits, out)
            return out.tolist()
        cap = self._cap
        fh, ih = self._f_host, self._i_host
        for i, (p, r, c) in enumerate(zip(params, requests, counters)):
            fh[i] = p.temperature
            fh[cap + i] = p.top_p
            fh[2 * cap + i] = uniform(p.seed, r, c)
            ih[i] = p.effective_top_k()
        # the previous call ended with a read-back of its result, so the earlier copies out of
        # the pinned buffers have finished
        self._f_dev.copy_(fh, non_blocking=True)
        self._i_dev.copy_(ih, non_blocking=True)
        fd = self._f_dev
        self.ops.sample(logits, fd[:n], self._i_dev[:n], fd[cap:cap + n], fd[2 * cap:2 * cap + n], out)
        return out.tolist()
