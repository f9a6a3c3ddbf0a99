"""The Python entry point: load a model folder, generate token ids.

    import tinyinfer_amd
    llm = tinyinfer_amd.LLM("model_dir", dtype="bfloat16", max_seq=2048)
    outs = llm.generate([[1, 2, 3], [4, 5]], max_new_tokens=16, temperature=0.0)

`generate` drives the scheduler, the step function and the device sampler: the
loop of /root/reference/src/main.cpp:210-297 with admission, portions and
preemption added.  Options carry the reference's names and meanings
(`max_new_tokens` = -n, `temperature` = -t, `top_k`, `top_p`, `seed`, `max_seq`).
"""
from __future__ import annotations

import time
from dataclasses import dataclass, field
from typing import List, Optional, Sequence

from .engine.engine import Engine, StepEntry
from .engine.scheduler import Request, Scheduler
from .sampling.sampler import Sampler, SamplingParams


@dataclass
class GenerationStats:
    prefill_ms: float = 0.0          # steps that held a portion of a prompt
    prefill_tokens: int = 0
    decode_ms: float = 0.0           # steps of single tokens only
    decode_tokens: int = 0
    steps: int = 0
    preemptions: int = 0


def run_requests(engine: Engine, scheduler: Scheduler, sampler: Optional[Sampler] = None,
                 stats: Optional[GenerationStats] = None, on_token=None, use_graph: bool = False) -> None:
    """Run until the scheduler has no work.  `on_token(request, token)` is called
    for every generated token."""
    import torch
    sampler = sampler or Sampler(engine.ops, engine.device)
    stats = stats if stats is not None else GenerationStats()
    while scheduler.has_work():
        plan = scheduler.plan()
        stats.preemptions += len(plan.preempted)
        entries = [StepEntry(e.request.key, e.request.tokens[e.start:e.start + e.n_tokens],
                             (e.n_tokens - 1,) if e.sample else ()) for e in plan.entries]
        decode_only = all(e.n_tokens == 1 for e in plan.entries)
        t0 = time.perf_counter()
        if use_graph:
            logits = engine.step_graph(entries)
        else:
            logits = engine.step(entries)
        sampled = {}
        asked = [e.request for e in plan.entries if e.sample]
        if asked:
            toks = sampler.sample(logits, [r.params for r in asked], [r.number for r in asked],
                                  [len(r.generated) for r in asked])
            sampled = {r.number: t for r, t in zip(asked, toks)}
        else:
            torch.cuda.synchronize()
        dt = (time.perf_counter() - t0) * 1e3
        n_tok = sum(e.n_tokens for e in plan.entries)
        if decode_only:
            stats.decode_ms += dt
            stats.decode_tokens += n_tok
        else:
            stats.prefill_ms += dt
            stats.prefill_tokens += n_tok
        stats.steps += 1
        before = {r.number: len(r.generated) for r in asked}
        for req in scheduler.commit(plan, sampled):
            engine.release(req.key)
        if on_token:
            for r in asked:
                if len(r.generated) > before[r.number]:
                    on_token(r, r.generated[-1])


def generate_ids(engine: Engine, prompts: Sequence[Sequence[int]], max_new_tokens: int = 128,
                 temperature: float = 0.0, top_k: int = 0, top_p: float = 1.0, seed: int = 42,
                 eos_token_ids: Optional[Sequence[int]] = None, chunk_size: int = 512,
                 max_batched_tokens: int = 2048, use_graph: bool = False,
                 stats: Optional[GenerationStats] = None) -> List[List[int]]:
    """Generated token ids for each prompt (the prompt itself is not repeated)."""
    if eos_token_ids is None:
        eos_token_ids = engine.model.spec.eos_token_ids
    scheduler = Scheduler(engine.cache, max_batched_tokens=max_batched_tokens, chunk_size=chunk_size)
    params = SamplingParams(float(temperature), int(top_k), float(top_p), int(seed))
    requests: List[Request] = [scheduler.add(p, max_new_tokens, params, eos_token_ids) for p in prompts]
    run_requests(engine, scheduler, stats=stats, use_graph=use_graph)
    return [list(r.generated) for r in requests]


class LLM:
    """A model folder made ready for generation."""

    def __init__(self, model_dir: str, dtype: str = "bfloat16", max_seq: int = 2048, max_requests: int = 16,
                 page_size: int = 16, max_tokens: Optional[int] = None, chunk_size: int = 512,
                 max_batched_tokens: int = 2048, use_graph: bool = False):
        if max_tokens is None:
            max_tokens = max_seq * max_requests
        self.engine = Engine.from_folder(model_dir, dtype, page_size=page_size, max_tokens=max_tokens,
                                         max_requests=max_requests, max_seq=max_seq)
        self.chunk_size = chunk_size
        self.max_batched_tokens = max_batched_tokens
        self.use_graph = use_graph
        self.last_stats = GenerationStats()

    def generate(self, prompts: Sequence[Sequence[int]], max_new_tokens: int = 128, temperature: float = 0.0,
                 top_k: int = 0, top_p: float = 1.0, seed: int = 42,
                 eos_token_ids: Optional[Sequence[int]] = None) -> List[List[int]]:
        self.last_stats = GenerationStats()
        return generate_ids(self.engine, prompts, max_new_tokens, temperature, top_k, top_p, seed, eos_token_ids,
                            self.chunk_size, self.max_batched_tokens, self.use_graph, self.last_stats)
