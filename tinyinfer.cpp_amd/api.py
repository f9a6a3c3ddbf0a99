"""The Python entry point: load a model folder, generate token ids.

    import tinyinfer_amd
    llm = tinyinfer_amd.LLM("model_dir", dtype="bfloat16", max_seq=2048)
    outs = llm.generate([[1, 2, 3], [4, 5]], max_new_tokens=16, temperature=0.0)

`generate` drives the scheduler, the step function and the device sampler: the
loop of /root/reference/src/main.cpp:210-297 with admission, portions and
preemption added (`run_requests`, engine/scheduler.cpp).  Options carry the
reference's names and meanings (`max_new_tokens` = -n, `temperature` = -t,
`top_k`, `top_p`, `seed`, `max_seq`).
"""
from __future__ import annotations

import json
from dataclasses import dataclass
from typing import List, Optional, Sequence

from . import native
from .engine.engine import Engine
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
    steps_ahead: int = 0             # of `steps`: launched before the ids of the step before were read


def run_requests(engine: Engine, scheduler: Scheduler, sampler: Optional[Sampler] = None,
                 stats: Optional[GenerationStats] = None, on_token=None, use_graph: bool = False,
                 run_ahead: bool = True, on_prompt_logits=None) -> None:
    """Run until the scheduler has no work.  `on_token(request, token)` is called for every
    generated token.  When a step fails, every request the scheduler still holds is given back
    to the cache before the error is raised.  `run_ahead`: while every running request decodes
    and nobody waits, the next step is launched before the last one's ids are read (it takes
    them from the device); the tokens are the same, `on_token` hears them a step later.
    `on_prompt_logits(request, logits)`: called with the 32-bit logits (a numpy array) behind the last token of
    each request's prompt, before its first token is drawn."""
    native.ensure_kernels(["sampling"])
    raised = []

    def relay(number, token):
        try:
            on_token(scheduler._requests[number], token)
            return 0
        except BaseException as e:  # noqa: BLE001  (it must not unwind through the library: the run is stopped there)
            raised.append(e)
            return 1

    def relay_logits(number, row, vocab):
        try:
            import numpy as np
            on_prompt_logits(scheduler._requests[number], np.ctypeslib.as_array(row, shape=(vocab,)).copy())
            return 0
        except BaseException as e:  # noqa: BLE001
            raised.append(e)
            return 1

    callback = native.ON_TOKEN(relay) if on_token else ctypes_null(native.ON_TOKEN)
    logits_callback = native.ON_LOGITS(relay_logits) if on_prompt_logits else ctypes_null(native.ON_LOGITS)
    try:
        out = native.text("ti_run_requests", engine._ptr, scheduler._ptr, sampler._ptr if sampler else None,
                          int(use_graph), int(run_ahead), callback, logits_callback)
    except native.EngineError:
        if raised:
            raise raised[0] from None
        raise
    finally:
        native.forget_contexts()
    if stats is not None:
        d = json.loads(out)
        stats.prefill_ms += d["prefill_ms"]
        stats.prefill_tokens += d["prefill_tokens"]
        stats.decode_ms += d["decode_ms"]
        stats.decode_tokens += d["decode_tokens"]
        stats.steps += d["steps"]
        stats.preemptions += d["preemptions"]
        stats.steps_ahead += d["steps_ahead"]


def ctypes_null(kind):
    import ctypes
    return ctypes.cast(None, kind)


def generate_ids(engine: Engine, prompts: Sequence[Sequence[int]], max_new_tokens: int = 128,
                 temperature: float = 0.0, top_k: int = 0, top_p: float = 1.0, seed: int = 42,
                 eos_token_ids: Optional[Sequence[int]] = None, chunk_size: int = 512,
                 max_batched_tokens: int = 2048, use_graph: bool = False,
                 stats: Optional[GenerationStats] = None, run_ahead: bool = True, on_prompt_logits=None) -> List[List[int]]:
    """Generated token ids for each prompt (the prompt itself is not repeated)."""
    if eos_token_ids is None:
        eos_token_ids = engine.model.spec.eos_token_ids
    scheduler = Scheduler(engine.cache, max_batched_tokens=max_batched_tokens, chunk_size=chunk_size)
    params = SamplingParams(float(temperature), int(top_k), float(top_p), int(seed))
    requests: List[Request] = [scheduler.add(p, max_new_tokens, params, eos_token_ids) for p in prompts]
    relay = None
    if on_prompt_logits:
        index = {}          # request number -> index of its prompt
        relay = lambda request, logits: on_prompt_logits(index[request.number], logits)     # noqa: E731
    for i, r in enumerate(requests):
        if relay:
            index[r.number] = i
    run_requests(engine, scheduler, stats=stats, use_graph=use_graph, run_ahead=run_ahead, on_prompt_logits=relay)
    return [list(r.generated) for r in requests]


class LLM:
    """A model folder made ready for generation (or, with `random_seed`, a config.json alone with
    random weights drawn on the device)."""

    def __init__(self, model_dir: str, dtype: str = "bfloat16", max_seq: int = 2048, max_requests: int = 16,
                 page_size: int = 16, max_tokens: Optional[int] = None, chunk_size: int = 512,
                 max_batched_tokens: int = 2048, use_graph: bool = False, num_pages: Optional[int] = None,
                 random_seed: Optional[int] = None):
        if max_tokens is None and num_pages is None:
            max_tokens = max_seq * max_requests
        options = dict(page_size=page_size, max_tokens=max_tokens, num_pages=num_pages, max_requests=max_requests,
                       max_seq=max_seq)
        if random_seed is None:
            self.engine = Engine.from_folder(model_dir, dtype, **options)
        else:
            from .config.base import read_config_json
            self.engine = Engine.from_config(read_config_json(model_dir), random_seed, dtype, **options)
        self.chunk_size = chunk_size
        self.max_batched_tokens = max_batched_tokens
        self.use_graph = use_graph
        self.last_stats = GenerationStats()

    def generate(self, prompts: Sequence[Sequence[int]], max_new_tokens: int = 128, temperature: float = 0.0,
                 top_k: int = 0, top_p: float = 1.0, seed: int = 42,
                 eos_token_ids: Optional[Sequence[int]] = None, on_prompt_logits=None) -> List[List[int]]:
        """`on_prompt_logits(i, logits)`: the 32-bit logits behind the last token of prompt i, before its first token is drawn."""
        self.last_stats = GenerationStats()
        return generate_ids(self.engine, prompts, max_new_tokens, temperature, top_k, top_p, seed, eos_token_ids,
                            self.chunk_size, self.max_batched_tokens, self.use_graph, self.last_stats,
                            on_prompt_logits=on_prompt_logits)
