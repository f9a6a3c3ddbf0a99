"""The step function, named from Python.

`Engine.step(entries)` takes a batch of (request, its next tokens, the places
whose logits are wanted): portions of prompts beside single decoded tokens, cut
anywhere.  It runs exactly the tokens it is given as one flat batch against the
cache that earlier steps left, and returns the logits at the wanted places.  The
step, its cache and its graphs are the host library's (engine/engine.cpp, where
the reference's `Inference::forward` is cited); this class builds the model,
hands the batch across and gives the logits back as a torch tensor over the
engine's own memory.
"""
from __future__ import annotations

import ctypes
import json
from dataclasses import dataclass, field
from typing import Hashable, Optional, Sequence

from .. import native
from ..cache.manager import CacheManager
from ..models.model import Model
from ..native import EngineError  # noqa: F401
from ..ops.kernels import Ops, required_libraries
from ..weights.loader import DTYPES, load_weights


def token_from_feedback(row: int) -> int:
    """In place of a token id: the id that the sampler's last call with `feed=engine` wrote to row
    `row` of the engine's token feedback.  The step then needs no id that the host has not read yet,
    so it can be launched before the step before it has finished."""
    return -1 - int(row)


@dataclass
class StepEntry:
    """The next tokens of one request, and the places among them (0-based) whose
    logits are wanted."""
    request: Hashable
    tokens: Sequence[int]
    want: Sequence[int] = field(default_factory=tuple)


class Engine:
    def __init__(self, model: Model, dtype: str = "bfloat16", page_size: int = 16, max_tokens: Optional[int] = None,
                 num_pages: Optional[int] = None, max_requests: int = 64, max_seq: Optional[int] = None,
                 device: str = "cuda", max_step_graphs: Optional[int] = None, stream: Optional[int] = None):
        if dtype not in DTYPES:
            raise EngineError(f"dtype must be one of {sorted(DTYPES)}, got {dtype!r}")
        t = native.torch()
        if not t.cuda.is_available():
            raise EngineError("no GPU: this engine runs on an AMD GPU only (there is no CPU path)")
        native.use_torch_allocator()
        native.ensure_kernels(required_libraries(dtype))
        self.model = model
        self.dtype = dtype
        self.act_dtype = t.bfloat16 if dtype == "bfloat16" else t.float32
        self.device = t.device(device)
        options = {"dtype": dtype, "page_size": int(page_size), "max_requests": int(max_requests)}
        if max_tokens is not None:
            options["max_tokens"] = int(max_tokens)
        if num_pages is not None:
            options["num_pages"] = int(num_pages)
        if max_seq is not None:
            options["max_seq"] = int(max_seq)
        if max_step_graphs is not None:
            options["max_step_graphs"] = int(max_step_graphs)
        if stream is not None:
            options["stream"] = int(stream)          # a HIP stream's handle (torch: Stream.cuda_stream); default: the null stream
        self._ptr = native.pointer("ti_engine_create", model._ptr, json.dumps(options).encode())
        info = self.info()
        self.page_size, self.max_seq, self.num_pages = info["page_size"], info["max_seq"], info["num_pages"]
        self.table_width = info["table_width"]
        self.feedback_rows = info["feedback_rows"]     # 0: no token feedback (a model with parts from outside the library)
        self.cache = CacheManager(_borrowed=native.pointer("ti_engine_cache", self._ptr), _owner=self)
        self.ops = Ops(_borrowed=native.pointer("ti_engine_ops", self._ptr))

    def __del__(self):
        try:
            if native._lib is not None and getattr(self, "_ptr", None):
                native._lib.ti_engine_release(self._ptr)
        except Exception:  # noqa: BLE001
            pass

    # ------------------------------------------------------------- construction
    @classmethod
    def from_folder(cls, path: str, dtype: str = "bfloat16", **options) -> "Engine":
        """Read `path/config.json`, pick the model by its architecture name, load `path/*.safetensors`."""
        from ..config.base import read_config_json
        from ..registry import config_and_spec
        _, spec = config_and_spec(read_config_json(path))
        model = Model(spec)
        load_weights(model, path, dtype, options.get("device", "cuda"))
        return cls(model, dtype, **options)

    @classmethod
    def from_config(cls, config: dict, seed: int, dtype: str = "bfloat16", **options) -> "Engine":
        """Random weights for `config` (a config.json dict), drawn on the device."""
        from ..registry import config_and_spec
        if dtype not in DTYPES:
            raise EngineError(f"dtype must be one of {sorted(DTYPES)}, got {dtype!r}")
        native.use_torch_allocator()
        native.ensure_kernels(required_libraries(dtype))
        _, spec = config_and_spec(config)
        model = Model(spec)
        native.call("ti_model_load_random", model._ptr, int(seed), dtype.encode())
        model.dtype = dtype
        return cls(model, dtype, **options)

    # --------------------------------------------------------------------- step
    def info(self) -> dict:
        return json.loads(native.text("ti_engine_info", self._ptr))

    @property
    def steps_run(self) -> int:
        return self.info()["steps_run"]

    @property
    def num_graphs(self) -> int:
        return self.info()["num_graphs"]

    def graph_keys(self):
        """What the captured graphs are keyed by: a batch size (a decode step), or a step's shape as
        ((tokens, (wanted places)), ...) per entry."""
        keys = []
        for k in self.info()["graphs"]:
            if k.startswith("d"):
                keys.append(int(k[1:]))
            else:
                shape = []
                for entry in k[1:].split(";")[:-1]:
                    n, want = entry.split(":")
                    shape.append((int(n), tuple(int(w) for w in want.split(",")[:-1])))
                keys.append(tuple(shape))
        return keys

    def release(self, request: Hashable) -> None:
        """The request is over: its pages and its slot are given back."""
        self.cache.release(request)

    def _step(self, entries: Sequence[StepEntry], use_graph: bool):
        n = len(entries)
        key = self.cache.key
        reqs = (ctypes.c_int64 * max(1, n))(*[key(e.request) for e in entries])
        counts = (ctypes.c_int * max(1, n))(*[len(e.tokens) for e in entries])
        wants = (ctypes.c_int * max(1, n))(*[len(e.want) for e in entries])
        flat, want_flat = [], []
        for e in entries:
            flat.extend(e.tokens)
            want_flat.extend(e.want)
        try:
            tokens = (ctypes.c_int * max(1, len(flat)))(*flat)
            want = (ctypes.c_int * max(1, len(want_flat)))(*want_flat)
        except TypeError:
            raise EngineError("token ids and wanted places must be integers") from None
        out = native.ti_tensor()
        try:
            native.call("ti_engine_step", self._ptr, int(use_graph), n, reqs, counts, tokens, wants, want, ctypes.byref(out))
        finally:
            native.forget_contexts()
        return native.wrap(out)

    def step(self, entries: Sequence[StepEntry]):
        """Run one batch.  Returns float32 logits [wanted, vocab] in the order of the entries and of
        their `want` (None if nothing is wanted).  The tensor is engine workspace: it is valid until
        the next step."""
        return self._step(entries, False)

    def step_graph(self, entries: Sequence[StepEntry]):
        """`step`, replayed from a captured HIP graph where there is one: a batch of single tokens
        that each want their logits has a graph per batch size, any other step one per shape once the
        shape has come twice (see `Engine::step_graph`, engine/engine.cpp)."""
        return self._step(entries, True)

    def kv_pool(self, group: int, layer: int):
        """[pages, 2, kv heads, P, head_dim] of one cache layer."""
        out = native.ti_tensor()
        native.call("ti_engine_kv_pool", self._ptr, group, layer, ctypes.byref(out))
        t = native.wrap(out)
        return t.view(t.shape[0], 2, t.shape[1] // 2, t.shape[2], t.shape[3])

    def page_pool(self, group: int, layer: int):
        """The pages of one cache layer as the library lays them out ([pages, P, ...] for a `PagedRowsNeed`)."""
        out = native.ti_tensor()
        native.call("ti_engine_kv_pool", self._ptr, group, layer, ctypes.byref(out))
        return native.wrap(out)

    def state(self, group: int, layer: int):
        out = native.ti_tensor()
        native.call("ti_engine_state", self._ptr, group, layer, ctypes.byref(out))
        return native.wrap(out)

    def synchronize(self) -> None:
        native.call("ti_engine_synchronize", self._ptr)
