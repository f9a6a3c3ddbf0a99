"""The step function.

`Engine.step(entries)` takes a batch of (request, its next tokens, the places
whose logits are wanted): portions of prompts beside single decoded tokens, cut
anywhere.  It reserves pages, runs exactly the tokens it is given as one flat
batch against the cache that earlier steps left, and returns the logits at the
wanted places.  The reference's `Inference::forward` has the same shape (flat
tokens with a position and a sequence id each, logits for chosen rows:
/root/reference/src/inference.h:26-42, src/inference.cu:178-265) over a
non-paged cache; its kernel sequence is src/inference.cu:28-72.

Per-step metadata (tokens, positions, block-table rows, output rows, work
lists) is packed into one pinned host buffer and reaches the device in one copy.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, Hashable, List, Optional, Sequence, Tuple

import numpy as np
import torch

from ..cache import CacheError, CacheManager, CacheStorage, OutOfPages, PagedGroup
from ..models.model import Model
from ..ops.kernels import get_ops
from ..weights.loader import DTYPES

PREFILL_TILE_Q = 128    # query rows per work item of the tiled attention kernels
PREFILL_TILE_SMALL = 64  # and of the kernel that pairs a tile of many keys with one of few
STEP_GRAPH_AFTER = 2              # a step's shape is captured when it comes for this many times ...
MAX_STEP_GRAPHS = 32              # ... and this many such graphs are kept
PAGE_SCATTER_WINDOW = 512  # free pages are first handed out shuffled within windows of this many (see PagePool)


class EngineError(RuntimeError):
    pass


@dataclass
class StepEntry:
    """The next tokens of one request, and the places among them (0-based) whose
    logits are wanted."""
    request: Hashable
    tokens: Sequence[int]
    want: Sequence[int] = field(default_factory=tuple)


class CacheView:
    """What a mixer sees of one paged group in this step: the block-table rows of
    the step's entries, `table[entry][page index] -> page id`."""

    def __init__(self, table: torch.Tensor, page_size: int):
        self.table = table
        self.page_size = page_size


class StepContext:
    """Everything a part may touch during one step."""

    def __init__(self, engine: "Engine"):
        self.engine = engine
        self.ops = engine.ops
        self.act_dtype = engine.act_dtype
        self.f32 = torch.float32
        self.dtype = engine.dtype
        self.device = engine.device
        self.M = 0
        self.tokens = self.positions = self.slots = None     # int32 [M]
        self.out_rows = None                                  # int32 [N]
        # per entry: (row0, n_tokens, start_pos, state_slot); the same as int32 [R, 4] on the device
        self.entries: List[Tuple[int, int, int, int]] = []
        self.entry_meta = None
        self.tiles = None                 # int32 [n_tiles, 2]: (entry, first row) of each query tile
        self.n_tiles = 0
        self._decode_fast = False         # the step was reserved by CacheManager.reserve_one_each
        self.tiles_small = None           # the same in tiles of PREFILL_TILE_SMALL rows, from the tile whose
        self.n_tiles_small = 0            # last row sees the most keys to the one that sees the fewest
        self.decode_only = False
        self.decode_rows = None           # int32: rows of single-token entries (None if decode_only)
        self.n_decode_rows = 0
        self.max_context = 0              # longest context (tokens) any row reads in this step
        self.portion_context = 0          # the same over the rows of portions (entries of several tokens) only
        self.split_context = 0            # the context length the decode kernel's split count is sized for
        self.run = 0                      # index into the model's run order
        self._views: Dict[int, CacheView] = {}

    def buf(self, name: str, shape, dtype) -> torch.Tensor:
        return self.engine._workspace(name, shape, dtype)

    def binding(self, part) -> Tuple[int, int]:
        return self.engine.model.bindings[self.run][id(part)]

    def kv_pool(self, group: int, layer: int) -> torch.Tensor:
        return self.engine.storage.kv[group][layer]

    def cache_view(self, group: int) -> CacheView:
        return self._views[group]

    def state(self, group: int, layer: int) -> torch.Tensor:
        """[slots, ...] float32 state of one cache layer; index with an entry's state slot."""
        return self.engine.storage.state[group][layer]


class Engine:
    def __init__(self, model: Model, dtype: str = "bfloat16", page_size: int = 16,
                 max_tokens: Optional[int] = None, num_pages: Optional[int] = None,
                 max_requests: int = 64, max_seq: Optional[int] = None, device: str = "cuda"):
        if dtype not in DTYPES:
            raise EngineError(f"dtype must be one of {sorted(DTYPES)}, got {dtype!r}")
        if not torch.cuda.is_available():
            raise EngineError("no GPU: this engine runs on an AMD GPU only (there is no CPU path)")
        self.model = model
        self.dtype = dtype
        self.act_dtype = DTYPES[dtype]
        self.device = torch.device(device)
        self.ops = get_ops()
        self.page_size = int(page_size)
        if num_pages is None:
            if max_tokens is None:
                raise EngineError("give the cache pool a size: max_tokens or num_pages")
            num_pages = -(-int(max_tokens) // self.page_size)
        self.num_pages = int(num_pages)
        if max_seq is None:
            max_seq = self.num_pages * self.page_size
            if model.spec.max_position_embeddings:
                max_seq = min(max_seq, model.spec.max_position_embeddings)
        self.max_seq = int(max_seq)
        self.cache = CacheManager(model.cache_groups, self.page_size, self.num_pages, max_requests, self.max_seq,
                                  scatter_window=PAGE_SCATTER_WINDOW)
        self.storage = CacheStorage(self.cache, self.act_dtype, self.device)
        self.table_width = self.cache.max_pages_per_request
        for part in model.parts():
            if hasattr(part, "prepare"):
                part.prepare(self.ops, self.max_seq)      # tables that depend on the longest sequence
        self._ws: Dict[tuple, object] = {}        # (name, dtype) -> tensor; (name, shape, dtype) -> (tensor, view)
        self._meta_dev = None
        self._meta_host: List[torch.Tensor] = []
        self._meta_events: List[Optional[torch.cuda.Event]] = []
        self._meta_turn = 0
        self.steps_run = 0
        self._graphs: Dict[object, "_DecodeGraph"] = {}       # batch size, or a step's shape -> its graph
        self._shapes_seen: Dict[tuple, int] = {}

    # ------------------------------------------------------------- construction
    @classmethod
    def from_folder(cls, path: str, dtype: str = "bfloat16", **options) -> "Engine":
        """Read `path/config.json`, pick the model by its architecture name, load
        `path/*.safetensors`."""
        from ..config.base import read_config_json
        from ..registry import config_and_spec
        from ..weights.loader import load_weights
        get_ops().preload(required_libraries(dtype))
        _, spec = config_and_spec(read_config_json(path))
        model = Model(spec)
        load_weights(model, path, dtype, options.get("device", "cuda"))
        return cls(model, dtype, **options)

    @classmethod
    def from_config(cls, config: dict, seed: int, dtype: str = "bfloat16", **options) -> "Engine":
        """Random weights for `config` (a config.json dict), drawn on the device."""
        from ..registry import config_and_spec
        from ..weights.loader import load_weights
        from ..weights.random_init import random_tensors
        get_ops().preload(required_libraries(dtype))
        _, spec = config_and_spec(config)
        model = Model(spec)
        device = options.get("device", "cuda")
        tensors = random_tensors(model, seed, DTYPES[dtype], device=device)
        load_weights(model, tensors, dtype, device)
        return cls(model, dtype, **options)

    # ---------------------------------------------------------------- workspace
    def _workspace(self, name: str, shape, dtype) -> torch.Tensor:
        """A named scratch tensor of this shape; the same memory for the same name in every layer
        and step (it grows when a larger one is asked for).  The views handed out are kept: a
        layer asks for the shapes the layer before asked for."""
        ws = self._ws
        shape = tuple(shape)
        hit = ws.get((name, shape, dtype))
        if hit is not None and hit[0] is ws.get((name, dtype)):
            return hit[1]
        n = 1
        for s in shape:
            n *= int(s)
        t = ws.get((name, dtype))
        if t is None or t.numel() < n:
            cap = max(n, 1)
            if t is not None:
                cap = max(cap, int(t.numel() * 1.5))
            t = torch.empty(cap, dtype=dtype, device=self.device)
            ws[(name, dtype)] = t
        view = t[:n].view(*shape)
        ws[(name, shape, dtype)] = (t, view)
        return view

    def _meta_buffers(self, n_ints: int, dev_fixed: Optional[torch.Tensor] = None):
        """A pinned host buffer (two take turns) and the device buffer, both >= n_ints.
        `dev_fixed`: use this device buffer (a captured graph reads its address)."""
        if dev_fixed is not None and dev_fixed.numel() < n_ints:
            raise EngineError("the fixed metadata buffer is too small for this step")
        if self._meta_dev is None or self._meta_dev.numel() < n_ints:
            cap = max(4096, int(n_ints * 1.5))
            self._meta_dev = torch.empty(cap, dtype=torch.int32, device=self.device)
            self._meta_host = [torch.empty(cap, dtype=torch.int32, pin_memory=True) for _ in range(2)]
            self._meta_events = [None, None]
        i = self._meta_turn
        self._meta_turn ^= 1
        ev = self._meta_events[i]
        if ev is not None:
            ev.synchronize()          # the copy that last read this buffer has finished
        return i, self._meta_host[i], (self._meta_dev if dev_fixed is None else dev_fixed)

    # --------------------------------------------------------------------- step
    def release(self, request: Hashable) -> None:
        """The request is over: its pages and its slot are given back."""
        self.cache.release(request)

    def step(self, entries: Sequence[StepEntry]) -> Optional[torch.Tensor]:
        """Run one batch.  Returns float32 logits [wanted, vocab] in the order of
        the entries and of their `want` (None if nothing is wanted).  The tensor
        is engine workspace: it is valid until the next step."""
        ctx = self.prepare(entries)
        logits = self.run(ctx)
        self.finish(ctx)
        return logits

    def prepare(self, entries: Sequence[StepEntry], meta_dev: Optional[torch.Tensor] = None) -> StepContext:
        """Check the batch, reserve pages, build and upload the step's metadata."""
        if not entries:
            raise EngineError("a step needs at least one entry")
        V = self.model.vocab_size
        cache = self.cache
        starts_fast = self._reserve_decode_step(entries)
        seen = set()
        token_arrays: Dict[Hashable, np.ndarray] = {}
        M = 0
        n_want = 0
        for e in (entries if starts_fast is None else ()):
            toks = e.tokens
            n = len(toks)
            if e.request in seen:
                raise EngineError(f"request {e.request!r} appears twice in one step")
            seen.add(e.request)
            if n == 0:
                raise EngineError(f"request {e.request!r}: an entry needs at least one token")
            if n > 64:
                # a long portion: one conversion serves the check here and the upload below
                arr = np.asarray(toks)
                if arr.ndim != 1 or arr.dtype.kind not in "iu":
                    raise EngineError(f"request {e.request!r}: token ids must be a flat sequence of integers")
                in_vocab = 0 <= int(arr.min()) and int(arr.max()) < V
                token_arrays[e.request] = arr
            else:
                in_vocab = 0 <= min(toks) and max(toks) < V
            if not in_vocab:
                bad = next(t for t in toks if not (0 <= int(t) < V))
                raise EngineError(f"request {e.request!r}: token id {bad} is outside the vocabulary [0, {V})")
            if e.want and not (0 <= min(e.want) and max(e.want) < n):
                bad = next(w for w in e.want if not (0 <= int(w) < n))
                raise EngineError(f"request {e.request!r}: wanted place {bad} is outside its {n} tokens")
            M += n
            n_want += len(e.want)

        paged = cache.paged_groups()
        if starts_fast is not None:
            M = len(entries)
            n_want = sum(len(e.want) for e in entries)
        # all or nothing: see that every group can cover every entry before taking a page
        n_new = 0 if starts_fast is not None else sum(1 for e in entries if not cache.has(e.request))
        if n_new > cache.num_free_slots():
            raise EngineError(f"{n_new} new requests but only {cache.num_free_slots()} free request slots")
        for gi, g in (paged if starts_fast is None else ()):
            need = 0
            for e in entries:
                known = cache.has(e.request)
                upto = (cache._requests[e.request].reserved if known else 0) + len(e.tokens)
                if upto > cache.max_seq:
                    raise EngineError(f"request {e.request!r}: {upto} tokens exceed max_seq = {cache.max_seq}")
                need += g.pages_to_cover(e.request if known else None, upto)
            if need > g.pool.num_free:
                raise OutOfPages(f"the step needs {need} new pages in cache group {gi}, {g.pool.num_free} are free")
        for e in (entries if starts_fast is None else ()):
            if not cache.has(e.request):
                cache.admit(e.request)
            cache.reserve(e.request, len(e.tokens))
        if cache.slots_to_clear:
            self.storage.clear_slots(cache.slots_to_clear)
            cache.slots_to_clear.clear()

        ctx = StepContext(self)
        ctx.M = M
        R = len(entries)
        W = self.table_width
        # layout: tokens | positions | slots | out_rows | entries [R,4] | tiles [n_tiles,2] |
        #         small tiles [n_small,2] | decode rows | tables
        n_tiles = sum(-(-len(e.tokens) // PREFILL_TILE_Q) for e in entries if len(e.tokens) > 1)
        n_small = sum(-(-len(e.tokens) // PREFILL_TILE_SMALL) for e in entries if len(e.tokens) > 1)
        ctx.decode_only = n_tiles == 0
        n_dec = 0 if ctx.decode_only else sum(1 for e in entries if len(e.tokens) == 1)
        ctx.n_tiles, ctx.n_tiles_small, ctx.n_decode_rows = n_tiles, n_small, n_dec
        o_tok, o_pos, o_slot = 0, M, 2 * M
        o_out = 3 * M
        o_ent = o_out + n_want
        o_tile = o_ent + 4 * R
        o_small = o_tile + 2 * n_tiles
        o_dec = o_small + 2 * n_small
        o_tab = o_dec + n_dec
        total = o_tab + len(paged) * R * W
        turn, host, dev = self._meta_buffers(total, meta_dev)
        h = host.numpy()
        out_rows: List[int] = []
        ent_flat: List[int] = []
        if ctx.decode_only:
            # single tokens only: three short lists, one assignment each
            starts = starts_fast if starts_fast is not None else [cache.length(e.request) for e in entries]
            h[o_tok:o_pos] = [e.tokens[0] for e in entries]
            h[o_pos:o_slot] = starts
            h[o_slot:o_out] = range(R)
            known = cache._requests
            slots = [known[e.request].slot for e in entries]
            ctx.entries = list(zip(range(R), [1] * R, starts, slots))
            ent = np.empty((R, 4), dtype=np.int32)
            ent[:, 0] = np.arange(R, dtype=np.int32)
            ent[:, 1] = 1
            ent[:, 2] = starts
            ent[:, 3] = slots
            ent_flat = ent.ravel()
            out_rows = [i for i, e in enumerate(entries) for _ in e.want]
            ctx.max_context = max(starts) + 1
        else:
            tiles: List[int] = []         # (entry, first row) pairs, flat
            small: List[Tuple[int, int, int]] = []   # (last position, entry, first row)
            dec_rows: List[int] = []
            row0 = 0
            for i, e in enumerate(entries):
                n = len(e.tokens)
                start = cache.length(e.request)
                rec = (row0, n, start, cache.slot(e.request))
                ctx.entries.append(rec)
                ent_flat.extend(rec)
                h[o_tok + row0:o_tok + row0 + n] = token_arrays.get(e.request, e.tokens)
                h[o_slot + row0:o_slot + row0 + n] = i
                if n > 1:
                    h[o_pos + row0:o_pos + row0 + n] = np.arange(start, start + n, dtype=np.int32)
                    for q0 in range(0, n, PREFILL_TILE_Q):
                        tiles.append(i)
                        tiles.append(row0 + q0)
                    for q0 in range(0, n, PREFILL_TILE_SMALL):
                        small.append((start + min(q0 + PREFILL_TILE_SMALL, n) - 1, i, row0 + q0))
                    if start + n > ctx.portion_context:
                        ctx.portion_context = start + n
                else:
                    h[o_pos + row0] = start
                    dec_rows.append(row0)
                for w in e.want:
                    out_rows.append(row0 + int(w))
                if start + n > ctx.max_context:
                    ctx.max_context = start + n
                row0 += n
            small.sort(key=lambda t: -t[0])
            h[o_tile:o_tab] = tiles + [v for t in small for v in t[1:]] + dec_rows
        ctx.split_context = ctx.max_context
        h[o_out:o_ent] = out_rows
        h[o_ent:o_tile] = ent_flat
        for k, (gi, g) in enumerate(paged):
            base = o_tab + k * R * W
            rows = g.rows
            h[base:base + R * W].reshape(R, W)[:] = [rows[e.request] for e in entries]
        dev[:total].copy_(host[:total], non_blocking=True)
        ev = torch.cuda.Event()
        ev.record()
        self._meta_events[turn] = ev

        ctx.tokens = dev[o_tok:o_tok + M]
        ctx.positions = dev[o_pos:o_pos + M]
        ctx.slots = dev[o_slot:o_slot + M]
        ctx.out_rows = dev[o_out:o_out + n_want] if n_want else None
        ctx.entry_meta = dev[o_ent:o_ent + 4 * R].view(R, 4)
        ctx.tiles = dev[o_tile:o_tile + 2 * n_tiles].view(-1, 2) if n_tiles else None
        ctx.tiles_small = dev[o_small:o_small + 2 * n_small].view(-1, 2) if n_small else None
        ctx.decode_rows = dev[o_dec:o_dec + n_dec] if n_dec else None
        for k, (gi, g) in enumerate(paged):
            base = o_tab + k * R * W
            ctx._views[gi] = CacheView(dev[base:base + R * W].view(R, W), self.page_size)
        ctx._entries_in = list(entries)
        ctx._decode_fast = starts_fast is not None
        return ctx

    def _reserve_decode_step(self, entries: Sequence[StepEntry]) -> Optional[List[int]]:
        """The common step, checked and reserved in one pass: every entry is one token of a
        request that is admitted already.  Returns the tokens' positions, or None for any
        other step (nothing has been done then; `prepare` takes its general path)."""
        cache = self.cache
        known = cache._requests
        for e in entries:
            r = known.get(e.request)
            if len(e.tokens) != 1 or r is None or r.reserved != r.length:
                return None
        reqs = [e.request for e in entries]
        if len(set(reqs)) != len(reqs):
            return None                                   # the general path names the request
        toks = [e.tokens[0] for e in entries]
        if not (0 <= min(toks) and max(toks) < self.model.vocab_size):
            return None                                   # the general path names the token
        for e in entries:
            for w in e.want:
                if w != 0:
                    return None
        try:
            return cache.reserve_one_each(reqs)
        except CacheError as err:
            if isinstance(err, OutOfPages):
                raise
            raise EngineError(str(err)) from None

    def run(self, ctx: StepContext) -> Optional[torch.Tensor]:
        """The model over the step's tokens: embedding, the layers in run order,
        then final norm and head on the wanted rows only."""
        model = self.model
        x = ctx.buf("x", (ctx.M, model.hidden_size), torch.float32)
        model.embedding.forward(ctx, ctx.tokens, x)
        for r, li in enumerate(model.run_order):
            ctx.run = r
            model.blocks[li].forward(ctx, x)
        if ctx.out_rows is None:
            self.ops.flush()
            return None
        h = model.final_norm.forward(ctx, x, rows=ctx.out_rows)
        return model.head.forward(ctx, h)

    def finish(self, ctx: StepContext) -> None:
        if ctx._decode_fast:
            self.cache.commit_one_each([e.request for e in ctx._entries_in])
        else:
            for e in ctx._entries_in:
                self.cache.commit(e.request, len(e.tokens))
        self.steps_run += 1

    # ------------------------------------------------------------------ graphs
    def step_graph(self, entries: Sequence[StepEntry]) -> Optional[torch.Tensor]:
        """`step`, replayed from a captured HIP graph where there is one.  A batch of single
        tokens that each want their logits has a graph per batch size, captured the first time
        (the reference keys its CUDA graphs the same way: /root/reference/src/inference.cu:267-295).
        Any other step has a shape: the token count and the wanted places of every entry, in
        order (a prompt arriving in equal portions beside the same decoding requests repeats
        its shape step after step); a shape is captured when it comes for the
        `STEP_GRAPH_AFTER`-th time, the `MAX_STEP_GRAPHS` most recently used are kept, and until
        then the step runs through `step`.

        What a replay reads is at fixed addresses: the graph has its own metadata buffer
        (tokens, positions, work lists, block-table rows: refreshed by one copy before each
        replay) and its own workspace; loop bounds are read on the device, and the numbers of
        runs the attention cuts contexts into are sized for the longest sequence, not for the
        step.  Sampling stays outside the graph."""
        if all(len(e.tokens) == 1 and tuple(e.want) == (0,) for e in entries):
            key = len(entries)
        else:
            key = tuple((len(e.tokens), tuple(e.want)) for e in entries)
        rec = self._graphs.get(key)
        if rec is None:
            if not isinstance(key, int):
                if len(self._shapes_seen) > 4096:
                    self._shapes_seen.clear()
                seen = self._shapes_seen[key] = self._shapes_seen.get(key, 0) + 1
                if seen < STEP_GRAPH_AFTER:
                    return self.step(entries)
                del self._shapes_seen[key]
                shapes = [k for k in self._graphs if not isinstance(k, int)]
                if len(shapes) >= MAX_STEP_GRAPHS:
                    del self._graphs[shapes[0]]            # the one unused for longest (see below)
            return self._capture(entries, key)
        if not isinstance(key, int):
            self._graphs[key] = self._graphs.pop(key)       # most recently used last
        saved = self._ws
        self._ws = rec.workspace
        try:
            ctx = self.prepare(entries, meta_dev=rec.meta)
        finally:
            self._ws = saved
        rec.graph.replay()
        self.finish(ctx)
        return rec.logits

    def _capture(self, entries: Sequence[StepEntry], key) -> Optional[torch.Tensor]:
        R = len(entries)
        paged = len(self.cache.paged_groups())
        M = sum(len(e.tokens) for e in entries)
        n_lists = sum(-(-len(e.tokens) // PREFILL_TILE_Q) + -(-len(e.tokens) // PREFILL_TILE_SMALL) for e in entries)
        rec = _DecodeGraph()
        # what `prepare` lays out: tokens, positions, slots, wanted rows, entries, work lists, tables
        rec.meta = torch.empty(3 * M + sum(len(e.want) for e in entries) + 4 * R + 2 * n_lists + R
                               + paged * R * self.table_width + 64, dtype=torch.int32, device=self.device)
        saved = self._ws
        self._ws = rec.workspace
        try:
            ctx = self.prepare(entries, meta_dev=rec.meta)
            ctx.split_context = self.max_seq
            if ctx.n_tiles:
                ctx.portion_context = max(ctx.portion_context, self.max_seq // 2)
            # a first run outside the graph: it computes this step's result and makes every
            # workspace buffer the graph will use
            side = torch.cuda.Stream()
            side.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(side):
                self.run(ctx)
            torch.cuda.current_stream().wait_stream(side)
            torch.cuda.synchronize()
            rec.graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(rec.graph):
                rec.logits = self.run(ctx)
        finally:
            self._ws = saved
        # capture records, it does not run: the first run above already wrote this step's
        # keys, values and logits, and a replay would write the same again
        self.finish(ctx)
        self._graphs[key] = rec
        return rec.logits


class _DecodeGraph:
    """A captured step (one batch size of single tokens, or one shape), with the buffers it reads and writes."""

    def __init__(self):
        self.graph = None
        self.meta: Optional[torch.Tensor] = None
        self.workspace: Dict[tuple, object] = {}
        self.logits: Optional[torch.Tensor] = None


def required_libraries(dtype: str):
    """The kernel libraries a model of this dtype needs (what a first call compiles)."""
    import os
    from ..csrc import build
    libs = ["core", "gemm_generic", "attention_generic", "sampling"]
    if dtype == "bfloat16":
        libs += [n for n in ("gemm_bf16", "attention_bf16")
                 if os.path.isfile(os.path.join(build.HERE, build.SOURCES[n]))]
    return libs
