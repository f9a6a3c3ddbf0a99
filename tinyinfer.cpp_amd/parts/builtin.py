"""The built-in parts, named from Python.  Each class holds the sizes it was built
with and a handle to the part of the host library that does the work
(parts/parts.cpp, where the formulas and their places in the reference are
given); `forward` hands torch tensors across.  Run inside a step, a part gets the
step's own context; run on its own (a test of one part), it gets a context of
its own made from the caller's `ctx.dtype` and `ctx.positions`.
"""
from __future__ import annotations

import ctypes
import json
import math
from typing import Optional

from .. import native
from ..spec import PartSpec, TensorNeed, cache_need_from_dict
from .base import Handle, Part, children_arrays, part_handle
from .registry import build_part, register_part

ti_tensor = native.ti_tensor


class _OwnContext:
    """A context of the library for parts that run outside a step."""

    def __init__(self, dtype: str):
        native.use_torch_allocator()
        from ..ops.kernels import required_libraries
        native.ensure_kernels(required_libraries(dtype))
        self.ptr = native.pointer("ti_ctx_create", dtype.encode(), None)

    def __del__(self):
        try:
            if native._lib is not None:
                native._lib.ti_ctx_release(self.ptr)
        except Exception:  # noqa: BLE001
            pass


def native_context(ctx, n_rows: int = 0, tokens=None) -> int:
    """The library's context behind `ctx`: the step's, or one of its own kept on `ctx`."""
    ptr = getattr(ctx, "_native", None)
    if ptr:
        return ptr
    own = getattr(ctx, "_ti_own", None)
    if own is None:
        own = ctx._ti_own = _OwnContext(ctx.dtype)
    pos = getattr(ctx, "positions", None)
    native.call("ti_ctx_set_rows", own.ptr, n_rows, None if pos is None else pos.data_ptr(),
                None if tokens is None else tokens.data_ptr())
    return own.ptr


class NativePart(Part):
    """A part of the host library.  `kind` names it in its family; `params` is what it was built from."""
    kind = ""

    def _create(self, params: dict, children=()):
        children = list(children)
        n, slots, handles = children_arrays(children)
        self._children = [p for _, p in children]
        self._ti_handle = Handle(native.pointer("ti_part_create", self.family.encode(), self.kind.encode(),
                                                self.prefix.encode(), json.dumps(params).encode(), n, slots, handles))

    def tensors(self):
        d = json.loads(native.text("ti_part_tensors", self._ti_handle.ptr))
        return {n: TensorNeed.from_dict(v) for n, v in d.items()}

    def children(self):
        return list(self._children)

    def cache_need(self):
        return cache_need_from_dict(json.loads(native.text("ti_part_cache_need", self._ti_handle.ptr)))

    def load(self, tensors) -> None:
        """Copy `tensors` (by name; torch tensors already in the dtype their role asks for) into the
        part's own memory."""
        names = list(tensors)
        ts = [tensors[n].contiguous() for n in names]
        on_host = bool(ts) and not ts[0].is_cuda
        if not on_host:
            native.use_torch_allocator()
        matrix = "float32"
        needs = self.tensors()
        for n, t in zip(names, ts):
            if n in needs and needs[n].role == "matrix":
                matrix = "bfloat16" if t.dtype == native.torch().bfloat16 else "float32"
        native.call("ti_part_load", self._ti_handle.ptr, len(ts), "\n".join(names).encode(), native.describe_many(ts),
                    matrix.encode(), int(on_host))

    def held(self, member: str):
        """A tensor the part holds ("weight", "w_qkv", ...), None if it has none of that name."""
        out = ti_tensor()
        native.call("ti_part_held", self._ti_handle.ptr, member.encode(), ctypes.byref(out))
        return native.wrap(out, keep=self._ti_handle)

    def _call(self, op: str, ctx_ptr, args=(), flags: int = 0, n_results: int = 0, fold=()):
        res = (ti_tensor * max(1, n_results))()
        native.call("ti_part_call", self._ti_handle.ptr, op.encode(), ctx_ptr, native.describe_many(args, fold), len(args),
                    flags, res)
        return [native.wrap(res[i]) for i in range(n_results)]


class Embedding(NativePart):
    family, kind = "embedding", "table"

    def __init__(self, prefix: str, vocab: int, dim: int):
        super().__init__(prefix)
        self.vocab, self.dim = int(vocab), int(dim)
        self._create({"vocab": self.vocab, "dim": self.dim})

    weight = property(lambda self: self.held("weight"))

    def forward(self, ctx, tokens, x):
        self._call("forward", native_context(ctx, tokens.shape[0], tokens), [x])


class LMHead(NativePart):
    """`tied`: True reads `tied_to`; False reads its own `weight`; None takes its own weight if the
    checkpoint holds one and `tied_to` otherwise."""
    family, kind = "head", "linear"

    def __init__(self, prefix: str, vocab: int, dim: int, tied, tied_to: str):
        super().__init__(prefix)
        self.vocab, self.dim, self.tied, self.tied_to = int(vocab), int(dim), tied, tied_to
        self._create({"vocab": self.vocab, "dim": self.dim, "tied": tied, "tied_to": tied_to})

    weight = property(lambda self: self.held("weight"))

    def forward(self, ctx, h_rows):
        return self._call("forward", native_context(ctx, h_rows.shape[0]), [h_rows], n_results=1)[0]


class RMSNorm(NativePart):
    family, kind = "norm", "rmsnorm"
    can_be_lazy = True

    def __init__(self, prefix: str, dim: int, eps: float):
        super().__init__(prefix)
        self.dim, self.eps = int(dim), float(eps)
        self._create({"dim": self.dim, "eps": self.eps})

    weight = property(lambda self: self.held("weight"))

    def forward(self, ctx, x, out=None, rows=None, lazy=False):
        """x: f32 [M, dim].  Returns the normed rows in the compute dtype; with `rows` (i32 [N]) only
        those rows of x are read, in that order."""
        res = self._call("forward", native_context(ctx, x.shape[0]), [x] + ([rows] if rows is not None else []),
                         n_results=1)[0]
        if out is not None:
            out.copy_(res)
            return out
        return res


class RotaryNeox(NativePart):
    family, kind = "pos", "rope_neox"

    def __init__(self, prefix: str, head_dim: int, theta: float):
        super().__init__(prefix)
        if head_dim % 2:
            raise ValueError(f"rotary: head_dim {head_dim} must be even")
        self.head_dim, self.theta = int(head_dim), float(theta)
        self._create({"head_dim": self.head_dim, "theta": self.theta})

    def to(self, device):
        native.use_torch_allocator()
        self._call("prepare", None, flags=0)
        return self

    def prepare(self, ops, max_positions: int):
        """Tabulate cos and sin for positions [0, max_positions)."""
        native.use_torch_allocator()
        self._call("prepare", None, flags=int(max_positions))

    inv_freq = property(lambda self: self.held("inv_freq"))
    table = property(lambda self: self.held("table"))

    def fused_rotation(self):
        """What the fused norm/rotate/cache-write kernels read."""
        return {"inv_freq": self.inv_freq, "table": self.table}

    def apply(self, ctx, q, k):
        """In place on f32 [M, heads, hd] views (strided rows allowed)."""
        self._call("apply", native_context(ctx, q.shape[0]), [q] + ([k] if k is not None else []))


class SwiGLU(NativePart):
    family, kind = "ffn", "swiglu"
    takes_lazy_norm = True

    def __init__(self, prefix: str, hidden: int, intermediate: int):
        super().__init__(prefix)
        self.hidden, self.intermediate = int(hidden), int(intermediate)
        self._create({"hidden": self.hidden, "intermediate": self.intermediate})

    w_gate_up = property(lambda self: self.held("w_gate_up"))
    w_down = property(lambda self: self.held("w_down"))

    def forward(self, ctx, h, x):
        self._call("forward", native_context(ctx, h.shape[0]), [h, x])


class Attention(NativePart):
    family, kind = "mixer", "attention"
    takes_lazy_norm = True

    def __init__(self, prefix: str, hidden: int, heads: int, kv_heads: int, head_dim: int, qk_norm: bool = True,
                 eps: float = 1e-6, window: Optional[int] = None, scale: Optional[float] = None, pos=None,
                 shares_kv: bool = False):
        super().__init__(prefix)
        if heads % kv_heads:
            raise ValueError(f"attention: heads {heads} not a multiple of kv_heads {kv_heads}")
        self.hidden, self.heads, self.kv_heads, self.head_dim = int(hidden), int(heads), int(kv_heads), int(head_dim)
        self.qk_norm, self.eps = bool(qk_norm), float(eps)
        self.window = None if window is None else int(window)
        self.scale = float(scale) if scale is not None else 1.0 / math.sqrt(self.head_dim)
        self.shares_kv = bool(shares_kv)
        if isinstance(pos, dict):
            pos = PartSpec.from_dict(pos)
        self.pos = build_part("pos", pos, prefix) if pos is not None else None
        self.nq = self.heads * self.head_dim
        self.nk = 0 if self.shares_kv else self.kv_heads * self.head_dim
        params = {"hidden": self.hidden, "heads": self.heads, "kv_heads": self.kv_heads, "head_dim": self.head_dim,
                  "qk_norm": self.qk_norm, "eps": self.eps, "window": self.window, "scale": self.scale,
                  "shares_kv": self.shares_kv}
        self._create(params, [("pos", self.pos)] if self.pos is not None else [])

    w_qkv = property(lambda self: self.held("w_qkv"))
    w_o = property(lambda self: self.held("w_o"))
    q_norm_w = property(lambda self: self.held("q_norm_w"))
    k_norm_w = property(lambda self: self.held("k_norm_w"))

    def forward(self, ctx, h, x):
        self._call("forward", native_context(ctx, h.shape[0]), [h, x])


class PreNormBlock(NativePart):
    """x += mixer(norm1(x)); x += ffn(norm2(x))."""
    family, kind = "block", "pre_norm"
    # which family each named slot of this arrangement is built from
    slots = {"norm1": "norm", "mixer": "mixer", "norm2": "norm", "ffn": "ffn"}

    def __init__(self, prefix: str, norm1, mixer, norm2, ffn):
        super().__init__(prefix)
        self.norm1, self.mixer, self.norm2, self.ffn = norm1, mixer, norm2, ffn
        self._create({}, [("norm1", norm1), ("mixer", mixer), ("norm2", norm2), ("ffn", ffn)])

    def forward(self, ctx, x):
        self._call("forward", native_context(ctx, x.shape[0]), [x])


register_part("embedding", "table", Embedding)
register_part("head", "linear", LMHead)
register_part("norm", "rmsnorm", RMSNorm)
register_part("pos", "rope_neox", RotaryNeox)
register_part("ffn", "swiglu", SwiGLU)
register_part("mixer", "attention", Attention)
register_part("block", "pre_norm", PreNormBlock)
