"""Parts of the host library, seen from Python.  A view holds a handle to the library's
part (parts/parts.cpp, where the formulas and their places in the reference are given)
and what the part was built from; `forward` hands torch tensors across.  Every family
has a view class, so a kind that the library or a plugin registers is usable from
Python without a line here; the built-in kinds have named views that add their
defaults and conveniences.  Run inside a step, a part gets the step's own context;
run on its own (a test of one part), it gets a context of its own made from the
caller's `ctx.dtype` and `ctx.positions`.
"""
from __future__ import annotations

import ctypes
import json
import math

from .. import native
from ..spec import TensorNeed, cache_need_from_dict
from .base import Handle, Part

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
    """A part of the host library.  `family` and `kind` name it; `params` is what it was built from (each
    entry also reads as an attribute, and so does every tensor the part holds: `part.w_qkv`)."""
    kind = ""

    def _adopted(self, handle: Handle, info: dict):
        self.prefix = info["prefix"]
        self.family, self.kind = info["family"], info["built_kind"] or info["kind"]
        self.params = info["params"]
        self._ti_handle = handle
        self._slots = list(info["slots"])
        self._children = []
        for i, slot in enumerate(self._slots):
            child = adopt(native.pointer("ti_part_child", handle.ptr, i))
            self._children.append(child)
            if not slot.isdigit():
                self.__dict__[slot] = child
        return self

    def __getattr__(self, name):
        if name.startswith("_"):
            raise AttributeError(name)
        params = self.__dict__.get("params") or {}
        if name in params:
            return params[name]
        if "_ti_handle" in self.__dict__:
            t = self.held(name)
            if t is not None:
                return t
        raise AttributeError(f"{type(self).__name__} ({self.__dict__.get('kind')}) has no parameter, child or tensor {name!r}")

    def tensors(self):
        d = json.loads(native.text("ti_part_tensors", self._ti_handle.ptr))
        return {n: TensorNeed.from_dict(v) for n, v in d.items()}

    def children(self):
        return list(self._children)

    def cache_need(self):
        return cache_need_from_dict(json.loads(native.text("ti_part_cache_need", self._ti_handle.ptr)))

    def info(self) -> dict:
        return json.loads(native.text("ti_part_info", self._ti_handle.ptr))

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


# ----------------------------------------------------------- one view per family
class NativeEmbedding(NativePart):
    def forward(self, ctx, tokens, x):
        self._call("forward", native_context(ctx, tokens.shape[0], tokens), [x])


class NativeHead(NativePart):
    def forward(self, ctx, h_rows):
        return self._call("forward", native_context(ctx, h_rows.shape[0]), [h_rows], n_results=1)[0]


class NativeNorm(NativePart):
    def forward(self, ctx, x, out=None, rows=None, lazy=False):
        """x: f32 [M, dim].  Returns the normed rows in the compute dtype; with `rows` (i32 [N]) only
        those rows of x are read, in that order."""
        res = self._call("forward", native_context(ctx, x.shape[0]), [x] + ([rows] if rows is not None else []),
                         n_results=1)[0]
        if out is not None:
            out.copy_(res)
            return out
        return res

    can_be_lazy = property(lambda self: self.info()["can_be_lazy"])


class NativePos(NativePart):
    def apply(self, ctx, q, k):
        """In place on f32 [M, heads, hd] views (strided rows allowed)."""
        self._call("apply", native_context(ctx, q.shape[0]), [q] + ([k] if k is not None else []))

    def prepare(self, ops, max_positions: int):
        """Whatever the part tabulates for positions [0, max_positions)."""
        native.use_torch_allocator()
        self._call("prepare", None, flags=int(max_positions))


class NativeMixer(NativePart):
    """Mixers and feed-forwards: `forward(ctx, h, x)` adds the part's output into x."""

    def forward(self, ctx, h, x):
        self._call("forward", native_context(ctx, h.shape[0]), [h, x])

    takes_lazy_norm = property(lambda self: self.info()["takes_lazy_norm"])


class NativeBlock(NativePart):
    def forward(self, ctx, x):
        self._call("forward", native_context(ctx, x.shape[0]), [x])


FAMILY_VIEWS = {"embedding": NativeEmbedding, "head": NativeHead, "norm": NativeNorm, "pos": NativePos, "mixer": NativeMixer,
                "ffn": NativeMixer, "block": NativeBlock}


# ------------------------------------------------------- the built-in kinds, by name
class Embedding(NativeEmbedding):
    pass


class LMHead(NativeHead):
    """`tied`: True reads `tied_to`; False reads its own `weight`; None takes its own weight if the
    checkpoint holds one and `tied_to` otherwise."""


class RMSNorm(NativeNorm):
    pass


class RotaryNeox(NativePos):
    def to(self, device):
        native.use_torch_allocator()
        self._call("prepare", None, flags=0)
        return self

    def fused_rotation(self):
        """What the fused norm/rotate/cache-write kernels read."""
        return {"inv_freq": self.held("inv_freq"), "table": self.held("table")}


class SwiGLU(NativeMixer):
    pass


class Attention(NativeMixer):
    window = property(lambda self: self.params.get("window"))
    qk_norm = property(lambda self: self.params.get("qk_norm", True))
    shares_kv = property(lambda self: bool(self.params.get("shares_kv")))
    scale = property(lambda self: self.params["scale"] if self.params.get("scale") is not None
                     else 1.0 / math.sqrt(self.params["head_dim"]))
    nq = property(lambda self: self.params["heads"] * self.params["head_dim"])
    nk = property(lambda self: 0 if self.shares_kv else self.params["kv_heads"] * self.params["head_dim"])
    pos = None            # (an attention without a position encoding has no such child)


class PreNormBlock(NativeBlock):
    """x += mixer(norm1(x)); x += ffn(norm2(x))."""


KIND_VIEWS = {("embedding", "table"): Embedding, ("head", "linear"): LMHead, ("norm", "rmsnorm"): RMSNorm,
              ("pos", "rope_neox"): RotaryNeox, ("ffn", "swiglu"): SwiGLU, ("mixer", "attention"): Attention,
              ("block", "pre_norm"): PreNormBlock}


def adopt(ptr: int):
    """The Python object for a part of the library, given a handle that becomes this object's own: the
    Python part itself if the part is implemented here, else a view of the library's part."""
    handle = Handle(ptr)
    info = json.loads(native.text("ti_part_info", ptr))
    if info["foreign_id"]:
        return native.foreign_object(info["foreign_id"])         # (the handle goes; the part keeps its own)
    cls = KIND_VIEWS.get((info["family"], info["built_kind"] or info["kind"])) or FAMILY_VIEWS[info["family"]]
    return cls.__new__(cls)._adopted(handle, info)
