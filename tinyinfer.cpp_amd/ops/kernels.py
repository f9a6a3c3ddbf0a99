"""The kernels, as Python calls on torch tensors.

Each call hands its tensors to the host library's `Ops` (ops/ops.cpp), which
checks devices, dtypes and shapes, picks the kernel for the sizes, and launches
the hand-written HIP kernel through the C interface of the kernel libraries
(`csrc/`).  Nothing here computes with torch, and nothing falls back to the CPU or
to a library: without a GPU or without the compiled libraries a call raises.
`Ops.lib(name)` gives a kernel library itself, for tests that call one kernel.
"""
from __future__ import annotations

import ctypes
import os
from typing import Dict, Optional

from .. import native
from ..csrc import build as _build
from ..native import KernelError  # noqa: F401

F32, BF16 = 0, 1
EPI = {"store": 0, "add": 1, "store_act": 2, "swiglu": 3}

_C_TYPES = {"int": ctypes.c_int, "long": ctypes.c_long, "float": ctypes.c_float, "unsigned long": ctypes.c_ulong}


def required_libraries(dtype: str):
    """The kernel libraries a model of this dtype needs (what a first call compiles)."""
    return _build.libraries_for(dtype)


def header_signatures(text: str) -> Dict[str, tuple]:
    """{function: (restype, [argtypes])} of the `int ti_...(...)`, `long ti_...(...)` and `void ti_...(...)`
    declarations of a kernels' header: pointers and streams as void pointers, int, long and
    float as themselves.  A declaration with any other type raises."""
    import re
    text = re.sub(r"//[^\n]*", "", text)
    out = {}
    for ret, name, args in re.findall(r"\b(int|long|void)\s+(ti_\w+)\s*\(([^)]*)\)\s*;", text):
        types = []
        for arg in (a.strip() for a in args.split(",")):
            if not arg or arg == "void":
                continue
            if "*" in arg or arg.startswith("hipStream_t"):
                types.append(ctypes.c_void_p)
                continue
            words = [w for w in arg.replace("const", " ").split()]
            kind = " ".join(words[:-1])
            if len(words) < 2 or kind not in _C_TYPES:
                raise KernelError(f"tinyinfer_kernels.h: cannot read the argument {arg!r} of {name}")
            types.append(_C_TYPES[kind])
        out[name] = ({"int": ctypes.c_int, "long": ctypes.c_long, "void": None}[ret], types)
    return out


_signatures: Optional[Dict[str, tuple]] = None


def declare_signatures(lib: ctypes.CDLL) -> None:
    """Give every function of the headers that this library exports its argument types."""
    global _signatures
    if _signatures is None:
        _signatures = {}
        for header in ("tinyinfer_kernels.h", "tinyinfer_kernels_tuning.h"):
            with open(os.path.join(_build.HERE, header)) as f:
                _signatures.update(header_signatures(f.read()))
    for name, (restype, argtypes) in _signatures.items():
        try:
            fn = getattr(lib, name)
        except AttributeError:
            continue
        fn.restype = restype
        fn.argtypes = argtypes


class NormedRows:
    """rmsnorm(x; weight, eps) that has not been computed yet: `Ops.linear` accepts it in place of
    the activation and runs the norm inside the product's kernel where a kernel for that exists,
    else it computes the rows into `out` first."""

    def __init__(self, x, weight, eps: float, out):
        self.x, self.weight, self.eps, self.out = x, weight, eps, out
        self.shape = out.shape
        self.dtype = out.dtype

    def materialize(self, ops: "Ops"):
        ops.rmsnorm(self.x, self.weight, self.eps, self.out)
        return self.out


_SWITCHES = {"use_fast_gemm": "fast_gemm", "use_fast_attention": "fast_attention", "use_fused_norm": "fused_norm",
             "use_fused_qk_decode": "fused_qk_decode", "use_fused_qkv_prefill": "fused_qkv_prefill",
             "use_split_k_add": "split_k_add", "use_deferred_add": "deferred_add", "use_paired_prefill": "paired_prefill",
             "use_portion_splits": "portion_splits", "use_early_page_ids": "early_page_ids",
             "use_radix_sample": "radix_sample"}
_LIB_OF = {"embed": "core", "rmsnorm": "core", "rope_neox": "core", "rope_table": "core", "qk_norm_rope_kv_write": "core",
           "qk_norm_inplace": "core", "argmax": "sampling", "sample": "sampling", "attention_rows": "attention_generic",
           "fill_random": "core", "fill_zero": "core"}


class Ops:
    """One method per op, on an `Ops` object of the host library: an engine's own, or one made here."""

    def __init__(self, _borrowed: Optional[int] = None):
        object.__setattr__(self, "_libs", {})
        object.__setattr__(self, "_own", _borrowed is None)
        if _borrowed is None:
            t = native.torch()
            if not t.cuda.is_available():
                raise KernelError("no GPU: the kernels of this framework run on an AMD GPU (gfx950) only")
            native.use_torch_allocator()
            _borrowed = native.pointer("ti_ops_create", None)
        object.__setattr__(self, "_ptr", _borrowed)

    def __del__(self):
        try:
            if self._own and native._lib is not None:
                native._lib.ti_ops_release(self._ptr)
        except Exception:  # noqa: BLE001
            pass

    # switches for tests and measurements (each leaves the results the same up to the order of sums)
    def __getattr__(self, name):
        if name in _SWITCHES:
            old = ctypes.c_int()
            native.call("ti_ops_switch", self._ptr, _SWITCHES[name].encode(), -1, ctypes.byref(old))
            if name in ("use_fast_gemm", "use_fast_attention"):
                lib = "gemm_bf16" if name == "use_fast_gemm" else "attention_bf16"
                return bool(old.value) and os.path.isfile(os.path.join(_build.HERE, _build.SOURCES[lib]))
            return bool(old.value)
        if name == "_pending":
            return type(self)._pending.fget(self)
        if name == "force_decode_splits":
            old = ctypes.c_int()
            native.call("ti_ops_switch", self._ptr, b"force_decode_splits", -1, ctypes.byref(old))
            return old.value
        if name == "force_paired_tiles":
            old = ctypes.c_int()
            native.call("ti_ops_switch", self._ptr, b"force_paired_tiles", -2, ctypes.byref(old))
            return None if old.value < 0 else bool(old.value)
        raise AttributeError(name)

    def __setattr__(self, name, value):
        if name in _SWITCHES:
            native.call("ti_ops_switch", self._ptr, _SWITCHES[name].encode(), int(bool(value)), None)
        elif name == "force_decode_splits":
            native.call("ti_ops_switch", self._ptr, b"force_decode_splits", int(value or 0), None)
        elif name == "force_paired_tiles":
            native.call("ti_ops_switch", self._ptr, b"force_paired_tiles", -1 if value is None else int(bool(value)), None)
        else:
            object.__setattr__(self, name, value)

    # ------------------------------------------------------------------ loading
    def lib(self, name: str) -> ctypes.CDLL:
        """A kernel library itself (the same one the host library has loaded)."""
        lib = self._libs.get(name)
        if lib is None:
            if not native.torch().cuda.is_available():
                raise KernelError("no GPU: the kernels of this framework run on an AMD GPU (gfx950) only")
            native.ensure_kernels([name])
            lib = ctypes.CDLL(_build.find(name))
            lib.ti_last_error.restype = ctypes.c_char_p
            declare_signatures(lib)
            self._libs[name] = lib
        return lib

    def preload(self, names):
        """Compile (if needed, several at a time) and register the libraries `names`."""
        if not native.torch().cuda.is_available():
            raise KernelError("no GPU: the kernels of this framework run on an AMD GPU (gfx950) only")
        native.ensure_kernels(list(names))

    @staticmethod
    def _check(lib, rc, what):
        if rc != 0:
            raise KernelError(f"{what}: {lib.ti_last_error().decode()}")

    def _raw_stream(self):
        return None

    _stream = _raw_stream

    def _call(self, op: str, tensors=(), numbers=(), text: Optional[str] = None, fold=(), libs=()) -> int:
        native.ensure_kernels(libs or [_LIB_OF.get(op, "core")])
        for t in tensors:
            if t is not None and not t.is_cuda:
                raise KernelError("kernel arguments must live on the GPU")
        res = native.ti_tensor()
        nums = (ctypes.c_double * max(1, len(numbers)))(*[float(v) for v in numbers])
        native.call("ti_ops_call", self._ptr, op.encode(), native.describe_many(tensors, fold), len(tensors), nums,
                    len(numbers), native.enc(text), ctypes.byref(res))
        return res.shape[0]

    @property
    def _pending(self):
        """The number of partial sums a product left for the next norm (None: none are waiting)."""
        return self._call("pending", libs=["core"]) or None

    def timing(self, on: bool) -> None:
        """Switch per-call timing with events on or off (see `Ops::timing`)."""
        self._call("timing", [], [int(bool(on))], libs=["core"])

    def tune(self, library: Optional[str] = None, name: str = "", value: int = 0) -> None:
        """Force a shape rule of a kernel library for this object's calls (`Ops::tune`; the names are listed in
        csrc/tinyinfer_kernels_tuning.h).  Without arguments: every override of this object goes."""
        if library is None:
            self._call("tune", [], [0], libs=["core"])
        else:
            self._call("tune", [], [int(value)], text=f"{library} {name}", libs=[library])

    def count_calls(self, on: bool) -> None:
        """List the calls without timing them (see `Ops::count_calls`): a step runs exactly as it does unobserved;
        `timing_report()` then gives the names, each ending in what the call took ("[mfma]", "[generic]", "[fused]")."""
        self._call("count_calls", [], [int(bool(on))], libs=["core"])

    def timing_report(self):
        """[{"name", "calls", "us"}] of the calls since timing was switched on (or last reported)."""
        import json
        return json.loads(native.text("ti_ops_timing_report", self._ptr))

    def flush(self):
        """Partial sums that a product left for the next norm are added now (same bits).  Every launch
        through this object does it first; code that reads such a residual with torch calls it itself."""
        self._call("flush", libs=["core"])

    # --------------------------------------------------------------------- ops
    def embed(self, table, tokens, x):
        self._call("embed", [table, tokens, x])

    def rmsnorm(self, x, w, eps, out, rows=None):
        self._call("rmsnorm", [x, w, out, rows], [eps])

    def rope_neox(self, x, positions, inv_freq):
        """In place on f32 x [M, heads, hd]; the last two dims contiguous, rows may be strided."""
        self._call("rope_neox", [x, positions, inv_freq])

    def rope_table(self, inv_freq, n_pos):
        """float32 [n_pos, hd/2, 2] = (cos, sin)(float(p) * inv_freq[k]), computed on the device."""
        t = native.torch()
        table = t.empty((n_pos, inv_freq.shape[0], 2), dtype=t.float32, device=inv_freq.device)
        self._call("rope_table", [inv_freq, table])
        return table

    def qk_norm_rope_kv_write(self, qkv, q_w, k_w, eps, inv_freq, positions, slots, view, pool, q_out, heads, kv_heads,
                              head_dim, rope_table=None):
        """qkv f32 [M, (heads + 2 kv_heads) hd] -> q_out T [M, heads hd] and the cache pages.
        kv_heads = 0: only q (nothing is written to the cache)."""
        self._call("qk_norm_rope_kv_write", [qkv, q_w, k_w, inv_freq, rope_table, positions, slots, view.table, pool, q_out],
                   [eps, heads, kv_heads, head_dim], fold=(8,))

    def qk_norm_inplace(self, qkv, q_w, k_w, eps, heads, kv_heads, head_dim):
        self._call("qk_norm_inplace", [qkv, q_w, k_w], [eps, heads, kv_heads, head_dim])

    def can_fuse_norm(self, n_rows: int, dtype) -> bool:
        """Whether `linear` has a kernel that takes the norm of this many rows in."""
        return bool(self._call("can_fuse_norm", [], [n_rows, native.dtype_code(dtype)], libs=["core"]))

    def linear(self, a, w, out, epilogue: str, may_defer: bool = False):
        """out (op)= a w^T.  a: T [M, K] (rows may be strided); w: T [N, K] contiguous.
        epilogue: "store" f32 out = ; "add" f32 out += ; "store_act" T out = ;
        "swiglu": w is [2F, K] = [gate; up], T out [M, F] = silu(gate) * up.
        may_defer (with "add"): the caller reads `out` next through this object (see `flush`)."""
        libs = ["gemm_generic"] + (["gemm_bf16", "core"] if w.dtype == native.torch().bfloat16 and self.use_fast_gemm else [])
        if isinstance(a, NormedRows):
            self._call("linear_normed", [a.x, a.weight, a.out, w, out], [a.eps, EPI[epilogue], int(may_defer)],
                       libs=libs + ["core"])
        else:
            self._call("linear", [a, w, out], [EPI[epilogue], int(may_defer)], libs=libs)

    def _linear_normed(self, a: NormedRows, w, out, epilogue: str) -> bool:
        """rmsnorm and product in one kernel; False if no kernel serves the shape (nothing was launched)."""
        return bool(self._call("linear_normed_only", [a.x, a.weight, a.out, w, out], [a.eps, EPI[epilogue]],
                               libs=["gemm_bf16", "core"]))

    def qkv_prepared(self, a, w, q_w, k_w, eps, inv_freq, rope_table, positions, slots, view, pool, q_out, heads, kv_heads,
                     head_dim) -> bool:
        """`linear(a, w, qkv, "store")` and `qk_norm_rope_kv_write` in one kernel, for steps of many tokens
        in bfloat16.  False if no kernel serves the step (nothing has been done then)."""
        if isinstance(a, NormedRows):
            return False
        return bool(self._call("qkv_prepared", [a, w, q_w, k_w, inv_freq, rope_table, positions, slots, view.table, pool, q_out],
                               [eps, heads, kv_heads, head_dim], fold=(9,), libs=["gemm_bf16", "core"]))

    # ----------------------------------------------------------------- attention
    def attention_rows(self, q, pool, table, positions, slots, out, heads, kv_heads, head_dim, scale, window):
        self._call("attention_rows", [q, pool, table, positions, slots, out], [heads, kv_heads, head_dim, scale, int(window or 0)],
                   fold=(1,))

    @staticmethod
    def _work(ctx):
        """The attention's work lists as a step context (or a test's stand-in for one) holds them."""
        g = lambda n, d=None: getattr(ctx, n, d)
        tensors = [ctx.positions, ctx.slots, g("entry_meta"), g("tiles"), g("tiles_small"), g("decode_rows")]
        numbers = [ctx.M, g("n_tiles", 0), g("n_tiles_small", 0), g("n_decode_rows", 0), int(bool(ctx.decode_only)),
                   g("max_context", 0), g("portion_context", 0), g("split_context", g("max_context", 0))]
        return tensors, numbers

    def attention(self, ctx, view, q, pool, out, heads, kv_heads, head_dim, scale, window):
        """Attention of every row of the step over its request's pages."""
        t, n = self._work(ctx)
        libs = ["attention_generic"] + (["attention_bf16"] if q.dtype == native.torch().bfloat16 and self.use_fast_attention else [])
        rows = [0.0, 0, 1] if getattr(ctx, "slots_are_rows", False) else []      # (unused, unused, slots[m] == m)
        self._call("attention", [q, pool, view.table, out] + t, [heads, kv_heads, head_dim, scale, int(window or 0)] + n + rows,
                   fold=(1,), libs=libs)

    def attention_from_projections(self, ctx, view, qkv, q_w, k_w, eps, inv_freq, rope_table, pool, write_kv, out, heads,
                                   kv_heads, head_dim, scale, window) -> bool:
        """`qk_norm_rope_kv_write` and `attention` in one kernel, for steps of single tokens in bfloat16.
        False if no kernel serves the step (nothing has been done then)."""
        if not self.use_fast_attention:
            return False
        t, n = self._work(ctx)
        return bool(self._call("attention_from_projections", [qkv, pool, view.table, out] + t + [q_w, k_w, inv_freq, rope_table],
                               [heads, kv_heads, head_dim, scale, int(window or 0)] + n + [eps, int(bool(write_kv))] +
                               ([1] if getattr(ctx, "slots_are_rows", False) else []),
                               fold=(1,), libs=["attention_bf16", "core"]))

    # ------------------------------------------------------------------ sampling
    def argmax(self, logits, out):
        if out.dtype != native.torch().int32 or out.shape[0] < logits.shape[0]:
            raise KernelError("argmax: logits must be contiguous float32 [n, V], out int32 [n]")
        self._call("argmax", [logits, out])

    def sample(self, logits, temperature, top_k, top_p, uniform, out):
        t = native.torch()
        n = logits.shape[0]
        for x, dt in ((temperature, t.float32), (top_k, t.int32), (top_p, t.float32), (uniform, t.float32), (out, t.int32)):
            if x.dtype != dt or x.shape[0] < n:
                raise KernelError("sample: per-row arguments must be float32/int32 [n]")
        self._call("sample", [logits, temperature, top_k, top_p, uniform, out])


# ---------------------------------------------- how the host library hands rows to the attention kernels
SERVED_HEAD_DIMS = (32, 64, 128)     # head sizes of the bfloat16 matrix-core attention kernels
MAX_SPLITS = 64                      # the merge kernel's limit
MIN_BLOCKS_PER_SPLIT = 16            # four 16-key blocks per wavefront at least


def compute_units() -> int:
    return int(get_ops()._call("compute_units", libs=["core"]))


def decode_splits(n_rows: int, kv_heads: int, heads: int, context: int, typical: int = 0, head_dim: int = 128) -> int:
    """Into how many runs the decode kernel splits the context (`Ops::decode_splits`, ops/ops.cpp)."""
    return int(native.lib().ti_decode_splits(n_rows, kv_heads, heads, context, typical or context, compute_units(), head_dim))


def portion_launch(ctx, heads: int, window: int):
    """(runs of keys, paired) for the prefill kernel with 64-row tiles (`Ops::portion_launch`)."""
    paired = ctypes.c_int()
    runs = native.lib().ti_portion_launch(ctx.n_tiles_small, heads, getattr(ctx, "portion_context", 0), int(window or 0),
                                          compute_units(), ctypes.byref(paired))
    return int(runs), bool(paired.value)


_OPS: Optional[Ops] = None


def get_ops() -> Ops:
    """An `Ops` object of the process for code that runs kernels outside an engine."""
    global _OPS
    if _OPS is None:
        _OPS = Ops()
    return _OPS
