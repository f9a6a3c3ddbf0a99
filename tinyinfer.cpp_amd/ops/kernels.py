"""The kernels, as Python calls on torch tensors.

Each call checks devices, dtypes and shapes on the host, then launches the
hand-written HIP kernel on torch's current stream through the C ABI of the
kernel libraries (`csrc/`).  Nothing here computes with torch, and nothing falls
back to the CPU or to a library: without a GPU or without the compiled
libraries a call raises.
"""
from __future__ import annotations

import ctypes
from typing import Dict, Optional

import torch

from ..csrc import build as _build

F32, BF16 = 0, 1
EPI = {"store": 0, "add": 1, "store_act": 2, "swiglu": 3}


class KernelError(RuntimeError):
    pass


_RAW_STREAM = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _code(dt: torch.dtype) -> int:
    if dt == torch.float32:
        return F32
    if dt == torch.bfloat16:
        return BF16
    raise KernelError(f"dtype {dt} is not served by the kernels (float32, bfloat16)")


def _ptr(t: Optional[torch.Tensor]):
    """The tensor's address as a plain int (None: a null pointer).  Every library function is
    called with the argument types its declaration in tinyinfer_kernels.h gives (see
    `declare_signatures`), so no ctypes object has to be built per pointer."""
    return None if t is None else t.data_ptr()


_C_TYPES = {"int": ctypes.c_int, "long": ctypes.c_long, "float": ctypes.c_float}


def header_signatures(text: str) -> Dict[str, tuple]:
    """{function: (restype, [argtypes])} of the `int ti_...(...)` and `void ti_...(...)`
    declarations of the kernels' header: pointers and streams as void pointers, int, long and
    float as themselves.  A declaration with any other type raises."""
    import re
    text = re.sub(r"//[^\n]*", "", text)
    out = {}
    for ret, name, args in re.findall(r"\b(int|void)\s+(ti_\w+)\s*\(([^)]*)\)\s*;", text):
        types = []
        for arg in (a.strip() for a in args.split(",")):
            if not arg or arg == "void":
                continue
            if "*" in arg or arg.startswith("hipStream_t"):
                types.append(ctypes.c_void_p)
                continue
            words = [w for w in arg.replace("const", " ").split()]
            if len(words) != 2 or words[0] not in _C_TYPES:
                raise KernelError(f"tinyinfer_kernels.h: cannot read the argument {arg!r} of {name}")
            types.append(_C_TYPES[words[0]])
        out[name] = (ctypes.c_int if ret == "int" else None, types)
    return out


_signatures: Optional[Dict[str, tuple]] = None


def declare_signatures(lib: ctypes.CDLL) -> None:
    """Give every function of the header that this library exports its argument types."""
    global _signatures
    if _signatures is None:
        import os
        with open(os.path.join(_build.HERE, "tinyinfer_kernels.h")) as f:
            _signatures = header_signatures(f.read())
    for name, (restype, argtypes) in _signatures.items():
        try:
            fn = getattr(lib, name)
        except AttributeError:
            continue
        fn.restype = restype
        fn.argtypes = argtypes


class NormedRows:
    """rmsnorm(x; weight, eps) that has not been computed yet.  A norm hands this to a
    consumer that said it can take it; `Ops.linear` accepts it in place of the activation
    and runs the norm inside the product's kernel where a kernel for that exists, else
    it computes the rows first (`materialize`)."""

    def __init__(self, x: torch.Tensor, weight: torch.Tensor, eps: float, out: torch.Tensor):
        self.x, self.weight, self.eps, self.out = x, weight, eps, out
        self.shape = out.shape
        self.dtype = out.dtype
        self._done = False

    def materialize(self, ops: "Ops") -> torch.Tensor:
        if not self._done:
            ops.rmsnorm(self.x, self.weight, self.eps, self.out)
            self._done = True
        return self.out


class Ops:
    """Loads kernel libraries on first use and exposes one method per op."""

    def __init__(self):
        self._libs: Dict[str, ctypes.CDLL] = {}
        # switches for tests and measurements: force the generic kernels
        import os
        have = lambda n: os.path.isfile(os.path.join(_build.HERE, _build.SOURCES[n]))
        self.use_fast_gemm = have("gemm_bf16")
        self.use_fast_attention = have("attention_bf16")
        self.use_fused_norm = True       # the norm before a product inside the product's kernel (few tokens)
        self.use_fused_qk_decode = True  # per-head norm, rotation and cache write inside the decode attention
        self.use_fused_qkv_prefill = True  # the same in the epilogue of the q/k/v product (steps of many tokens)
        self.use_split_k_add = True          # products into the residual of few tiles: K split over workgroups
        self.use_deferred_add = True       # ... and its partial sums added by the norm that comes next
        self._partials = None
        self._pending = None               # (residual, splits): partial sums not yet added
        self.use_paired_prefill = True   # small prefill launches: a heavy and a light tile per workgroup
        self.use_portion_splits = True   # ... and the keys of a short portion against a long context cut into runs
        self.force_paired_tiles = None   # True / False: that kernel with / without pairs, whatever the launch

    # ------------------------------------------------------------------ loading
    def lib(self, name: str) -> ctypes.CDLL:
        lib = self._libs.get(name)
        if lib is None:
            if not torch.cuda.is_available():
                raise KernelError("no GPU: the kernels of this framework run on an AMD GPU (gfx950) only")
            path = _build.ensure([name])[name]
            lib = ctypes.CDLL(path)
            lib.ti_last_error.restype = ctypes.c_char_p
            declare_signatures(lib)
            self._libs[name] = lib
        return lib

    def preload(self, names):
        """Compile (if needed, several at a time) and load the libraries `names`."""
        need = [n for n in names if n not in self._libs]
        if need:
            if not torch.cuda.is_available():
                raise KernelError("no GPU: the kernels of this framework run on an AMD GPU (gfx950) only")
            _build.ensure(need)
            for n in need:
                self.lib(n)

    @staticmethod
    def _check(lib, rc, what):
        if rc != 0:
            raise KernelError(f"{what}: {lib.ti_last_error().decode()}")

    def _stream(self):
        """The current stream's handle.  Every launch asks for it; torch's raw accessor, where this
        build of torch has it, answers in well under a microsecond (the public one builds a
        Stream object: ~8 us a call).  Partial sums that a product left for later (see `flush`)
        are added first: whatever is launched next finds the residual complete."""
        if self._pending is not None:
            self.flush()
        return self._raw_stream()

    @staticmethod
    def _raw_stream():
        if _RAW_STREAM is not None:
            return _RAW_STREAM(torch.cuda.current_device()) or None      # 0, the default stream: a null pointer
        return torch.cuda.current_stream().cuda_stream or None

    def flush(self):
        """A product into the residual whose K was split over workgroups (17..64 rows, few
        columns) may leave its partial sums in a workspace, for the norm that reads the residual
        next to add on its way (`linear(..., may_defer=True)`).  Every other launch through this
        object adds them first, with a kernel of their own, in the same order: the same bits.
        Code that reads such a residual without going through this object calls `flush` itself."""
        pend, self._pending = self._pending, None
        if pend is None:
            return
        out, ks = pend
        lib = self.lib("gemm_bf16")
        rc = lib.ti_gemm_bf16_partials_add(_ptr(out), _ptr(self._partials), ks, out.numel(),
                                           self._raw_stream())
        self._check(lib, rc, "linear(bf16): adding the partial sums")

    @staticmethod
    def _dev(*ts):
        for t in ts:
            if t is not None and not t.is_cuda:
                raise KernelError("kernel arguments must live on the GPU")

    # --------------------------------------------------------------------- ops
    def embed(self, table, tokens, x):
        V, H = table.shape
        M = tokens.shape[0]
        self._dev(table, tokens, x)
        if x.shape != (M, H) or x.dtype != torch.float32 or tokens.dtype != torch.int32:
            raise KernelError(f"embed: x {tuple(x.shape)}/{x.dtype}, tokens {tokens.dtype} do not fit [{M},{H}]")
        if not (table.is_contiguous() and x.is_contiguous()):
            raise KernelError("embed: table and x must be contiguous")
        lib = self.lib("core")
        rc = lib.ti_embed(_code(table.dtype), _ptr(table), _ptr(tokens), _ptr(x), M, H, V, self._stream())
        self._check(lib, rc, "embed")

    def rmsnorm(self, x, w, eps, out, rows=None):
        H = x.shape[-1]
        n = x.shape[0] if rows is None else rows.shape[0]
        self._dev(x, w, out, rows)
        if x.dtype != torch.float32 or w.dtype != torch.float32 or w.shape != (H,):
            raise KernelError(f"rmsnorm: x {x.dtype} / weight {tuple(w.shape)} {w.dtype} do not fit width {H}")
        if out.shape != (n, H) or not out.is_contiguous() or not x.is_contiguous():
            raise KernelError(f"rmsnorm: out {tuple(out.shape)} does not fit [{n},{H}] or is not contiguous")
        if rows is not None and rows.dtype != torch.int32:
            raise KernelError("rmsnorm: rows must be int32")
        lib = self.lib("core")
        pend = self._pending
        if pend is not None and rows is None and pend[0].data_ptr() == x.data_ptr() and pend[0].shape == x.shape:
            # the product before left its partial sums: this norm adds them on its way
            rc = lib.ti_rmsnorm_add_partials(_code(out.dtype), _ptr(x), _ptr(self._partials), pend[1], _ptr(w),
                                             _ptr(out), n, H, eps, self._raw_stream())
            if rc == 0:
                self._pending = None
                return
            if rc != 3:
                self._check(lib, rc, "rmsnorm")
        rc = lib.ti_rmsnorm(_code(out.dtype), _ptr(x), _ptr(w), _ptr(rows), _ptr(out), n, H,
                            eps, self._stream())
        self._check(lib, rc, "rmsnorm")

    def rope_neox(self, x, positions, inv_freq):
        """In place on f32 x [M, heads, hd]; the last two dims contiguous, rows may be strided."""
        M, heads, hd = x.shape
        self._dev(x, positions, inv_freq)
        if x.dtype != torch.float32 or x.stride(2) != 1 or x.stride(1) != hd:
            raise KernelError("rope: x must be float32 with contiguous heads")
        if inv_freq.shape != (hd // 2,) or inv_freq.dtype != torch.float32 or positions.dtype != torch.int32:
            raise KernelError("rope: inv_freq must be float32 [hd/2], positions int32")
        lib = self.lib("core")
        rc = lib.ti_rope_neox(_ptr(x), _ptr(positions), _ptr(inv_freq), M, heads, hd,
                              x.stride(0), self._stream())
        self._check(lib, rc, "rope")

    def rope_table(self, inv_freq, n_pos):
        """float32 [n_pos, hd/2, 2] = (cos, sin)(float(p) * inv_freq[k]), computed on the device."""
        self._dev(inv_freq)
        half = inv_freq.shape[0]
        table = torch.empty((n_pos, half, 2), dtype=torch.float32, device=inv_freq.device)
        lib = self.lib("core")
        rc = lib.ti_rope_table(_ptr(table), _ptr(inv_freq), half, n_pos, self._stream())
        self._check(lib, rc, "rope_table")
        return table

    def qk_norm_rope_kv_write(self, qkv, q_w, k_w, eps, inv_freq, positions, slots, view, pool, q_out,
                              heads, kv_heads, head_dim, rope_table=None):
        """qkv f32 [M, (heads + 2 kv_heads) hd] -> q_out T [M, heads hd] and the cache pages.
        kv_heads = 0: only q (nothing is written to the cache)."""
        M = qkv.shape[0]
        width = (heads + 2 * kv_heads) * head_dim
        self._dev(qkv, q_w, k_w, inv_freq, positions, slots, view.table, pool, q_out)
        if qkv.shape != (M, width) or qkv.dtype != torch.float32 or not qkv.is_contiguous():
            raise KernelError(f"qk_norm_rope_kv_write: qkv {tuple(qkv.shape)} {qkv.dtype} does not fit [{M},{width}]")
        if q_out.shape != (M, heads * head_dim) or not q_out.is_contiguous():
            raise KernelError("qk_norm_rope_kv_write: q_out has the wrong shape")
        for wt in (q_w, k_w):
            if wt is not None and (wt.shape != (head_dim,) or wt.dtype != torch.float32):
                raise KernelError("qk_norm_rope_kv_write: norm weights must be float32 [head_dim]")
        if inv_freq is not None and (inv_freq.shape != (head_dim // 2,) or inv_freq.dtype != torch.float32):
            raise KernelError("qk_norm_rope_kv_write: inv_freq must be float32 [head_dim/2]")
        if kv_heads > 0:
            if pool.dim() != 5 or pool.shape[1] != 2 or pool.shape[2] != kv_heads or pool.shape[4] != head_dim \
                    or pool.dtype != q_out.dtype or not pool.is_contiguous():
                raise KernelError(f"qk_norm_rope_kv_write: pool {tuple(pool.shape)} {pool.dtype} does not fit "
                                  f"[pages,2,{kv_heads},P,{head_dim}] of {q_out.dtype}")
        lib = self.lib("core")
        if rope_table is not None and (rope_table.dtype != torch.float32 or not rope_table.is_contiguous()
                                       or rope_table.shape[1:] != (head_dim // 2, 2)):
            raise KernelError("qk_norm_rope_kv_write: the sin/cos table must be float32 [positions, head_dim/2, 2]")
        rc = lib.ti_qk_norm_rope_kv_write(
            _code(q_out.dtype), _ptr(qkv), _ptr(q_w), _ptr(k_w), _ptr(inv_freq), _ptr(rope_table),
            0 if rope_table is None else rope_table.shape[0], _ptr(positions), _ptr(slots),
            _ptr(view.table), view.table.shape[1], _ptr(pool), _ptr(q_out), M, heads, kv_heads, head_dim,
            pool.shape[3], eps, self._stream())
        self._check(lib, rc, "qk_norm_rope_kv_write")

    def qk_norm_inplace(self, qkv, q_w, k_w, eps, heads, kv_heads, head_dim):
        """Per-head RMSNorm of the q heads (and the k heads behind them) of f32 qkv [M, width], in
        place; a weight that is None leaves its heads alone."""
        self._dev(qkv, q_w, k_w)
        if qkv.dim() != 2 or qkv.dtype != torch.float32 or not qkv.is_contiguous() \
                or qkv.shape[1] < (heads + kv_heads) * head_dim:
            raise KernelError(f"qk_norm_inplace: qkv {tuple(qkv.shape)} {qkv.dtype} does not hold "
                              f"{heads} + {kv_heads} heads of {head_dim}")
        for wt in (q_w, k_w):
            if wt is not None and (wt.shape != (head_dim,) or wt.dtype != torch.float32):
                raise KernelError("qk_norm_inplace: norm weights must be float32 [head_dim]")
        lib = self.lib("core")
        rc = lib.ti_qk_norm_inplace(_ptr(qkv), qkv.shape[1], _ptr(q_w), _ptr(k_w), qkv.shape[0], heads, kv_heads,
                                    head_dim, eps, self._stream())
        self._check(lib, rc, "qk_norm_inplace")

    # ---------------------------------------------------------- matrix products
    def linear(self, a, w, out, epilogue: str, may_defer: bool = False):
        """out (op)= a w^T.  a: T [M, K] (rows may be strided); w: T [N, K] contiguous.
        epilogue: "store" f32 out = ; "add" f32 out += ; "store_act" T out = ;
        "swiglu": w is [2F, K] = [gate; up], T out [M, F] = silu(gate) * up.
        may_defer (with "add"): the caller reads `out` next through this object (see `flush`)."""
        epi = EPI[epilogue]
        if isinstance(a, NormedRows):
            if self._linear_normed(a, w, out, epilogue):
                return
            a = a.materialize(self)
        M, K = a.shape
        rows = w.shape[0]
        N = rows // 2 if epilogue == "swiglu" else rows
        self._dev(a, w, out)
        if w.shape[1] != K or a.dtype != w.dtype or a.stride(1) != 1 or not w.is_contiguous():
            raise KernelError(f"linear: a {tuple(a.shape)} {a.dtype} and w {tuple(w.shape)} {w.dtype} do not fit")
        if epilogue == "swiglu" and rows % 2:
            raise KernelError("linear: a SwiGLU weight needs an even number of rows")
        want = torch.float32 if epilogue in ("store", "add") else a.dtype
        if out.shape != (M, N) or out.dtype != want or not out.is_contiguous():
            raise KernelError(f"linear[{epilogue}]: out {tuple(out.shape)} {out.dtype} does not fit [{M},{N}] {want}")
        if M == 0:
            return
        code = _code(a.dtype)
        if code == BF16 and self.use_fast_gemm and self._linear_bf16(a, w, out, epi, M, N, K, may_defer):
            return
        lib = self.lib("gemm_generic")
        rc = lib.ti_gemm_generic(code, _ptr(a), _ptr(w), _ptr(out), M, N, K, a.stride(0), epi,
                                 self._stream())
        self._check(lib, rc, "linear")

    def qkv_prepared(self, a, w, q_w, k_w, eps, inv_freq, rope_table, positions, slots, view, pool, q_out,
                     heads, kv_heads, head_dim) -> bool:
        """`linear(a, w, qkv, "store")` and `qk_norm_rope_kv_write` in one kernel, for steps of many
        tokens in bfloat16: w is [(heads + 2 kv_heads) hd, K] (kv_heads = 0: q heads only).  False if
        no kernel serves the step; then nothing has been done and the caller makes the two calls."""
        if not (self.use_fused_qkv_prefill and self.use_fast_gemm) or isinstance(a, NormedRows):
            return False
        if a.dtype != torch.bfloat16 or w.dtype != torch.bfloat16 or q_out.dtype != torch.bfloat16:
            return False
        M, K = a.shape
        N = (heads + 2 * kv_heads) * head_dim
        self._dev(a, w, q_w, k_w, inv_freq, rope_table, positions, slots, view.table, pool, q_out)
        if w.shape != (N, K) or a.stride(1) != 1 or not w.is_contiguous():
            raise KernelError(f"qkv_prepared: a {tuple(a.shape)} and w {tuple(w.shape)} do not fit {N} rows of heads")
        if q_out.shape != (M, heads * head_dim) or not q_out.is_contiguous():
            raise KernelError("qkv_prepared: q_out has the wrong shape")
        if positions.shape[0] != M or slots.shape[0] != M or positions.dtype != torch.int32 or slots.dtype != torch.int32:
            raise KernelError("qkv_prepared: positions and slots must be int32 [M]")
        for wt in (q_w, k_w):
            if wt is not None and (wt.shape != (head_dim,) or wt.dtype != torch.float32):
                raise KernelError("qkv_prepared: norm weights must be float32 [head_dim]")
        if inv_freq is not None and (inv_freq.shape != (head_dim // 2,) or inv_freq.dtype != torch.float32):
            raise KernelError("qkv_prepared: inv_freq must be float32 [head_dim/2]")
        if rope_table is not None and (rope_table.dtype != torch.float32 or not rope_table.is_contiguous()
                                       or rope_table.shape[1:] != (head_dim // 2, 2)):
            raise KernelError("qkv_prepared: the sin/cos table must be float32 [positions, head_dim/2, 2]")
        if kv_heads > 0 and (pool.dim() != 5 or pool.shape[1] != 2 or pool.shape[2] != kv_heads
                             or pool.shape[4] != head_dim or pool.dtype != torch.bfloat16
                             or not pool.is_contiguous() or not view.table.is_contiguous()):
            raise KernelError(f"qkv_prepared: pool {tuple(pool.shape)} {pool.dtype} does not fit "
                              f"[pages,2,{kv_heads},P,{head_dim}] of bfloat16")
        lib = self.lib("gemm_bf16")
        rc = lib.ti_gemm_bf16_qkv_prep(
            _ptr(a), _ptr(w), M, K, a.stride(0), _ptr(q_w), _ptr(k_w), eps,
            _ptr(inv_freq), _ptr(rope_table), 0 if rope_table is None else rope_table.shape[0],
            _ptr(positions), _ptr(slots), _ptr(view.table), view.table.shape[1], _ptr(pool), _ptr(q_out),
            heads, kv_heads, head_dim, pool.shape[3], self._stream())
        if rc == 3:
            return False
        self._check(lib, rc, "qkv_prepared")
        return True

    NORMED_MAX_ROWS = 16
    PARTIALS_BYTES = 4 << 20

    def can_fuse_norm(self, n_rows: int, dtype: torch.dtype) -> bool:
        """Whether `linear` has a kernel that takes the norm of this many rows in."""
        return (self.use_fused_norm and self.use_fast_gemm and dtype == torch.bfloat16
                and 0 < n_rows <= self.NORMED_MAX_ROWS)

    def _linear_normed(self, a: NormedRows, w, out, epilogue) -> bool:
        """rmsnorm and product in one kernel; False if no kernel serves the shape."""
        M, K = a.shape
        if not self.can_fuse_norm(M, a.dtype) or w.dtype != torch.bfloat16:
            return False
        rows = w.shape[0]
        N = rows // 2 if epilogue == "swiglu" else rows
        self._dev(a.x, a.weight, w, out)
        if w.dim() != 2 or w.shape[1] != K or not w.is_contiguous() or (epilogue == "swiglu" and rows % 2):
            raise KernelError(f"linear: normed rows {tuple(a.shape)} and w {tuple(w.shape)} do not fit")
        if a.x.shape != (M, K) or a.x.dtype != torch.float32 or not a.x.is_contiguous() \
                or a.weight.shape != (K,) or a.weight.dtype != torch.float32:
            raise KernelError("linear: the rows to norm must be float32 [M, K] with a float32 weight [K]")
        want = torch.float32 if epilogue in ("store", "add") else torch.bfloat16
        if out.shape != (M, N) or out.dtype != want or not out.is_contiguous():
            raise KernelError(f"linear[{epilogue}]: out {tuple(out.shape)} {out.dtype} does not fit [{M},{N}] {want}")
        lib = self.lib("gemm_bf16")
        rc = lib.ti_gemm_bf16_normed(_ptr(a.x), _ptr(a.weight), a.eps, _ptr(w), _ptr(out),
                                     M, N, K, EPI[epilogue], self._stream())
        if rc == 3:
            return False
        self._check(lib, rc, "linear(normed)")
        return True

    def _linear_bf16(self, a, w, out, epi, M, N, K, may_defer=False) -> bool:
        """The MFMA kernels; False if they refuse the shape (the generic kernel takes it)."""
        if K % 8 or a.stride(0) % 8 or a.data_ptr() % 16 or w.data_ptr() % 16:
            return False
        lib = self.lib("gemm_bf16")
        if M > 16 and epi == EPI["add"] and self.use_split_k_add:
            # a product of few tiles: K split over workgroups; their sums go through a workspace
            stream = self._stream()
            ws = self._partials
            if ws is None or ws.device != a.device:
                ws = self._partials = torch.empty(self.PARTIALS_BYTES // 4, dtype=torch.float32, device=a.device)
            # 1: the sums are left for the next norm; 2: the same product, added at once
            defer = 0 if not may_defer else 1 if self.use_deferred_add else 2
            splits = ctypes.c_int(0)
            rc = lib.ti_gemm_bf16_add_split(_ptr(a), _ptr(w), _ptr(out), M, N, K, a.stride(0), epi, _ptr(ws),
                                            self.PARTIALS_BYTES, defer, ctypes.byref(splits), stream)
            if rc == 0:
                if splits.value:
                    self._pending = (out, splits.value)
                return True
            if rc != 3:
                self._check(lib, rc, "linear(bf16, split K)")
        rc = lib.ti_gemm_bf16(_ptr(a), _ptr(w), _ptr(out), M, N, K, a.stride(0), epi, self._stream())
        if rc == 3:          # "shape not served": not an error
            return False
        self._check(lib, rc, "linear(bf16)")
        return True

    # ----------------------------------------------------------------- attention
    def attention_rows(self, q, pool, table, positions, slots, out, heads, kv_heads, head_dim, scale, window):
        M = q.shape[0]
        self._dev(q, pool, table, positions, slots, out)
        if q.shape != (M, heads * head_dim) or out.shape != q.shape or q.dtype != pool.dtype or out.dtype != q.dtype:
            raise KernelError("attention: q/out/pool shapes or dtypes do not fit")
        if pool.dim() != 5 or pool.shape[1] != 2 or pool.shape[2] != kv_heads or pool.shape[4] != head_dim:
            raise KernelError(f"attention: pool {tuple(pool.shape)} does not fit [pages,2,{kv_heads},P,{head_dim}]")
        if not (q.is_contiguous() and out.is_contiguous() and pool.is_contiguous() and table.is_contiguous()):
            raise KernelError("attention: arguments must be contiguous")
        lib = self.lib("attention_generic")
        rc = lib.ti_attention_rows(_code(q.dtype), _ptr(q), _ptr(pool), _ptr(table), table.shape[1],
                                   _ptr(positions), _ptr(slots), _ptr(out), M, heads, kv_heads, head_dim,
                                   pool.shape[3], scale, int(window or 0), self._stream())
        self._check(lib, rc, "attention")

    def attention(self, ctx, view, q, pool, out, heads, kv_heads, head_dim, scale, window):
        """Attention of every row of the step over its request's pages."""
        if q.dtype == torch.bfloat16 and self.use_fast_attention:
            from . import attention_bf16
            if attention_bf16.run(self, ctx, view, q, pool, out, heads, kv_heads, head_dim, scale, window):
                return
        self.attention_rows(q, pool, view.table, ctx.positions, ctx.slots, out, heads, kv_heads, head_dim,
                            scale, window)

    def attention_from_projections(self, ctx, view, qkv, q_w, k_w, eps, inv_freq, rope_table, pool, write_kv,
                                   out, heads, kv_heads, head_dim, scale, window) -> bool:
        """`qk_norm_rope_kv_write` and `attention` in one kernel, for steps of single tokens
        in bfloat16: qkv f32 [M, (heads + 2 kv_heads) hd] (only the q heads if not write_kv).
        False if no kernel serves the step; then nothing has been done and the caller
        makes the two calls."""
        if not (self.use_fused_qk_decode and self.use_fast_attention and ctx.decode_only
                and pool.dtype == torch.bfloat16):
            return False
        M = qkv.shape[0]
        width = (heads + (2 * kv_heads if write_kv else 0)) * head_dim
        self._dev(qkv, q_w, k_w, inv_freq, rope_table, pool, view.table, out)
        if qkv.dim() != 2 or qkv.shape[1] < width or qkv.dtype != torch.float32 or not qkv.is_contiguous():
            raise KernelError(f"attention_from_projections: qkv {tuple(qkv.shape)} {qkv.dtype} does not fit "
                              f"[{M}, >= {width}] float32")
        if out.shape != (M, heads * head_dim) or out.dtype != torch.bfloat16 or not out.is_contiguous():
            raise KernelError("attention_from_projections: out has the wrong shape or dtype")
        if pool.dim() != 5 or pool.shape[1] != 2 or pool.shape[2] != kv_heads or pool.shape[4] != head_dim \
                or not pool.is_contiguous() or not view.table.is_contiguous():
            raise KernelError(f"attention_from_projections: pool {tuple(pool.shape)} does not fit "
                              f"[pages,2,{kv_heads},P,{head_dim}]")
        for wt in (q_w, k_w):
            if wt is not None and (wt.shape != (head_dim,) or wt.dtype != torch.float32):
                raise KernelError("attention_from_projections: norm weights must be float32 [head_dim]")
        if inv_freq is not None and (inv_freq.shape != (head_dim // 2,) or inv_freq.dtype != torch.float32):
            raise KernelError("attention_from_projections: inv_freq must be float32 [head_dim/2]")
        if rope_table is not None and (rope_table.dtype != torch.float32 or not rope_table.is_contiguous()
                                       or rope_table.shape[1:] != (head_dim // 2, 2)):
            raise KernelError("attention_from_projections: the sin/cos table must be float32 [positions, head_dim/2, 2]")
        from . import attention_bf16
        return attention_bf16.run_decode_prepared(self, ctx, view, qkv, q_w, k_w, eps, inv_freq, rope_table, pool,
                                                  write_kv, out, heads, kv_heads, head_dim, scale, window)

    # ------------------------------------------------------------------ sampling
    def argmax(self, logits, out):
        n, V = logits.shape
        self._dev(logits, out)
        if logits.dtype != torch.float32 or not logits.is_contiguous() or out.dtype != torch.int32 or out.shape[0] < n:
            raise KernelError("argmax: logits must be contiguous float32 [n, V], out int32 [n]")
        scratch = getattr(self, "_argmax_scratch", None)
        if scratch is None or scratch.numel() < 2 * 64 * n:
            scratch = self._argmax_scratch = torch.empty(2 * 64 * max(n, 64), dtype=torch.int32, device=logits.device)
        lib = self.lib("sampling")
        rc = lib.ti_argmax(_ptr(logits), _ptr(out), _ptr(scratch), n, V, self._stream())
        self._check(lib, rc, "argmax")

    def sample(self, logits, temperature, top_k, top_p, uniform, out):
        n, V = logits.shape
        self._dev(logits, temperature, top_k, top_p, uniform, out)
        if logits.dtype != torch.float32 or not logits.is_contiguous():
            raise KernelError("sample: logits must be contiguous float32 [n, V]")
        for t, dt in ((temperature, torch.float32), (top_k, torch.int32), (top_p, torch.float32),
                      (uniform, torch.float32), (out, torch.int32)):
            if t.dtype != dt or t.shape[0] < n:
                raise KernelError("sample: per-row arguments must be float32/int32 [n]")
        lib = self.lib("sampling")
        rc = lib.ti_sample(_ptr(logits), _ptr(temperature), _ptr(top_k), _ptr(top_p), _ptr(uniform), _ptr(out),
                           n, V, self._stream())
        self._check(lib, rc, "sample")


_OPS: Optional[Ops] = None


def get_ops() -> Ops:
    global _OPS
    if _OPS is None:
        _OPS = Ops()
    return _OPS
