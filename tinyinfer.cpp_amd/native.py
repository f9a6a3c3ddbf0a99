"""The binding to the host library (`libtinyinfer`, the C interface at the end of
include/inference.h) through ctypes: loading and building it, errors as Python
exceptions, torch tensors as tensor descriptors and back, torch's allocator as
the library's source of device memory, and the call table through which the
library runs parts that are defined in Python.

Nothing here computes.  Configuration, weights, parts, cache manager, step
function, scheduler and sampler are the library's; the Python package names
them and hands tensors across.
"""
from __future__ import annotations

import bisect
import ctypes
import json
import threading
import traceback
from typing import Any, Dict, List, Optional, Sequence

from .csrc import build as _build

c_int, c_i64, c_u64, c_void_p, c_char_p, c_float, c_double, c_size_t = (
    ctypes.c_int, ctypes.c_int64, ctypes.c_uint64, ctypes.c_void_p, ctypes.c_char_p, ctypes.c_float,
    ctypes.c_double, ctypes.c_size_t)
P = ctypes.POINTER


class ti_tensor(ctypes.Structure):
    _fields_ = [("data", c_void_p), ("dtype", c_int), ("ndim", c_int), ("shape", c_i64 * 4), ("stride", c_i64 * 4)]


# ------------------------------------------------------------------------ errors
class Error(RuntimeError):
    pass


class ConfigError(ValueError):
    """A config.json that this framework cannot serve; the text names the key."""


class CacheError(Error):
    pass


class OutOfPages(CacheError):
    """A reservation that the free pages cannot cover.  Nothing was taken."""


class EngineError(Error):
    pass


class SchedulerError(Error):
    pass


class KernelError(Error):
    pass


class FileError(ValueError):
    """A model folder or weights file that cannot be read."""


class WeightsError(ValueError):
    """The weights do not fit the model: every fault in one error."""

    def __init__(self, message, missing=(), unexpected=(), wrong_shape=(), wrong_dtype=()):
        super().__init__(message)
        self.missing, self.unexpected = list(missing), list(unexpected)
        self.wrong_shape, self.wrong_dtype = list(wrong_shape), list(wrong_dtype)


_ERRORS = {"ConfigError": ConfigError, "CacheError": CacheError, "OutOfPages": OutOfPages, "EngineError": EngineError,
           "SchedulerError": SchedulerError, "KernelError": KernelError, "FileError": FileError, "Error": Error}

FOREIGN_CALL = ctypes.CFUNCTYPE(c_int, c_u64, c_char_p, c_void_p, P(ti_tensor), c_int, c_char_p, P(ti_tensor))
ALLOC = ctypes.CFUNCTYPE(c_void_p, c_void_p, c_size_t)
RELEASE = ctypes.CFUNCTYPE(None, c_void_p, c_void_p)
FOREIGN_MAKE = ctypes.CFUNCTYPE(c_int, c_char_p, c_char_p, c_char_p, c_char_p, c_int, P(c_char_p), P(c_void_p), P(c_void_p))
ON_TOKEN = ctypes.CFUNCTYPE(c_int, c_i64, c_int)
ON_LOGITS = ctypes.CFUNCTYPE(c_int, c_i64, P(c_float), c_i64)

_OUT_TEXT = P(c_char_p)
_OUT_PTR = P(c_void_p)
_TT = P(ti_tensor)
_SIGNATURES = {
    "ti_kernels_register": [c_char_p, c_char_p],
    "ti_load_plugin": [c_char_p],
    "ti_set_allocator": [ALLOC, RELEASE, c_void_p],
    "ti_set_foreign_calls": [FOREIGN_CALL],
    "ti_qwen3_config": [c_char_p, _OUT_TEXT],
    "ti_typed_config": [c_char_p, _OUT_TEXT],
    "ti_set_foreign_factory": [FOREIGN_MAKE],
    "ti_register_foreign_kind": [c_char_p, c_char_p, c_char_p],
    "ti_part_child": [c_void_p, c_int, _OUT_PTR],
    "ti_model_from_spec": [c_char_p, _OUT_PTR],
    "ti_model_part": [c_void_p, c_char_p, c_int, _OUT_PTR],
    "ti_spec_from_config": [c_char_p, _OUT_TEXT],
    "ti_architecture_registered": [c_char_p, P(c_int)],
    "ti_registered_architectures": [_OUT_TEXT],
    "ti_registered_parts": [c_char_p, _OUT_TEXT],
    "ti_block_slots": [c_char_p, _OUT_TEXT],
    "ti_part_create": [c_char_p, c_char_p, c_char_p, c_char_p, c_int, P(c_char_p), P(c_void_p), _OUT_PTR],
    "ti_part_create_foreign": [c_char_p, c_u64, c_char_p, c_char_p, c_int, P(c_char_p), P(c_void_p), _OUT_PTR],
    "ti_part_tensors": [c_void_p, _OUT_TEXT],
    "ti_part_cache_need": [c_void_p, _OUT_TEXT],
    "ti_part_info": [c_void_p, _OUT_TEXT],
    "ti_part_held": [c_void_p, c_char_p, _TT],
    "ti_part_pointer": [c_void_p, _OUT_PTR],
    "ti_part_load": [c_void_p, c_int, c_char_p, _TT, c_char_p, c_int],
    "ti_ctx_create": [c_char_p, c_void_p, _OUT_PTR],
    "ti_ctx_set_rows": [c_void_p, c_i64, c_void_p, c_void_p],
    "ti_part_call": [c_void_p, c_char_p, c_void_p, _TT, c_int, c_int, _TT],
    "ti_ctx_info": [c_void_p, _OUT_TEXT],
    "ti_ctx_pointers": [c_void_p, _OUT_PTR, _OUT_PTR, _OUT_PTR],
    "ti_ctx_binding": [c_void_p, c_void_p, P(c_int), P(c_int)],
    "ti_ctx_kv_pool": [c_void_p, c_int, c_int, _TT],
    "ti_ctx_state": [c_void_p, c_int, c_int, _TT],
    "ti_ctx_cache_view": [c_void_p, c_int, _TT, P(c_int)],
    "ti_ctx_buf": [c_void_p, c_char_p, c_int, c_int, P(c_i64), _TT],
    "ti_ctx_ops": [c_void_p, _OUT_PTR],
    "ti_model_create": [c_char_p, c_void_p, c_int, P(c_void_p), c_void_p, c_void_p, _OUT_PTR],
    "ti_model_tensors": [c_void_p, _OUT_TEXT],
    "ti_model_cache_groups": [c_void_p, _OUT_TEXT],
    "ti_model_bindings": [c_void_p, _OUT_TEXT],
    "ti_model_load_folder": [c_void_p, c_char_p, c_char_p, c_int],
    "ti_model_load_tensors": [c_void_p, c_int, c_char_p, _TT, c_int, c_char_p, c_char_p, c_int],
    "ti_model_load_random": [c_void_p, c_u64, c_char_p],
    "ti_model_write_random_folder": [c_void_p, c_char_p, c_char_p, c_u64, c_char_p],
    "ti_weights_error_lists": [_OUT_TEXT],
    "ti_cache_create": [c_char_p, c_int, c_int, c_int, c_int, c_int, _OUT_PTR],
    "ti_cache_call": [c_void_p, c_char_p, c_i64, c_i64, c_i64, P(c_i64)],
    "ti_cache_table": [c_void_p, c_int, c_i64, _OUT_TEXT],
    "ti_cache_many": [c_void_p, c_char_p, c_int, P(c_i64), _OUT_TEXT],
    "ti_cache_dump": [c_void_p, _OUT_TEXT],
    "ti_pool_create": [c_int, c_int, _OUT_PTR],
    "ti_pool_call": [c_void_p, c_char_p, c_i64, P(c_i64)],
    "ti_pool_free_list": [c_void_p, _OUT_TEXT],
    "ti_engine_create": [c_void_p, c_char_p, _OUT_PTR],
    "ti_engine_info": [c_void_p, _OUT_TEXT],
    "ti_engine_cache": [c_void_p, _OUT_PTR],
    "ti_engine_ops": [c_void_p, _OUT_PTR],
    "ti_engine_step": [c_void_p, c_int, c_int, P(c_i64), P(c_int), P(c_int), P(c_int), P(c_int), _TT],
    "ti_engine_release_request": [c_void_p, c_i64],
    "ti_engine_kv_pool": [c_void_p, c_int, c_int, _TT],
    "ti_engine_state": [c_void_p, c_int, c_int, _TT],
    "ti_engine_synchronize": [c_void_p],
    "ti_sampler_create": [c_void_p, _OUT_PTR],
    "ti_sampler_sample": [c_void_p, _TT, c_int, P(c_float), P(c_int), P(c_float), P(c_u64), P(c_i64), P(c_i64), P(c_int)],
    "ti_sampler_sample_async": [c_void_p, _TT, c_int, P(c_float), P(c_int), P(c_float), P(c_u64), P(c_i64), P(c_i64), c_void_p,
                                P(c_u64)],
    "ti_sampler_collect": [c_void_p, c_u64, c_int, P(c_int)],
    "ti_scheduler_create": [c_void_p, c_int, c_int, c_int, _OUT_PTR],
    "ti_scheduler_add": [c_void_p, c_int, P(c_int), c_int, c_float, c_int, c_float, c_u64, c_int, P(c_int), P(c_i64)],
    "ti_scheduler_plan": [c_void_p, _OUT_TEXT],
    "ti_scheduler_plan_ahead": [c_void_p, _OUT_TEXT],
    "ti_scheduler_commit": [c_void_p, c_int, P(c_i64), P(c_int), _OUT_TEXT],
    "ti_scheduler_abort": [c_void_p, c_i64],
    "ti_scheduler_set_next_number": [c_void_p, c_i64],
    "ti_scheduler_state": [c_void_p, _OUT_TEXT],
    "ti_scheduler_request": [c_void_p, c_i64, _OUT_TEXT],
    "ti_run_requests": [c_void_p, c_void_p, c_void_p, c_int, c_int, ON_TOKEN, ON_LOGITS, _OUT_TEXT],
    "ti_ops_create": [c_void_p, _OUT_PTR],
    "ti_ops_switch": [c_void_p, c_char_p, c_int, P(c_int)],
    "ti_ops_timing_report": [c_void_p, _OUT_TEXT],
    "ti_ops_call": [c_void_p, c_char_p, _TT, c_int, P(c_double), c_int, c_char_p, _TT],
}
_VOID = {"ti_part_release": [c_void_p], "ti_ctx_release": [c_void_p], "ti_model_release": [c_void_p],
         "ti_cache_release": [c_void_p], "ti_pool_release": [c_void_p], "ti_engine_release": [c_void_p],
         "ti_sampler_release": [c_void_p], "ti_scheduler_release": [c_void_p], "ti_ops_release": [c_void_p],
         "ti_set_foreign_error": [c_char_p]}

_lib: Optional[ctypes.CDLL] = None
_lock = threading.Lock()


def lib() -> ctypes.CDLL:
    """The host library, compiled at the first call if it is not there."""
    global _lib
    if _lib is not None:
        return _lib
    # torch brings a HIP runtime of its own: it has to be in the process before this library's
    # dependency on one is resolved, or two runtimes meet
    torch()
    with _lock:
        if _lib is not None:
            return _lib
        handle = ctypes.CDLL(_build.ensure_host())
        for name, args in _SIGNATURES.items():
            fn = getattr(handle, name)
            fn.restype = c_int
            fn.argtypes = args
        for name, args in _VOID.items():
            fn = getattr(handle, name)
            fn.restype = None
            fn.argtypes = args
        handle.ti_error_kind.restype = c_char_p
        handle.ti_error_message.restype = c_char_p
        handle.ti_uniform.restype = c_float
        handle.ti_uniform.argtypes = [c_u64, c_u64, c_u64]
        handle.ti_decode_splits.restype = c_int
        handle.ti_decode_splits.argtypes = [c_int] * 7
        handle.ti_portion_launch.restype = c_int
        handle.ti_portion_launch.argtypes = [c_int] * 5 + [P(c_int)]
        handle.ti_detach_allocator.restype = None
        handle.ti_set_foreign_calls(_foreign_trampoline)
        handle.ti_set_foreign_factory(_foreign_make_trampoline)
        _lib = handle
        # kernel libraries that are built already are made known; the others when they are asked for
        for name in _build.SOURCES:
            path = _build.find(name)
            if path:
                handle.ti_kernels_register(name.encode(), path.encode())
                _registered.add(name)
    return _lib


_registered = set()


def load_plugin(path: str) -> None:
    """Open a shared library that registers parts, architectures or kernel libraries with the host library
    (`tinyinfer::load_plugin`): a model made of them then builds, loads and steps like any other."""
    call("ti_load_plugin", path.encode())


def ensure_kernels(names: Sequence[str]) -> None:
    """Compile (if needed, several at a time) the kernel libraries `names` and tell the host library where they are."""
    need = [n for n in names if n not in _registered]
    if not need:
        return
    handle = lib()
    need = [n for n in names if n not in _registered]
    paths = _build.ensure(need)
    _build.write_manifest()
    for n in need:
        check(handle.ti_kernels_register(n.encode(), paths[n].encode()))
        _registered.add(n)


def check(rc: int) -> None:
    if rc == 0:
        return
    handle = _lib
    kind = handle.ti_error_kind().decode()
    message = handle.ti_error_message().decode(errors="replace")
    if kind == "WeightsError":
        out = c_char_p()
        handle.ti_weights_error_lists(ctypes.byref(out))
        lists = json.loads(out.value.decode())
        raise WeightsError(message, lists["missing"], lists["unexpected"], lists["wrong_shape"], lists["wrong_dtype"])
    raise _ERRORS.get(kind, Error)(message)


def text(name: str, *args) -> str:
    """Call a function whose last argument is a string result."""
    out = c_char_p()
    check(getattr(lib(), name)(*args, ctypes.byref(out)))
    return out.value.decode()


def pointer(name: str, *args) -> int:
    """Call a function whose last argument is a pointer result."""
    out = c_void_p()
    check(getattr(lib(), name)(*args, ctypes.byref(out)))
    return out.value


def call(name: str, *args) -> None:
    check(getattr(lib(), name)(*args))


def enc(s: Optional[str]) -> Optional[bytes]:
    return None if s is None else s.encode()


# --------------------------------------------------------------------- tensors
_TORCH = None
_CODES: Dict[Any, int] = {}
_DTYPES: Dict[int, Any] = {}


def torch():
    global _TORCH
    if _TORCH is None:
        import torch as t
        _TORCH = t
        for code, dt in enumerate((t.float32, t.bfloat16, t.int32, t.float16, t.float64, t.int64)):
            _CODES[dt] = code
            _DTYPES[code] = dt
    return _TORCH


def dtype_code(dt) -> int:
    torch()
    if dt not in _CODES:
        raise KernelError(f"dtype {dt} cannot cross into the library (float32, bfloat16, int32, float16, float64, int64)")
    return _CODES[dt]


def describe(t, fold_pool: bool = False) -> ti_tensor:
    """The descriptor of a torch tensor (None: an undefined tensor).  `fold_pool`: a cache pool
    [pages, 2, kv heads, P, hd] crosses as [pages, 2 x kv heads, P, hd] (a descriptor has four dims)."""
    d = ti_tensor()
    if t is None:
        return d
    if fold_pool and t.dim() == 5:
        if not t.is_contiguous():
            raise KernelError("a cache pool must be contiguous")
        t = t.view(t.shape[0], t.shape[1] * t.shape[2], t.shape[3], t.shape[4])
    if t.dim() > 4:
        raise KernelError(f"a tensor of {t.dim()} dimensions cannot cross into the library (at most 4)")
    d.data = t.data_ptr()
    d.dtype = dtype_code(t.dtype)
    d.ndim = t.dim()
    for i in range(t.dim()):
        d.shape[i] = t.shape[i]
        d.stride[i] = t.stride(i)
    return d


def describe_many(ts: Sequence, fold: Sequence[int] = ()):
    arr = (ti_tensor * max(1, len(ts)))()
    for i, t in enumerate(ts):
        arr[i] = describe(t, i in fold)
    return arr


# Device memory of the library comes from torch's allocator: every allocation is a uint8 tensor
# kept here until the library gives it back, and any pointer into one can be seen as a tensor.
_allocs: Dict[int, Any] = {}
_starts: List[int] = []
_alloc_lock = threading.Lock()
_allocator_set = False


@ALLOC
def _alloc(_user, nbytes):
    t = torch().empty(max(int(nbytes), 4), dtype=torch().uint8, device="cuda")
    p = t.data_ptr()
    with _alloc_lock:
        _allocs[p] = t
        bisect.insort(_starts, p)
    return p


@RELEASE
def _release(_user, p):
    with _alloc_lock:
        if _allocs.pop(p, None) is not None:
            i = bisect.bisect_left(_starts, p)
            if i < len(_starts) and _starts[i] == p:
                del _starts[i]


def use_torch_allocator() -> None:
    """From now on the library's device memory is torch's (called before the first device allocation)."""
    global _allocator_set
    if not _allocator_set:
        import atexit
        call("ti_set_allocator", _alloc, _release, None)
        # what the library still holds when the interpreter ends is not handed back through Python
        atexit.register(lambda: _lib.ti_detach_allocator())
        _allocator_set = True


def _owner(ptr: int):
    with _alloc_lock:
        i = bisect.bisect_right(_starts, ptr) - 1
        if i >= 0:
            base = _allocs[_starts[i]]
            if ptr < _starts[i] + base.numel():
                return base
    return None


def wrap(d: ti_tensor, keep=None):
    """A torch tensor over the memory a descriptor names (None for an undefined one): a view of the
    allocation it lies in, or, for host memory of the library, a tensor over that memory.  `keep`:
    an object that owns the memory, kept alive by the tensor."""
    if not d.data:
        return None
    t = torch()
    dt = _DTYPES[d.dtype]
    shape = [d.shape[i] for i in range(d.ndim)]
    stride = [d.stride[i] for i in range(d.ndim)]
    extent = 1 + sum((s - 1) * st for s, st in zip(shape, stride)) if all(s > 0 for s in shape) else 0
    item = t.empty(0, dtype=dt).element_size()
    base = _owner(d.data)
    if base is not None:
        off = d.data - base.data_ptr()
        flat = base[off:off + extent * item].view(dt)
    else:
        buf = (ctypes.c_char * max(1, extent * item)).from_address(d.data)
        flat = t.frombuffer(buf, dtype=dt, count=extent)
        if keep is not None:
            flat._ti_keep = keep
    return t.as_strided(flat, shape, stride)


def wrap_pool(d: ti_tensor, kv_heads: int):
    """A cache pool as [pages, 2, kv heads, P, hd]."""
    t = wrap(d)
    return t.view(t.shape[0], 2, kv_heads, t.shape[2], t.shape[3])


# ---------------------------------------------------------------- foreign parts
_foreign_parts: Dict[int, Any] = {}
_foreign_next = [1]
_contexts: Dict[int, Any] = {}


def register_foreign(part) -> int:
    i = _foreign_next[0]
    _foreign_next[0] += 1
    _foreign_parts[i] = part
    return i


def foreign_object(part_id: int):
    """The Python part behind a part of the library that is implemented here."""
    return _foreign_parts[part_id]


def forget_contexts() -> None:
    """The step is over: what its Python-side contexts kept alive may go."""
    _contexts.clear()


def _python_context(ctx_ptr: int):
    ctx = _contexts.get(ctx_ptr)
    if ctx is None:
        from .engine.context import StepContext
        ctx = _contexts[ctx_ptr] = StepContext(ctx_ptr)
    return ctx


def _dispatch(part, op: str, ctx_ptr, args, n_args: int, names: Optional[bytes], result) -> None:
    tensors = [wrap(args[i]) for i in range(n_args)]
    if op == "load":
        part.load(dict(zip(names.decode().split("\n"), tensors)) if n_args else {})
        return
    if op == "prepare":
        if hasattr(part, "prepare"):
            from .ops.kernels import get_ops
            part.prepare(get_ops(), int(names.decode()))
        return
    ctx = _python_context(ctx_ptr)
    family = part.family
    out = None
    if op == "apply":
        part.apply(ctx, tensors[0], tensors[1] if n_args > 1 else None)
    elif family == "embedding":
        part.forward(ctx, ctx.tokens, tensors[0])
    elif family == "norm":
        out = part.forward(ctx, tensors[0], rows=tensors[1] if n_args > 1 else None)
        if hasattr(out, "materialize"):
            out = out.materialize(ctx.ops)
    elif family in ("mixer", "ffn"):
        part.forward(ctx, tensors[0], tensors[1])
    elif family == "block":
        part.forward(ctx, tensors[0])
    elif family == "head":
        out = part.forward(ctx, tensors[0])
    else:
        raise Error(f"a {family} part has no call {op!r}")
    if out is not None:
        ctx._keep.append(out)                 # the library reads it after this call returns
        result[0] = describe(out.contiguous() if not out.is_contiguous() else out)
    ctx.ops.flush()


@FOREIGN_CALL
def _foreign_trampoline(part_id, op, ctx_ptr, args, n_args, names, result):
    try:
        _dispatch(_foreign_parts[part_id], op.decode(), ctx_ptr, args, n_args, names, result)
        return 0
    except BaseException as e:  # noqa: BLE001  (an exception must not unwind through the library)
        _lib.ti_set_foreign_error(f"{type(e).__name__}: {e}\n{traceback.format_exc()}".encode())
        return 1


@FOREIGN_MAKE
def _foreign_make_trampoline(family, kind, prefix, params_json, n_children, slots, children, out):
    """The library builds a model and comes to a kind that was registered from Python: make the part here and
    hand back the library's part behind it."""
    try:
        from .parts.base import part_handle
        from .parts.registry import make_registered
        kids = [(slots[i].decode(), children[i]) for i in range(n_children)]
        part = make_registered(family.decode(), kind.decode(), prefix.decode(), json.loads(params_json.decode()), kids)
        out[0] = part_handle(part).ptr
        return 0
    except BaseException as e:  # noqa: BLE001  (an exception must not unwind through the library)
        _lib.ti_set_foreign_error(f"{type(e).__name__}: {e}\n{traceback.format_exc()}".encode())
        return 1
