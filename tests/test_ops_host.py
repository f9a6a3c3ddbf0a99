"""What the kernels' Python side decides on the host.  The argument types that Python gives the kernel
libraries come from the declarations in tinyinfer_kernels.h: pointers are passed as plain ints,
which ctypes would cut to 32 bits for a function without declared types.  And the number of runs the
decode attention cuts a context into."""
import ctypes
import os
import re

import tinyinfer_amd  # noqa: F401
from tinyinfer_amd.csrc import build
from tinyinfer_amd.ops import kernels


def header_text():
    with open(os.path.join(build.HERE, "tinyinfer_kernels.h")) as f:
        return f.read()


def test_every_function_python_calls_is_declared():
    declared = kernels.header_signatures(header_text())
    ops_dir = os.path.dirname(kernels.__file__)
    called = set()
    for name in os.listdir(ops_dir):
        if name.endswith(".py"):
            with open(os.path.join(ops_dir, name)) as f:
                called |= set(re.findall(r"lib\.(ti_\w+)\(", f.read()))
    called.discard("ti_last_error")
    assert called, "no calls found: the pattern of this test is out of date"
    assert not called - set(declared), f"called but not declared in the header: {sorted(called - set(declared))}"


def test_declarations_are_read_as_written():
    sig = kernels.header_signatures(header_text())
    restype, args = sig["ti_rmsnorm"]
    # int ti_rmsnorm(int out_dtype, const float* x, const float* w, const int* rows, void* out, int n_rows, int H,
    #                float eps, hipStream_t stream)
    assert restype is ctypes.c_int
    assert args == [ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int,
                    ctypes.c_int, ctypes.c_float, ctypes.c_void_p]
    restype, args = sig["ti_gemm_bf16"]
    assert args[6] is ctypes.c_long and args[-1] is ctypes.c_void_p and len(args) == 9
    assert sig["ti_gemm_bf16_force_tile"] == (None, [ctypes.c_int])
    # what the call sites pass for such arguments is accepted
    assert ctypes.c_void_p.from_param(None) is None
    ctypes.c_void_p.from_param(ctypes.byref(ctypes.c_int(0)))
    ctypes.c_void_p.from_param(1 << 45)
    ctypes.c_long.from_param(ctypes.c_long(5))
    ctypes.c_float.from_param(ctypes.c_float(1.0))


def test_a_declaration_with_an_unknown_type_is_refused():
    import pytest
    with pytest.raises(kernels.KernelError):
        kernels.header_signatures("int ti_x(double y);")


def test_context_splits_of_the_decode_kernel(monkeypatch):
    """The number of runs the decode attention cuts the context into: bounded by the context the
    launch is sized for, chosen for the typical one, and never just beyond a whole round of the
    compute units when fewer runs fill one round (12 rows x 8 kv heads: 2 runs, not 3)."""
    from tinyinfer_amd.ops import attention_bf16 as a
    monkeypatch.setattr(a, "compute_units", lambda: 256)
    assert a.decode_splits(8, 8, 16, 4096, 2112) == 4          # 256 workgroups
    assert a.decode_splits(12, 8, 16, 4096, 2112) == 2         # 192, not 288
    assert a.decode_splits(24, 8, 16, 4096, 2112) == 1         # 192 in one round, and no merge
    assert a.decode_splits(64, 8, 16, 4096, 2112) == 1
    assert a.decode_splits(1, 8, 16, 4096, 2112) == 16         # bounded: 16 blocks of 16 keys a run at least
    assert a.decode_splits(1, 8, 16, 100, 100) == 1            # a short context is not split
    assert a.decode_splits(1, 1, 64, 10 ** 6, 10 ** 6) <= a.MAX_SPLITS
    for rows in range(1, 70):
        for context in (300, 2000, 9000, 40000):
            s = a.decode_splits(rows, 8, 16, context)
            assert 1 <= s <= max(1, min(-(-context // 16) // a.MIN_BLOCKS_PER_SPLIT, a.MAX_SPLITS))
