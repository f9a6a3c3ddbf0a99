"""What the kernels' host side decides.  The argument types that Python gives the kernel libraries
(tests that call one kernel) come from the declarations in tinyinfer_kernels.h: pointers are passed as
plain ints, which ctypes would cut to 32 bits for a function without declared types.  And the number of
runs the decode attention cuts a context into."""
import ctypes
import os
import re

import tinyinfer_amd  # noqa: F401
from tinyinfer_amd.csrc import build
from tinyinfer_amd.ops import kernels


def header_text():
    with open(os.path.join(build.HERE, "tinyinfer_kernels.h")) as f:
        return f.read()


def test_every_kernel_the_host_library_calls_is_declared():
    """ops.cpp resolves kernels by name (`KERNEL("lib", ti_fn)`) with the type of the header's declaration:
    a name the header does not declare would not compile.  Here: every such name is in the header, and the
    library it is looked up in is one the build knows."""
    declared = kernels.header_signatures(header_text())
    with open(os.path.join(os.path.dirname(build.HERE), "ops", "ops.cpp")) as f:
        used = re.findall(r'KERNEL\("(\w+)",\s*(ti_\w+)\)', f.read())
    assert len(used) > 15, "the pattern of this test is out of date"
    for lib, fn in used:
        assert fn in declared, fn
        assert lib in build.SOURCES, lib


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
    with open(os.path.join(build.HERE, "tinyinfer_kernels_tuning.h")) as f:
        tuning = kernels.header_signatures(f.read())
    assert tuning["ti_tuning_set"] == (ctypes.c_int, [ctypes.c_void_p, ctypes.c_long]) and tuning["ti_tuning_reset"] == (None, [])
    assert sig["ti_fill_random"][1][6] is ctypes.c_ulong
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
    from tinyinfer_amd.ops import kernels as a
    monkeypatch.setattr(a, "compute_units", lambda: 256)
    assert a.decode_splits(8, 8, 16, 4096, 2112) == 4          # 256 workgroups
    assert a.decode_splits(12, 8, 16, 4096, 2112) == 2         # 192, not 288
    assert a.decode_splits(24, 8, 16, 4096, 2112) == 1         # 192 in one round, and no merge
    assert a.decode_splits(64, 8, 16, 4096, 2112) == 1
    assert a.decode_splits(1, 8, 16, 4096, 2112) == 16         # bounded: 16 blocks of 16 keys a run at least
    assert a.decode_splits(1, 8, 16, 100, 100) == 1            # a short context is not split
    assert a.decode_splits(1, 1, 64, 10 ** 6, 10 ** 6) <= a.MAX_SPLITS
    # half the bytes per token (head size 64): a run is worth its prologue only if twice as long
    assert a.decode_splits(12, 8, 16, 4096, 2112, head_dim=64) <= a.decode_splits(12, 8, 16, 4096, 2112)
    for rows in range(1, 70):
        for context in (300, 2000, 9000, 40000):
            s = a.decode_splits(rows, 8, 16, context)
            assert 1 <= s <= max(1, min(-(-context // 16) // a.MIN_BLOCKS_PER_SPLIT, a.MAX_SPLITS))
