"""The entry point that allocates nothing: `ti_argmax_static` (csrc/sampling.hip) keeps the partial
results of the two-stage argmax in a device array of the library's own.  Called through ctypes, twice
in a row, the second time with a smaller input, it gives what `ti_argmax` gives with a workspace and
what a plain loop on the host gives (the lowest index of the largest value that is a number; 0 if a
row holds none); sizes beyond its fixed array are refused with a message."""
import ctypes

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def host_argmax(rows: np.ndarray) -> np.ndarray:
    """The rule, computed plainly: not-a-number is never chosen; among equals the lowest index; a row of
    nothing but not-a-number gives 0."""
    out = np.zeros(rows.shape[0], dtype=np.int32)
    for r, row in enumerate(rows):
        ok = np.flatnonzero(~np.isnan(row))
        if ok.size:
            out[r] = ok[np.flatnonzero(row[ok] == row[ok].max())[0]]
    return out


def test_argmax_without_allocation_matches_the_one_with_a_workspace():
    import tinyinfer_amd  # noqa: F401
    from tinyinfer_amd import native
    from tinyinfer_amd.csrc import build
    native.ensure_kernels(["sampling"])
    lib = ctypes.CDLL(build.find("sampling"))
    lib.ti_last_error.restype = ctypes.c_char_p
    lib.ti_argmax_static.restype = ctypes.c_int
    lib.ti_argmax_static.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_void_p]
    lib.ti_argmax.restype = ctypes.c_int
    lib.ti_argmax.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_void_p]
    g = torch.Generator().manual_seed(5)
    # the second call is smaller in rows and in width: what the first left in the array must not matter
    for rows, V in ((200, 151936), (7, 20011), (256, 1000), (1, 17)):
        logits = torch.randn(rows, V, generator=g)
        logits[0, V - 1] = logits[0, 3] = logits.max() + 1.0          # a tie: the lowest index wins
        if rows > 6:
            logits[2] = float("-inf")                                  # nothing but -inf: the first one
            logits[1, 5] = float("nan")
            logits[3] = float("nan")                                   # nothing that is a number: 0
            logits[4] = float("-inf")
            logits[4, :9] = float("nan")                               # the first number is a -inf at index 9
            logits[5, V // 2:] = logits[5].max() + 1.0               # half a row of equals, across the slices of the first stage
            logits[6, 0] = float("nan")
            logits[6, 1] = float("inf")
        dev = logits.cuda()
        got = torch.full((rows,), -1, dtype=torch.int32, device="cuda")
        want = torch.full((rows,), -2, dtype=torch.int32, device="cuda")
        work = torch.empty(2 * 64 * rows, dtype=torch.int32, device="cuda")
        torch.cuda.synchronize()
        rc = lib.ti_argmax_static(dev.data_ptr(), got.data_ptr(), rows, V, None)
        assert rc == 0, lib.ti_last_error().decode()
        # the kernels of ti_argmax's two-stage path, with a workspace (it takes that path from 16,384 columns
        # on; below it reads a row with one workgroup: the same choice by the same rule)
        rc = lib.ti_argmax(dev.data_ptr(), want.data_ptr(), work.data_ptr(), rows, V, None)
        assert rc == 0, lib.ti_last_error().decode()
        torch.cuda.synchronize()
        assert torch.equal(got, want), (rows, V)
        assert got[0].item() == 3
        expected = host_argmax(logits.numpy())
        assert np.array_equal(got.cpu().numpy(), expected), (rows, V, np.flatnonzero(got.cpu().numpy() != expected)[:8])
        clean = torch.nan_to_num(logits, nan=float("-inf"))
        untied = [r for r in range(rows) if (clean[r] == clean[r].max()).sum() == 1]
        assert len(untied) >= rows - 5 and torch.equal(got.cpu()[untied].long(), torch.argmax(clean[untied], dim=1))
    too_many = torch.zeros(257, 8, device="cuda")
    out = torch.empty(257, dtype=torch.int32, device="cuda")
    assert lib.ti_argmax_static(too_many.data_ptr(), out.data_ptr(), 257, 8, None) != 0
    assert "256" in lib.ti_last_error().decode()
