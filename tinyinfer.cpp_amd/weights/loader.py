"""Weights by tensor name, from a model folder or from a dict of tensors.

Checking and loading are the host library's (weights/weights.cpp): every fault of
a checkpoint is reported in one error (missing, unexpected, wrong shape, wrong
kind of dtype), tensors go straight into the parts' own (fused) buffers, and the
dtype on the device follows the role a part gives the tensor:
  matrix  the engine's compute dtype: bfloat16 stays bfloat16 under
          --dtype bfloat16; under float32 every matrix is widened (exactly)
  vector  float32 (norm weights take part in 32-bit arithmetic only)
  table   int32
A matrix stored in 32-bit is rounded to bfloat16 only when the engine runs in
bfloat16, and a line on stderr says so.
"""
from __future__ import annotations

from typing import Mapping, Union

from .. import native
from ..native import WeightsError as _NativeWeightsError

DTYPES = ("bfloat16", "float32")


class WeightsError(_NativeWeightsError):
    """`wrong_shape` holds (name, shape found, shape expected); `str()` lists everything."""


def _parse_shapes(items):
    out = []
    for text in items:
        # "<name> is [a, b], expected [c, d]"
        name, rest = text.split(" is ", 1)
        got, want = rest.split(", expected ")
        out.append((name, tuple(int(v) for v in got.strip("[]").split(",") if v.strip()),
                    tuple(int(v) for v in want.strip("[]").split(",") if v.strip())))
    return out


def _raise(e: _NativeWeightsError):
    raise WeightsError(str(e), e.missing, e.unexpected, _parse_shapes(e.wrong_shape), e.wrong_dtype) from None


def load_weights(model, source: Union[str, Mapping[str, "object"]], dtype: str = "bfloat16", device="cuda") -> None:
    """Check `source` (a model folder, or torch tensors by name) against what the model asks for and
    load it.  device "cpu": the weights stay in host memory, to be looked at (such a model cannot run)."""
    if dtype not in DTYPES:
        raise ValueError(f"dtype must be one of {sorted(DTYPES)}, got {dtype!r}")
    to_host = str(device) == "cpu"
    if not to_host:
        native.use_torch_allocator()
    try:
        if isinstance(source, str):
            native.call("ti_model_load_folder", model._ptr, source.encode(), dtype.encode(), int(to_host))
        else:
            names = list(source)
            ts = [source[n].contiguous() for n in names]
            on_device = bool(ts) and ts[0].is_cuda
            if on_device:
                # on the device a tensor must have the dtype its role asks for already
                t = native.torch()
                want = {"matrix": t.bfloat16 if dtype == "bfloat16" else t.float32, "vector": t.float32, "table": t.int32}
                needs = model.tensors()
                ts = [x.to(want[needs[n].role]) if n in needs else x for n, x in zip(names, ts)]
            native.call("ti_model_load_tensors", model._ptr, len(ts), "\n".join(names).encode(), native.describe_many(ts),
                        int(on_device), dtype.encode(), b"weights", int(to_host))
    except _NativeWeightsError as e:
        _raise(e)
    model.dtype = None if to_host else dtype
