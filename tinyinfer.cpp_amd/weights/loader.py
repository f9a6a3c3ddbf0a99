"""Weights by tensor name, from a model folder or from a dict of tensors.

Every fault of a checkpoint is reported in one error: tensors the model asks
for and the files lack, tensors the files hold and nothing asks for, and
tensors of the wrong shape (the full shape is compared; the reference compares
element counts only, /root/reference/src/model.cpp:74-80,104-109, so a
transposed matrix would pass there).

Dtypes on the device, by the role a part gives the tensor:
  matrix  the engine's compute dtype: bfloat16 stays bfloat16 under
          --dtype bfloat16; under float32 every matrix is widened (exactly)
  vector  float32 (norm weights take part in 32-bit arithmetic only)
  table   int32
A matrix stored in 32-bit is rounded to bfloat16 only when the engine runs in
bfloat16, and a line on stderr says so.
"""
from __future__ import annotations

import sys
from typing import Dict, Mapping, Union

import torch

from .safetensors_io import open_model_files

DTYPES = {"bfloat16": torch.bfloat16, "float32": torch.float32}


class WeightsError(ValueError):
    def __init__(self, where, missing, unexpected, wrong_shape, wrong_dtype=()):
        self.missing = list(missing)
        self.unexpected = list(unexpected)
        self.wrong_shape = list(wrong_shape)
        self.wrong_dtype = list(wrong_dtype)
        lines = [f"{where}: the weights do not fit the model"]
        if self.missing:
            lines.append(f"  missing ({len(self.missing)}): " + ", ".join(self.missing))
        if self.unexpected:
            lines.append(f"  unexpected ({len(self.unexpected)}): " + ", ".join(self.unexpected))
        if self.wrong_shape:
            lines.append(f"  wrong shape ({len(self.wrong_shape)}): " + ", ".join(
                f"{n} is {list(got)}, expected {list(want)}" for n, got, want in self.wrong_shape))
        if self.wrong_dtype:
            lines.append(f"  wrong dtype ({len(self.wrong_dtype)}): " + ", ".join(
                f"{n} is {got}, expected {want}" for n, got, want in self.wrong_dtype))
        super().__init__("\n".join(lines))


def _target_dtype(role: str, compute: torch.dtype) -> torch.dtype:
    if role == "matrix":
        return compute
    if role == "vector":
        return torch.float32
    if role == "table":
        return torch.int32
    raise ValueError(f"unknown tensor role {role!r}")


def load_weights(model, source: Union[str, Mapping[str, torch.Tensor]], dtype: str = "bfloat16",
                 device: Union[str, torch.device] = "cuda") -> None:
    """Check `source` against `model.tensors()` and hand every part its tensors."""
    if dtype not in DTYPES:
        raise ValueError(f"dtype must be one of {sorted(DTYPES)}, got {dtype!r}")
    compute = DTYPES[dtype]
    needs = model.tensors()

    if isinstance(source, str):
        files = open_model_files(source)
        where = source
        info: Dict[str, tuple] = {}
        owner = {}
        for f in files:
            for n in f.names():
                info[n] = f.info(n)
                owner[n] = f
        fetch = lambda n: owner[n].tensor(n)
    else:
        files = []
        where = "weights"
        info = {n: (t.dtype, tuple(t.shape)) for n, t in source.items()}
        fetch = lambda n: source[n]

    missing = [n for n, need in needs.items() if n not in info and not need.optional]
    unexpected = [n for n in info if n not in needs]
    wrong_shape = [(n, info[n][1], need.shape) for n, need in needs.items()
                   if n in info and tuple(info[n][1]) != tuple(need.shape)]
    wrong_dtype = []
    for n, need in needs.items():
        if n not in info:
            continue
        dt = info[n][0]
        if need.role == "table":
            if dt.is_floating_point:
                wrong_dtype.append((n, dt, "an integer type"))
        elif not dt.is_floating_point:
            wrong_dtype.append((n, dt, "a floating-point type"))
    if missing or unexpected or wrong_shape or wrong_dtype:
        raise WeightsError(where, missing, unexpected, wrong_shape, wrong_dtype)

    rounded = []
    loaded: Dict[str, torch.Tensor] = {}
    for n, need in needs.items():
        if n not in info:
            continue
        t = fetch(n)
        want = _target_dtype(need.role, compute)
        if need.role == "matrix" and want == torch.bfloat16 and t.dtype in (torch.float32, torch.float64):
            rounded.append(n)
        # move first, convert on the device: one pass over the bytes on the host
        t = t.to(device)
        if t.dtype != want:
            t = t.to(want)
        elif t.device.type == "cpu" and isinstance(source, str):
            t = t.clone()            # do not keep aliasing the file mapping
        loaded[n] = t.contiguous()
    if rounded:
        print(f"[tinyinfer] {len(rounded)} matrices stored in 32-bit are rounded to bfloat16 for "
              f"--dtype bfloat16 (first: {rounded[0]})", file=sys.stderr)

    for part in model.parts():
        mine = {n: loaded[n] for n in part.tensors() if n in loaded}
        part.load(mine)
    for f in files:
        f.close()
