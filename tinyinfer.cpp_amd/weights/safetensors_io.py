"""Reading and writing safetensors files.

Format: 8 bytes little-endian header length n, n bytes of JSON
`{name: {"dtype", "shape", "data_offsets": [begin, end]}, "__metadata__": {...}}`,
then the tensor bytes; offsets count from the end of the header.  (The
reference's loader made the classic mistake of treating data offsets as
file-absolute: /root/reference/docs/report.md:84-91.)

Reading maps the file and hands out tensors that alias the mapping; nothing is
executed from the file.
"""
from __future__ import annotations

import json
import mmap
import os
import struct
from typing import Dict, Iterable, List, Tuple

import numpy as np
import torch

_DTYPES = {
    "F32": (torch.float32, 4), "F16": (torch.float16, 2), "BF16": (torch.bfloat16, 2),
    "F64": (torch.float64, 8), "I64": (torch.int64, 8), "I32": (torch.int32, 4),
    "I16": (torch.int16, 2), "I8": (torch.int8, 1), "U8": (torch.uint8, 1), "BOOL": (torch.bool, 1),
}
_NAMES = {v[0]: k for k, v in _DTYPES.items()}


class SafetensorsError(ValueError):
    pass


class SafetensorsFile:
    """One mapped file: `names()`, `info(name) -> (dtype, shape)`, `tensor(name)`."""

    def __init__(self, path: str):
        self.path = path
        size = os.path.getsize(path)
        if size < 8:
            raise SafetensorsError(f"{path}: too short to be a safetensors file")
        self._f = open(path, "rb")
        (n,) = struct.unpack("<Q", self._f.read(8))
        if n <= 0 or 8 + n > size:
            raise SafetensorsError(f"{path}: header length {n} does not fit the file ({size} bytes)")
        try:
            header = json.loads(self._f.read(n).decode("utf-8"))
        except (UnicodeDecodeError, json.JSONDecodeError) as e:
            raise SafetensorsError(f"{path}: header is not JSON ({e})") from None
        self._base = 8 + n
        self.metadata = header.pop("__metadata__", {}) or {}
        self._entries: Dict[str, Tuple[torch.dtype, Tuple[int, ...], int, int]] = {}
        for name, e in header.items():
            dt = e.get("dtype")
            if dt not in _DTYPES:
                raise SafetensorsError(f"{path}: tensor '{name}' has dtype {dt!r}, which is not served")
            tdt, isz = _DTYPES[dt]
            shape = tuple(int(s) for s in e["shape"])
            b, en = (int(o) for o in e["data_offsets"])
            numel = 1
            for s in shape:
                numel *= s
            if en - b != numel * isz or b < 0 or self._base + en > size:
                raise SafetensorsError(
                    f"{path}: tensor '{name}' {dt}{list(shape)} needs {numel * isz} bytes but its "
                    f"offsets [{b}, {en}) give {en - b} (file holds {size - self._base} data bytes)")
            self._entries[name] = (tdt, shape, b, en)
        self._map = mmap.mmap(self._f.fileno(), 0, access=mmap.ACCESS_READ) if size > 0 else None

    def names(self) -> List[str]:
        return list(self._entries)

    def info(self, name: str):
        tdt, shape, _, _ = self._entries[name]
        return tdt, shape

    def tensor(self, name: str) -> torch.Tensor:
        """A CPU tensor that aliases the mapping (read-only: clone or move before writing)."""
        tdt, shape, b, e = self._entries[name]
        if e == b:
            return torch.empty(shape, dtype=tdt)
        buf = np.frombuffer(self._map, dtype=np.uint8, count=e - b, offset=self._base + b)
        import warnings
        with warnings.catch_warnings():
            warnings.simplefilter("ignore")          # numpy marks the mapping read-only
            t = torch.from_numpy(buf)
        return t.view(tdt).reshape(shape)

    def close(self):
        # tensors handed out keep the mapping alive through numpy's reference
        self._f.close()


def open_model_files(model_dir: str) -> List[SafetensorsFile]:
    """`model.safetensors`, or the shards an index file lists, or every *.safetensors."""
    single = os.path.join(model_dir, "model.safetensors")
    if os.path.isfile(single):
        return [SafetensorsFile(single)]
    index = os.path.join(model_dir, "model.safetensors.index.json")
    if os.path.isfile(index):
        with open(index, "r", encoding="utf-8") as f:
            files = sorted(set(json.load(f)["weight_map"].values()))
    else:
        files = sorted(n for n in os.listdir(model_dir) if n.endswith(".safetensors"))
    if not files:
        raise SafetensorsError(f"{model_dir}: no model.safetensors (and no other *.safetensors) in the model folder")
    return [SafetensorsFile(os.path.join(model_dir, n)) for n in files]


def write_safetensors(path: str, tensors: Dict[str, torch.Tensor], metadata: Dict[str, str] = None) -> None:
    """Write `tensors` (CPU or device; made contiguous) in the order given."""
    header = {}
    if metadata:
        header["__metadata__"] = {str(k): str(v) for k, v in metadata.items()}
    off = 0
    blobs = []
    for name, t in tensors.items():
        if t.dtype not in _NAMES:
            raise SafetensorsError(f"tensor '{name}': dtype {t.dtype} cannot be written")
        t = t.detach().to("cpu").contiguous()
        n = t.numel() * t.element_size()
        header[name] = {"dtype": _NAMES[t.dtype], "shape": list(t.shape), "data_offsets": [off, off + n]}
        off += n
        blobs.append(t)
    hj = json.dumps(header, separators=(",", ":")).encode("utf-8")
    hj += b" " * ((8 - len(hj) % 8) % 8)
    with open(path, "wb") as f:
        f.write(struct.pack("<Q", len(hj)))
        f.write(hj)
        for t in blobs:
            if t.numel():
                f.write(t.reshape(-1).view(torch.uint8).numpy().data)
