"""Reading and writing of safetensors files by tensor name.

The format is an 8-byte little-endian header length, a JSON header
{name: {"dtype", "shape", "data_offsets": [begin, end]}} and the raw
little-endian tensor bytes, offsets counted from the end of the header.  The
file is memory-mapped and a tensor's bytes are copied out only when it is
asked for, so a checkpoint larger than host memory can be loaded tensor by
tensor.
"""
from __future__ import annotations

import json
import mmap
import os
import struct

import numpy as np
import torch

_DTYPES = {
    "F64": (torch.float64, np.float64, 8),
    "F32": (torch.float32, np.float32, 4),
    "F16": (torch.float16, np.float16, 2),
    "BF16": (torch.bfloat16, np.uint16, 2),
    "I64": (torch.int64, np.int64, 8),
    "I32": (torch.int32, np.int32, 4),
    "I16": (torch.int16, np.int16, 2),
    "I8": (torch.int8, np.int8, 1),
    "U8": (torch.uint8, np.uint8, 1),
    "BOOL": (torch.bool, np.bool_, 1),
}
_NAMES = {v[0]: k for k, v in _DTYPES.items()}


class SafetensorsError(ValueError):
    pass


class SafetensorsFile:
    """One file, opened for reading by name."""

    def __init__(self, path: str):
        self.path = path
        size = os.path.getsize(path)
        if size < 8:
            raise SafetensorsError(f"{path}: too short to be a safetensors file")
        self._f = open(path, "rb")
        (n,) = struct.unpack("<Q", self._f.read(8))
        if n > size - 8:
            raise SafetensorsError(f"{path}: header length {n} exceeds the file")
        try:
            header = json.loads(self._f.read(n).decode("utf-8"))
        except (UnicodeDecodeError, json.JSONDecodeError) as e:
            raise SafetensorsError(f"{path}: header is not JSON: {e}") from e
        self.metadata = header.pop("__metadata__", None) or {}
        self._base = 8 + n
        self._entries = {}
        for name, info in header.items():
            code = info.get("dtype")
            if code not in _DTYPES:
                raise SafetensorsError(f"{path}: tensor {name!r} has unsupported dtype {code!r}")
            shape = tuple(int(s) for s in info["shape"])
            begin, end = (int(x) for x in info["data_offsets"])
            count = int(np.prod(shape, dtype=np.int64)) if shape else 1
            if end - begin != count * _DTYPES[code][2] or begin < 0 or self._base + end > size:
                raise SafetensorsError(f"{path}: tensor {name!r} has inconsistent offsets or shape")
            self._entries[name] = (code, shape, begin, end)
        self._map = mmap.mmap(self._f.fileno(), 0, access=mmap.ACCESS_READ) if size > 0 else None

    def names(self) -> list[str]:
        return list(self._entries)

    def shape(self, name: str) -> tuple:
        return self._entries[name][1]

    def dtype(self, name: str) -> torch.dtype:
        return _DTYPES[self._entries[name][0]][0]

    def tensor(self, name: str) -> torch.Tensor:
        """A fresh CPU tensor in the stored dtype."""
        code, shape, begin, end = self._entries[name]
        tdt, ndt, _ = _DTYPES[code]
        raw = np.frombuffer(self._map, dtype=ndt, count=(end - begin) // np.dtype(ndt).itemsize,
                            offset=self._base + begin).copy()
        t = torch.from_numpy(raw)
        if tdt == torch.bfloat16:
            t = t.view(torch.bfloat16)
        return t.reshape(shape)

    def close(self) -> None:
        if self._map is not None:
            self._map.close()
            self._map = None
        self._f.close()


def write_safetensors(path: str, tensors: dict, metadata: dict | None = None) -> None:
    """Writes CPU tensors under their names, in the order given."""
    header = {}
    if metadata:
        header["__metadata__"] = {str(k): str(v) for k, v in metadata.items()}
    offset = 0
    blobs = []
    for name, t in tensors.items():
        t = t.detach().contiguous().cpu()
        if t.dtype not in _NAMES:
            raise SafetensorsError(f"tensor {name!r}: dtype {t.dtype} cannot be stored")
        if t.dtype == torch.bfloat16:
            raw = t.view(torch.int16).numpy().tobytes()
        else:
            raw = t.numpy().tobytes()
        header[name] = {"dtype": _NAMES[t.dtype], "shape": list(t.shape), "data_offsets": [offset, offset + len(raw)]}
        offset += len(raw)
        blobs.append(raw)
    text = json.dumps(header, separators=(",", ":")).encode("utf-8")
    text += b" " * (-len(text) % 8)
    with open(path, "wb") as f:
        f.write(struct.pack("<Q", len(text)))
        f.write(text)
        for raw in blobs:
            f.write(raw)
