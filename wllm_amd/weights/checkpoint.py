"""A model folder's tensors by name, checked against what the model expects.

The reference merges every *.safetensors file of a folder into one dict and
reports missing and unexpected names after `load_state_dict(strict=False)`
(src/wllm/models/llama.py:640-649).  Here the model's parts say which names and
shapes they expect, and `Checkpoint.check` raises one `WeightError` that lists
all missing tensors, all unexpected tensors and all wrong shapes together.
"""
from __future__ import annotations

import glob
import json
import os
from dataclasses import dataclass

import torch

from wllm_amd.weights.safetensors_io import SafetensorsError, SafetensorsFile


class WeightError(RuntimeError):
    """The checkpoint does not hold what the model needs."""

    def __init__(self, message: str, missing=(), unexpected=(), wrong_shape=(), wrong_dtype=()):
        super().__init__(message)
        self.missing = list(missing)
        self.unexpected = list(unexpected)
        self.wrong_shape = list(wrong_shape)
        self.wrong_dtype = list(wrong_dtype)


@dataclass(frozen=True)
class ExpectedTensor:
    shape: tuple
    # "matrix": takes the model's dtype; "vector": used in float32 arithmetic and
    # kept in float32 on the device (exact for bfloat16 and float32 storage alike);
    # "table": integers, kept as int32
    role: str = "matrix"
    optional: bool = False
    # how the random-weights mode draws it: "weight" (normal, std) or "norm" (normal, norm_std)
    init: str = "weight"


_FLOATS = (torch.float32, torch.bfloat16, torch.float16, torch.float64)
_INTS = (torch.int64, torch.int32, torch.int16, torch.int8, torch.uint8)


class Checkpoint:
    def __init__(self, folder: str):
        self.folder = folder
        index = os.path.join(folder, "model.safetensors.index.json")
        if os.path.isfile(index):
            with open(index, "r", encoding="utf-8") as f:
                files = sorted(set(json.load(f).get("weight_map", {}).values()))
            for p in files:
                # the index is part of an untrusted folder: it names files of that folder, nothing else
                if not isinstance(p, str) or os.path.basename(p) != p or not p.endswith(".safetensors"):
                    raise WeightError(f"{index}: weight_map names {p!r}; expected the plain name of a "
                                      f".safetensors file in the same folder")
            paths = [os.path.join(folder, p) for p in files]
        else:
            paths = sorted(glob.glob(os.path.join(folder, "*.safetensors")))
        if not paths:
            raise WeightError(f"no *.safetensors file in {folder!r}")
        self._files = []
        self._where = {}
        duplicates = []
        for p in paths:
            if not os.path.isfile(p):
                raise WeightError(f"{p}: named by the index but not present")
            try:
                f = SafetensorsFile(p)
            except SafetensorsError as e:
                raise WeightError(str(e)) from e
            self._files.append(f)
            for name in f.names():
                if name in self._where:
                    duplicates.append(name)
                self._where[name] = f
        if duplicates:
            raise WeightError(f"tensor(s) stored in more than one file: {sorted(duplicates)}")

    def names(self) -> list[str]:
        return list(self._where)

    def __contains__(self, name: str) -> bool:
        return name in self._where

    def shape(self, name: str) -> tuple:
        return self._where[name].shape(name)

    def stored_dtype(self, name: str) -> torch.dtype:
        return self._where[name].dtype(name)

    def tensor(self, name: str) -> torch.Tensor:
        return self._where[name].tensor(name)

    def check(self, expected: dict, ignored_suffixes: tuple = (), allowed_extra: tuple = ()) -> None:
        """Raises one WeightError that lists everything wrong, or returns."""
        missing, wrong_shape, wrong_dtype = [], [], []
        for name, exp in expected.items():
            if name not in self._where:
                if not exp.optional:
                    missing.append(name)
                continue
            shape = self.shape(name)
            if tuple(shape) != tuple(exp.shape):
                wrong_shape.append((name, tuple(shape), tuple(exp.shape)))
            dt = self.stored_dtype(name)
            ok = dt in _INTS if exp.role == "table" else dt in _FLOATS
            if not ok:
                wrong_dtype.append((name, str(dt)))
        unexpected = [n for n in self._where
                      if n not in expected and n not in allowed_extra
                      and not any(n.endswith(s) for s in ignored_suffixes)]
        if missing or unexpected or wrong_shape or wrong_dtype:
            lines = [f"checkpoint {self.folder!r} does not match the model:"]
            if missing:
                lines.append(f"  missing tensors ({len(missing)}): {sorted(missing)}")
            if unexpected:
                lines.append(f"  unexpected tensors ({len(unexpected)}): {sorted(unexpected)}")
            if wrong_shape:
                lines.append(f"  wrong shapes ({len(wrong_shape)}): " + "; ".join(
                    f"{n}: stored {list(s)}, expected {list(e)}" for n, s, e in sorted(wrong_shape)))
            if wrong_dtype:
                lines.append(f"  wrong dtypes ({len(wrong_dtype)}): " + "; ".join(
                    f"{n}: {d}" for n, d in sorted(wrong_dtype)))
            raise WeightError("\n".join(lines), missing, unexpected, wrong_shape, wrong_dtype)

    def close(self) -> None:
        for f in self._files:
            f.close()


class TensorFetcher:
    """What a part's `load` receives: tensors by name, converted for their role.

    Matrices take the model's dtype.  Vectors that enter float32 arithmetic are
    kept in float32 (the conversion from bfloat16 is exact, and a tensor stored in
    32 bits stays so).  Integer tables are kept as int32.
    """

    def __init__(self, checkpoint: Checkpoint, dtype: torch.dtype, device, tiled_copies: bool = False):
        self.checkpoint = checkpoint
        self.dtype = dtype
        self.device = device
        # whether parts keep a second, tile-major copy of each matrix for the few-row product kernels
        self.tiled_copies = tiled_copies

    def has(self, name: str) -> bool:
        return name in self.checkpoint

    def matrix(self, name: str) -> torch.Tensor:
        return self.checkpoint.tensor(name).to(self.dtype)

    def vector(self, name: str) -> torch.Tensor:
        return self.checkpoint.tensor(name).to(torch.float32)

    def table(self, name: str) -> torch.Tensor:
        return self.checkpoint.tensor(name).to(torch.int32)

    def to_device(self, t: torch.Tensor) -> torch.Tensor:
        return t.contiguous().to(self.device)
