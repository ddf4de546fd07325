"""Random weights: writes a model folder (config.json, model.safetensors) from a
configuration and a seed.

Each tensor is drawn from a generator keyed by (seed, tensor name), so the values
do not depend on the order in which tensors are made.  Matrices (and biases) are
normal(0, std); norm weights are normal(0, norm_std), stored as the checkpoint
stores them (for Gemma: the offset w of (1 + w)).  Values are rounded to bfloat16
before storage, so a float32 run and a bfloat16 run of the same folder use the
same numbers.
"""
from __future__ import annotations

import hashlib
import json
import os

import torch

from wllm_amd.weights.safetensors_io import write_safetensors


def _generator(seed: int, name: str) -> torch.Generator:
    digest = hashlib.sha256(f"{seed}:{name}".encode("utf-8")).digest()
    g = torch.Generator(device="cpu")
    g.manual_seed(int.from_bytes(digest[:8], "little") & 0x7FFF_FFFF_FFFF_FFFF)
    return g


def random_tensor(seed: int, name: str, shape: tuple, std: float,
                  store_dtype: torch.dtype = torch.bfloat16) -> torch.Tensor:
    t = torch.randn(tuple(shape), generator=_generator(seed, name), dtype=torch.float32) * std
    return t.to(torch.bfloat16).to(store_dtype)


def write_random_model(folder: str, config_json: dict, expected: dict, seed: int, *,
                       std: float = 0.02, norm_std: float = 0.1,
                       store_dtype: torch.dtype = torch.bfloat16) -> str:
    """`expected` is the model's {tensor name: ExpectedTensor}; optional tensors
    are left out.  Returns the folder."""
    os.makedirs(folder, exist_ok=True)
    tensors = {}
    for name, exp in expected.items():
        if exp.optional:
            continue
        if exp.role == "table":
            raise ValueError(f"{name}: no random initialisation for integer tables")
        s = norm_std if exp.init == "norm" else std
        tensors[name] = random_tensor(seed, name, exp.shape, s, store_dtype)
    write_safetensors(os.path.join(folder, "model.safetensors"), tensors,
                      metadata={"format": "pt", "seed": seed})
    with open(os.path.join(folder, "config.json"), "w", encoding="utf-8") as f:
        json.dump(config_json, f, indent=1, sort_keys=True)
    return folder


class RandomFetcher:
    """Random weights made on the device, for measurements at sizes whose folder would be
    many gigabytes: the same distributions as `write_random_model`, drawn by the device's
    generator (so not the same numbers as a written folder of that seed)."""

    def __init__(self, expected: dict, seed: int, dtype: torch.dtype, device, std: float = 0.02,
                 norm_std: float = 0.1, tiled_copies: bool = False):
        self.expected, self.dtype, self.device = expected, dtype, torch.device(device)
        self.tiled_copies = tiled_copies
        self.std, self.norm_std = std, norm_std
        self._gen = torch.Generator(device=self.device)
        self._seed = seed

    def has(self, name: str) -> bool:
        return name in self.expected and not self.expected[name].optional

    def _draw(self, name: str, dtype: torch.dtype) -> torch.Tensor:
        exp = self.expected[name]
        digest = hashlib.sha256(f"{self._seed}:{name}".encode("utf-8")).digest()
        self._gen.manual_seed(int.from_bytes(digest[:8], "little") & 0x7FFF_FFFF_FFFF_FFFF)
        t = torch.empty(tuple(exp.shape), dtype=torch.bfloat16, device=self.device)
        t.normal_(0.0, self.norm_std if exp.init == "norm" else self.std, generator=self._gen)
        return t.to(dtype)

    def matrix(self, name: str) -> torch.Tensor:
        return self._draw(name, self.dtype)

    def vector(self, name: str) -> torch.Tensor:
        return self._draw(name, torch.float32)

    def to_device(self, t: torch.Tensor) -> torch.Tensor:
        return t.contiguous().to(self.device)
