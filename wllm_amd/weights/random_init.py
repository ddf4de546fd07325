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
