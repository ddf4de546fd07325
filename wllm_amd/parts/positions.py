"""Position encodings.  "rope": inv_freq[j] = 1 / theta^(2j / rotary_dim) built in
float32 exactly as the reference builds it (src/wllm/models/llama.py:52-56); the
angle position * inv_freq[j] and its sine and cosine are computed in float32
inside the rotation kernel (llama.py:58-62), and element j is paired with
j + rotary_dim/2 (llama.py:47-49,65-71).  The table stays float32 in every
mode.  "none": no rotation."""
from __future__ import annotations

import torch

from wllm_amd.parts.registry import register_position
from wllm_amd.parts.specs import PositionSpec


@register_position("rope")
class RotaryPosition:
    def __init__(self, spec: PositionSpec):
        if spec.pairing != "half":
            raise ValueError(f"rope pairing {spec.pairing!r} is not implemented; only 'half'")
        if spec.rotary_dim <= 0 or spec.rotary_dim % 2:
            raise ValueError(f"rotary_dim must be positive and even, got {spec.rotary_dim}")
        self.spec = spec
        self.inv_freq = None

    def prepare(self, device) -> None:
        d = self.spec.rotary_dim
        inv = 1.0 / (self.spec.theta ** (torch.arange(0, d, 2, dtype=torch.float32) / d))
        self.inv_freq = inv.to(device)


@register_position("none")
class NoPosition:
    def __init__(self, spec: PositionSpec):
        self.spec = spec
        self.inv_freq = None

    def prepare(self, device) -> None:
        pass
