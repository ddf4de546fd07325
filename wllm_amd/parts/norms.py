"""Norms.  "rms": y = x * rsqrt(mean(x^2) + eps) * (weight_offset + w) in float32,
cast after the multiply.  With weight_offset 1 this is the reference's
GemmaRMSNorm (src/wllm/models/gemma.py:41-51); with 0 the plain RMSNorm.  The
kernel also adds a pending contribution to the residual stream before it
normalises, which saves one pass over the stream per norm."""
from __future__ import annotations

import torch

from wllm_amd.kernels import ops
from wllm_amd.parts.registry import register_norm
from wllm_amd.parts.specs import NormSpec
from wllm_amd.weights.checkpoint import ExpectedTensor


@register_norm("rms")
class RMSNorm:
    def __init__(self, spec: NormSpec):
        self.spec = spec
        self.weight = None

    def expected_tensors(self) -> dict:
        return {self.spec.weight: ExpectedTensor((self.spec.size,), role="vector", init="norm")}

    def load(self, fetch) -> None:
        self.weight = fetch.to_device(fetch.vector(self.spec.weight))

    def forward(self, x: torch.Tensor, out: torch.Tensor, delta=None, rows=None) -> torch.Tensor:
        ops.rms_norm(x, self.weight, self.spec.eps, self.spec.weight_offset, out, delta=delta, rows=rows)
        return out

    def on_load(self, residual: torch.Tensor, sumsq: torch.Tensor, dtype: torch.dtype):
        """This norm of `residual` as a recipe for a kernel that applies it while it reads."""
        return ops.NormOnLoad(residual, sumsq, self.weight, self.spec.eps, self.spec.weight_offset, dtype)
