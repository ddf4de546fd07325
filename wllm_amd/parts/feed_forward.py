"""Feed-forward parts.  "gated_mlp": down(act(gate(x)) * up(x)) without biases;
with act = gelu_tanh it is the reference's GemmaMLP (src/wllm/models/gemma.py:54-62).
Gate and up matrices are stacked at load so that one product makes both halves
of the row the activation kernel reads."""
from __future__ import annotations

import torch

from wllm_amd.kernels import ops
from wllm_amd.parts.common import Product, load_matrix
from wllm_amd.parts.registry import register_feed_forward
from wllm_amd.parts.specs import GatedMLPSpec
from wllm_amd.weights.checkpoint import ExpectedTensor


@register_feed_forward("gated_mlp")
class GatedMLP:
    def __init__(self, spec: GatedMLPSpec):
        if spec.activation not in ops.ACTIVATIONS:
            raise ValueError(f"activation {spec.activation!r} is not implemented; known: {ops.ACTIVATIONS}")
        self.spec = spec
        self.w_gate_up = self.t_gate_up = None      # the matrix and its tile-major copy
        self.w_down = self.t_down = None

    def expected_tensors(self) -> dict:
        s = self.spec
        return {
            s.gate_weight: ExpectedTensor((s.intermediate_size, s.hidden_size)),
            s.up_weight: ExpectedTensor((s.intermediate_size, s.hidden_size)),
            s.down_weight: ExpectedTensor((s.hidden_size, s.intermediate_size)),
        }

    def load(self, fetch) -> None:
        s = self.spec
        self.w_gate_up, self.t_gate_up = load_matrix(
            fetch, torch.cat([fetch.matrix(s.gate_weight), fetch.matrix(s.up_weight)], dim=0), halves=2)
        self.w_down, self.t_down = load_matrix(fetch, fetch.matrix(s.down_weight))

    def flops(self, tokens: int) -> float:
        """Floating-point operations of `tokens` tokens (what a measurement divides by its time)."""
        return 6.0 * tokens * self.spec.hidden_size * self.spec.intermediate_size

    def takes_norm_on_load(self, rows: int, dtype: torch.dtype) -> bool:
        """Whether `forward` may be given `ops.NormOnLoad` instead of the normalised tensor."""
        return ops.gated_linear_norm_takes(rows, dtype, self.spec.hidden_size)

    def forward(self, ctx, h):
        s = self.spec
        n = h.shape[0]
        act = ctx.buffer("ffn_act", (n, s.intermediate_size), h.dtype)
        if isinstance(h, ops.NormOnLoad):
            ops.gated_linear(h, self.w_gate_up, act, s.activation, None, self.t_gate_up)
        else:
            gate_up = ctx.buffer("gate_up", (n, 2 * s.intermediate_size), h.dtype)
            ops.gated_linear(h, self.w_gate_up, act, s.activation, gate_up, self.t_gate_up)
        return Product("ffn_out", act, self.w_down, self.t_down)
