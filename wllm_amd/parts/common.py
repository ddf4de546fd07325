"""Helpers shared by parts."""
from __future__ import annotations

from typing import Optional

import torch

from wllm_amd.kernels import ops


def project(ctx, name: str, x: torch.Tensor, weight: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """x @ weight^T into the step's scratch.  Where the product kernel splits these sizes over the
    input axis, the result is the float32 stack of partial sums [S, n, out] for a consumer that adds
    them as it reads (the next norm, the rotation); else the plain result [n, out], in `out` if given."""
    n, width = x.shape[0], weight.shape[0]
    splits = ops.linear_splits(n, width, x.shape[1], x.dtype)
    if splits > 1:
        stack = ctx.buffer(name + "_parts", (splits, n, width), torch.float32)
        ops.linear(x, weight, stack)
        return stack
    if out is None:
        out = ctx.buffer(name, (n, width), x.dtype)
    ops.linear(x, weight, out)
    return out
