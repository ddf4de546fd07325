"""Helpers shared by parts."""
from __future__ import annotations

from typing import Optional

import torch

from wllm_amd.kernels import ops


def project(ctx, name: str, x: torch.Tensor, weight: torch.Tensor, out: Optional[torch.Tensor] = None,
            tiles: Optional[torch.Tensor] = None) -> torch.Tensor:
    """x @ weight^T into the step's scratch.  Where the product kernel splits these sizes over the
    input axis, the result is the float32 stack of partial sums [S, n, out] for a consumer that adds
    them as it reads (the next norm, the rotation); else the plain result [n, out], in `out` if given.
    `tiles` is the weight's tile-major copy (`load_matrix`), if one was made."""
    n, width = x.shape[0], weight.shape[0]
    splits = ops.linear_splits(n, width, x.shape[1], x.dtype)
    if splits > 1:
        stack = ctx.buffer(name + "_parts", (splits, n, width), torch.float32)
        ops.linear(x, weight, stack, tiles)
        return stack
    if out is None:
        out = ctx.buffer(name, (n, width), x.dtype)
    ops.linear(x, weight, out, tiles)
    return out


class Product:
    """A part's contribution to the residual stream that is still a product to be made:
    x @ weight^T.  The stream it is added to chooses how: into the stream at once by a kernel that
    also leaves what the next norm needs (`ops.linear_residual`), or as a tensor (or a stack of
    partial sums) that the next norm kernel adds."""

    def __init__(self, name: str, x: torch.Tensor, weight: torch.Tensor, tiles: Optional[torch.Tensor] = None):
        self.name, self.x, self.weight, self.tiles = name, x, weight, tiles

    def make(self, ctx) -> torch.Tensor:
        return project(ctx, self.name, self.x, self.weight, tiles=self.tiles)


def load_matrix(fetch, matrix: torch.Tensor, halves: int = 1):
    """A weight matrix on the device as the product kernels want it: (the matrix, row by row, for
    products of many rows; its tile-major copy for the few rows of a decode step, or None).  The
    copy doubles the weight's memory and is made only where the loader asks for it
    (`fetch.tiled_copies`) and the few-row kernels take the weight (bfloat16 with an input size that
    is a multiple of 32, float32 with a multiple of 4)."""
    weight = fetch.to_device(matrix)
    tiles = ops.tile_weight(weight, halves) if getattr(fetch, "tiled_copies", False) else None
    return weight, tiles
