"""Arrangements of a mixer and a feed-forward around the residual stream.

"pre_norm": x += mixer(norm(x)); x += feed_forward(norm(x)), the reference's
decoder layer (src/wllm/models/gemma.py:83-93).  The residual stream is float32.
A part's contribution is not added at once: it is left pending on the stream and
the next norm kernel adds it while it normalises, so the sum is formed in
float32 and the stream is read and written once per norm.  In a decode step of few
rows the norm kernel can fall away altogether (`ResidualStream`).
"""
from __future__ import annotations

from typing import Optional

import torch

from wllm_amd.kernels import ops
from wllm_amd.parts.common import Product
from wllm_amd.parts.registry import build_feed_forward, build_mixer, build_norm, register_block
from wllm_amd.parts.specs import BlockSpec


class ResidualStream:
    """x (float32 [n, H]) plus a contribution not yet added to it.

    Two ways lead from one part to the next.  The general one: the part's contribution (a tensor,
    or a stack of partial sums) stays pending and the next norm kernel adds it while it
    normalises.  The short one, for the few rows of a decode step: a contribution that is still a
    product (`common.Product`) is added to x by the product kernel itself, which also leaves the
    rows' sums of squares (`sumsq`); a next part that can apply the norm while it reads x
    (`takes_norm_on_load`) then needs no norm kernel at all."""

    def __init__(self, x: torch.Tensor, pending: Optional[torch.Tensor] = None):
        self.x = x
        self.pending = pending
        self.sumsq: Optional[torch.Tensor] = None      # float32 [n, bands]: sums of squares of x as it is now

    def normed(self, norm, out: torch.Tensor, rows=None) -> torch.Tensor:
        """norm(x + pending).  Without `rows` the sum becomes the new x."""
        norm.forward(self.x, out, delta=self.pending, rows=rows)
        if rows is None and self.pending is not None:
            self.pending = None
            self.sumsq = None
        return out

    def input_for(self, ctx, norm, part):
        """What `part` gets as its input: the normalised stream as a tensor, or, where the part and
        the norm allow it, the recipe to normalise it while reading (`ops.NormOnLoad`)."""
        n, hidden = self.x.shape
        if (self.pending is None and self.sumsq is not None and hasattr(norm, "on_load")
                and getattr(part, "takes_norm_on_load", lambda *a: False)(n, ctx.dtype)):
            return norm.on_load(self.x, self.sumsq, ctx.dtype)
        return self.normed(norm, ctx.buffer("normed", (n, hidden), ctx.dtype))

    def add(self, ctx, y) -> None:
        if self.pending is not None:
            raise RuntimeError("a contribution is already pending; normalise before adding another")
        if isinstance(y, Product):
            n, hidden = self.x.shape
            if ops.linear_residual_takes(n, y.x.dtype, hidden, y.x.shape[1]):
                sumsq = ctx.buffer("sumsq", ops.linear_residual_sumsq_shape(n, hidden), torch.float32)
                ops.linear_residual(y.x, y.weight, self.x, sumsq, y.tiles)
                self.sumsq = sumsq
                return
            y = y.make(ctx)
        self.pending = y


@register_block("pre_norm")
class PreNormBlock:
    def __init__(self, spec: BlockSpec):
        self.spec = spec
        self.mixer = build_mixer(spec.mixer)
        self.feed_forward = build_feed_forward(spec.feed_forward)
        self.mixer_norm = build_norm(spec.mixer_norm)
        self.feed_forward_norm = build_norm(spec.feed_forward_norm)

    def parts(self) -> list:
        return [self.mixer_norm, self.mixer, self.feed_forward_norm, self.feed_forward]

    def forward(self, ctx, entry: int, stream: ResidualStream) -> None:
        h = stream.input_for(ctx, self.mixer_norm, self.mixer)
        stream.add(ctx, self.mixer.forward(ctx, entry, h))
        h = stream.input_for(ctx, self.feed_forward_norm, self.feed_forward)
        stream.add(ctx, self.feed_forward.forward(ctx, h))
