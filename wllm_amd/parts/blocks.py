"""Arrangements of a mixer and a feed-forward around the residual stream.

"pre_norm": x += mixer(norm(x)); x += feed_forward(norm(x)), the reference's
decoder layer (src/wllm/models/gemma.py:83-93).  The residual stream is float32.
A part's contribution is not added at once: it is left pending on the stream and
the next norm kernel adds it while it normalises, so the sum is formed in
float32 and the stream is read and written once per norm.
"""
from __future__ import annotations

from typing import Optional

import torch

from wllm_amd.parts.registry import build_feed_forward, build_mixer, build_norm, register_block
from wllm_amd.parts.specs import BlockSpec


class ResidualStream:
    """x (float32 [n, H]) plus a contribution not yet added to it."""

    def __init__(self, x: torch.Tensor, pending: Optional[torch.Tensor] = None):
        self.x = x
        self.pending = pending

    def normed(self, norm, out: torch.Tensor, rows=None) -> torch.Tensor:
        """norm(x + pending).  Without `rows` the sum becomes the new x."""
        norm.forward(self.x, out, delta=self.pending, rows=rows)
        if rows is None:
            self.pending = None
        return out

    def add(self, y: torch.Tensor) -> None:
        if self.pending is not None:
            raise RuntimeError("a contribution is already pending; normalise before adding another")
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
        n, hidden = stream.x.shape
        h = stream.normed(self.mixer_norm, ctx.buffer("normed", (n, hidden), ctx.dtype))
        stream.add(self.mixer.forward(ctx, entry, h))
        h = stream.normed(self.feed_forward_norm, ctx.buffer("normed", (n, hidden), ctx.dtype))
        stream.add(self.feed_forward.forward(ctx, h))
