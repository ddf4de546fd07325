"""Registries of part kinds: norm, position encoding, mixer, feed-forward, block.

A part is a class built from its specification alone.  It says which checkpoint
tensors it expects, loads them, and runs on the flat batch of a step.  The
interfaces:

norm          expected_tensors(); load(fetch); forward(x, out, delta=None, rows=None)
position      prepare(device); `inv_freq`: float32 [rotary_dim / 2] that the mixer's rotation kernels
              turn queries and keys by, or None; optionally `apply(ctx, qkv, *, num_heads,
              num_kv_heads, head_dim)`, a step of its own on the projected rows [tokens,
              (heads + 2 kv heads) * head_dim] in place (positions in `ctx.positions`) before keys
              are cached, for encodings that are no rotation; optionally `expected_tensors()`
              and `load(fetch)` for tensors of its own
mixer         expected_tensors(); load(fetch); cache_need() -> CacheNeed | None;
              state_shape() -> tuple | None; forward(ctx, entry, h) -> y
feed-forward  expected_tensors(); load(fetch); forward(ctx, h) -> y
block         built from a BlockSpec and the parts above; forward(ctx, entry, stream)

`ctx` is the step's `StepContext`, `entry` the index of the schedule entry being
run, `h` the normalised input [tokens, hidden] in the activation dtype, `y` the
part's contribution to the residual stream: a tensor of the same shape and dtype, a
float32 stack of partial sums [S, tokens, hidden], or a `common.Product` (a last
product x @ W^T that the stream makes itself).  A part that defines
`takes_norm_on_load(rows, dtype) -> bool` may be given `ops.NormOnLoad` as `h` when it
says yes: the recipe of the norm, for a kernel that applies it while it reads.
"""
from __future__ import annotations

_NORMS: dict = {}
_POSITIONS: dict = {}
_MIXERS: dict = {}
_FEED_FORWARDS: dict = {}
_BLOCKS: dict = {}


def _register(table: dict, what: str):
    def register(kind: str, cls=None, *, replace: bool = False):
        def add(c):
            if kind in table and not replace:
                raise ValueError(f"{what} kind {kind!r} is already registered")
            table[kind] = c
            return c
        return add(cls) if cls is not None else add
    return register


def _build(table: dict, what: str):
    def build(spec, *args, **kwargs):
        kind = spec.kind if hasattr(spec, "kind") else spec.arrangement
        if kind not in table:
            raise ValueError(f"unknown {what} kind {kind!r}; registered: {sorted(table)}")
        return table[kind](spec, *args, **kwargs)
    return build


register_norm = _register(_NORMS, "norm")
register_position = _register(_POSITIONS, "position encoding")
register_mixer = _register(_MIXERS, "mixer")
register_feed_forward = _register(_FEED_FORWARDS, "feed-forward")
register_block = _register(_BLOCKS, "block arrangement")

build_norm = _build(_NORMS, "norm")
build_position = _build(_POSITIONS, "position encoding")
build_mixer = _build(_MIXERS, "mixer")
build_feed_forward = _build(_FEED_FORWARDS, "feed-forward")
build_block = _build(_BLOCKS, "block arrangement")
