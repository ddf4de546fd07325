"""The operations the parts are made of, each one a hand-written gfx950 kernel.

Every function checks on the host that operand shapes, dtypes and devices are
what its kernel and grid assume, then calls the kernel library.  There is no
other implementation behind them: without the built library they raise
`KernelLibraryMissing`.  Activations are float32 or bfloat16 ("T" below); the
residual stream, norm weights, rotation frequencies and logits are float32
always.

`use_backend` swaps the object the calls go to.  The engine never does; it is
the seam through which tests check the engine's bookkeeping against a plain
emulation of each kernel's contract.
"""
from __future__ import annotations

import contextlib
from typing import Optional

import torch

_ACT = (torch.float32, torch.bfloat16)
HEAD_DIM_STEP, MAX_HEAD_DIM = 4, 256      # what `paged_attention` takes: multiples of 4 up to 256
_backend = None


class KernelShapeError(ValueError):
    """An operand does not have the shape, dtype or layout the kernel needs."""


def backend():
    global _backend
    if _backend is None:
        from wllm_amd.kernels.hip_backend import HipBackend
        _backend = HipBackend()
    return _backend


@contextlib.contextmanager
def use_backend(obj):
    global _backend
    old, _backend = _backend, obj
    try:
        yield obj
    finally:
        _backend = old


def _need(cond: bool, msg) -> None:
    """`msg` is the message or a function that makes it (so that it is made only on failure)."""
    if not cond:
        raise KernelShapeError(msg() if callable(msg) else msg)


def _dense(t: torch.Tensor, name: str, dtype, shape=None) -> None:
    # the messages are made only when a check fails: this runs for every operand of every launch
    if not isinstance(t, torch.Tensor):
        raise KernelShapeError(f"{name}: expected a tensor")
    if isinstance(dtype, tuple):
        if t.dtype not in dtype:
            raise KernelShapeError(f"{name}: dtype {t.dtype}, expected one of {dtype}")
    elif t.dtype != dtype:
        raise KernelShapeError(f"{name}: dtype {t.dtype}, expected {dtype}")
    if not t.is_contiguous():
        raise KernelShapeError(f"{name}: must be contiguous")
    if shape is not None and tuple(t.shape) != tuple(shape):
        raise KernelShapeError(f"{name}: shape {tuple(t.shape)}, expected {tuple(shape)}")


# ---- operations that parts bring with them ------------------------------------------------------
class RegisteredOp:
    """An operation added by `register_op`: a kernel of a library of its own (or of the framework's)
    with its host-side check, its launch and, for tests without a GPU, its plain emulation."""

    def __init__(self, name, entry_point, argtypes, launch, check, emulate, library):
        self.name, self.entry_point, self.argtypes = name, entry_point, list(argtypes)
        self.launch, self.check, self.emulate, self.library = launch, check, emulate, library


_REGISTERED: dict = {}


def register_op(name: str, *, entry_point: str, argtypes, launch, check=None, emulate=None, library=None,
                replace: bool = False) -> RegisteredOp:
    """Adds an operation without a change to this package: a new part's kernel is a `.hip` file and a
    Python file of the part's own.

    entry_point, argtypes: the `extern "C"` function (returning 0, a HIP error code, or -1 for sizes it
        does not take) and its ctypes signature, the stream last.
    library: a function that returns the loaded library holding it (`library.load(source_dir=...)` of a
        folder of kernels), or None for the framework's own library.
    check(*args, **kwargs): raises `KernelShapeError` unless shapes, dtypes and layouts are what the kernel
        and its grid assume; it runs on the host before every launch.
    launch(fn, stream, *args, **kwargs) -> int: calls `fn` with raw pointers (`ops.pointer(tensor)`) and the stream.
    emulate(*args, **kwargs): the same contract in plain torch, for the tests that run the engine's
        bookkeeping without a GPU; never used by the engine.

    `ops.call(name, ...)` then checks the operands and launches on the stream of the step."""
    if name in _REGISTERED and not replace:
        raise ValueError(f"operation {name!r} is already registered")
    op = RegisteredOp(name, entry_point, argtypes, launch, check, emulate, library)
    _REGISTERED[name] = op
    return op


def call(name: str, *args, **kwargs) -> None:
    """Runs a registered operation on the current backend."""
    op = _REGISTERED.get(name)
    if op is None:
        raise KeyError(f"operation {name!r} is not registered; known: {sorted(_REGISTERED)}")
    if op.check is not None:
        op.check(*args, **kwargs)
    backend().run_registered(op, args, kwargs)


def pointer(t: Optional[torch.Tensor]):
    """A tensor's address as a ctypes argument (None: a null pointer)."""
    import ctypes
    return ctypes.c_void_p(t.data_ptr()) if t is not None else ctypes.c_void_p(0)


def embed_lookup(ids: torch.Tensor, table: torch.Tensor, scale: float, out: torch.Tensor) -> None:
    """out[i] = float32(table[ids[i]]) * scale.  ids int32 [n], table T [V, H], out float32 [n, H]."""
    _dense(ids, "ids", torch.int32)
    _need(ids.dim() == 1, "ids: expected one axis")
    _dense(table, "table", _ACT)
    _need(table.dim() == 2, "table: expected [vocab, hidden]")
    _dense(out, "out", torch.float32, (ids.shape[0], table.shape[1]))
    if ids.shape[0]:
        call("embed_lookup", ids, table, float(scale), out)


def feed_tokens(ids: torch.Tensor, dst: torch.Tensor, src: torch.Tensor, source: torch.Tensor) -> None:
    """ids[dst[j]] = source[src[j]] for every j with dst[j] >= 0 (entries out of range are skipped).
    All int32 and one axis; dst and src of equal length.  It feeds a step the tokens that the step
    before it sampled on the device."""
    for t, name in ((ids, "ids"), (dst, "dst"), (src, "src"), (source, "source")):
        _dense(t, name, torch.int32)
        _need(t.dim() == 1, lambda: f"{name}: expected one axis")
    _need(dst.shape == src.shape, "dst and src: expected equal lengths")
    if dst.shape[0]:
        call("feed_tokens", ids, dst, src, source)


def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float, offset: float, out: torch.Tensor,
             delta: Optional[torch.Tensor] = None, rows: Optional[torch.Tensor] = None) -> None:
    """out = x * rsqrt(mean(x^2) + eps) * (offset + weight), all in float32, cast to out's dtype.

    x float32 [n, H]; weight float32 [H]; out T [m, H].  With `delta` (T [n, H], or a stack
    float32 [S, n, H] of partial sums that are added in order) the row normalised is
    x + delta.  Without `rows`, m = n and the sum is written back
    to x (the residual stream moves on).  With `rows` (int32 [m]) only those rows are
    read, x is left alone and out[i] belongs to row rows[i].
    """
    _dense(x, "x", torch.float32)
    _need(x.dim() == 2, "x: expected [tokens, hidden]")
    n, h = x.shape
    _dense(weight, "weight", torch.float32, (h,))
    if delta is not None:
        if delta.dim() == 3:
            _dense(delta, "delta", torch.float32, (delta.shape[0], n, h))
            _need(delta.shape[0] >= 1, "delta: an empty stack")
        else:
            _dense(delta, "delta", _ACT, (n, h))
    m = n
    if rows is not None:
        _dense(rows, "rows", torch.int32)
        _need(rows.dim() == 1, "rows: expected one axis")
        m = rows.shape[0]
    _dense(out, "out", _ACT, (m, h))
    if m:
        backend().rms_norm(x, weight, float(eps), float(offset), out, delta, rows)


def rope_and_cache_write(qkv: torch.Tensor, bias: Optional[torch.Tensor], positions: torch.Tensor,
                         inv_freq: Optional[torch.Tensor], slots: Optional[torch.Tensor],
                         cache: Optional[torch.Tensor], *, num_heads: int, num_kv_heads: int,
                         head_dim: int, page_size: int, parts: Optional[torch.Tensor] = None) -> None:
    """Adds `bias`, rotates queries and keys in place and stores keys and values in pages.

    qkv T [n, (num_heads + 2*num_kv_heads) * head_dim]: queries, then keys, then values.
    bias float32 of a row's width, or None.  positions int32 [n].  inv_freq float32
    [rotary_dim/2] (None: no rotation): element j of a head is paired with j + rotary_dim/2
    and the pair is turned by position * inv_freq[j], the angle and its sine and cosine in
    float32.  slots int32 [n]: page * page_size + offset for each token; cache
    T [pages, 2, num_kv_heads, page_size*head_dim] holds a page's keys as [page_size,
    head_dim] and its values as [head_dim, page_size].  slots and cache None: nothing is
    stored (the layer reads another layer's cache).  `parts` (float32 [S, n, width]): the
    projection arrives as a stack of partial sums; their sum in order replaces what qkv holds
    on entry.
    """
    width = (num_heads + 2 * num_kv_heads) * head_dim
    _dense(qkv, "qkv", _ACT)
    _need(qkv.dim() == 2 and qkv.shape[1] == width, lambda: f"qkv: shape {tuple(qkv.shape)}, expected [n, {width}]")
    n = qkv.shape[0]
    if bias is not None:
        _dense(bias, "bias", torch.float32, (width,))
    if parts is not None:
        _need(parts.dim() == 3 and parts.shape[0] >= 1, "parts: expected [S, n, width]")
        _dense(parts, "parts", torch.float32, (parts.shape[0], n, width))
    _dense(positions, "positions", torch.int32, (n,))
    rotary_dim = 0
    if inv_freq is not None:
        _dense(inv_freq, "inv_freq", torch.float32)
        _need(inv_freq.dim() == 1, "inv_freq: expected one axis")
        rotary_dim = 2 * inv_freq.shape[0]
        _need(0 < rotary_dim <= head_dim, lambda: f"rotary_dim {rotary_dim} does not fit head_dim {head_dim}")
    _need((slots is None) == (cache is None), "slots and cache go together")
    if cache is not None:
        _dense(slots, "slots", torch.int32, (n,))
        _dense(cache, "cache", qkv.dtype)
        _need(cache.dim() == 4 and tuple(cache.shape[1:]) == (2, num_kv_heads, page_size * head_dim),
              lambda: f"cache: shape {tuple(cache.shape)}, expected [pages, 2, {num_kv_heads}, {page_size * head_dim}]")
    if n:
        backend().rope_and_cache_write(qkv, bias, positions, inv_freq, slots, cache, num_heads, num_kv_heads,
                                       head_dim, rotary_dim, page_size, parts)


def linear_residual_takes(rows: int, dtype: torch.dtype, out_features: int, in_features: int) -> bool:
    """Whether `linear_residual` has a kernel for these sizes."""
    return bool(backend().linear_residual_takes(rows, dtype, out_features, in_features))


SUMSQ_BAND = 16      # columns whose squares `linear_residual` adds into one entry of `sumsq`


def linear_residual_sumsq_shape(rows: int, out_features: int) -> tuple:
    """The shape of the `sumsq` operand of `linear_residual` for a residual of [rows, out_features]."""
    return (rows, out_features // SUMSQ_BAND)


def linear_residual(x: torch.Tensor, weight: torch.Tensor, residual: torch.Tensor, sumsq: torch.Tensor,
                    tiles: Optional[torch.Tensor] = None) -> None:
    """residual += x @ weight^T in float32, and sumsq[m, b] = the sum of squares of the new
    residual[m, 16b : 16b + 16].  x T [m, k]; weight T [n, k] (`tiles`: its tile-major copy);
    residual float32 [m, n]; sumsq float32 [m, n / 16].  A row's mean square is then the sum of
    its row of `sumsq` over n: what a norm needs, without a pass over the residual.  Only for sizes
    that `linear_residual_takes`."""
    _dense(x, "x", _ACT)
    _need(x.dim() == 2, "x: expected [rows, in]")
    m, k = x.shape
    _dense(weight, "weight", x.dtype)
    _need(weight.dim() == 2 and weight.shape[1] == k, lambda: f"weight: shape {tuple(weight.shape)}, expected [out, {k}]")
    n = weight.shape[0]
    _check_tiles(tiles, weight, 1)
    _need(linear_residual_takes(m, x.dtype, n, k), "linear_residual: no kernel for these sizes")
    _dense(residual, "residual", torch.float32, (m, n))
    _dense(sumsq, "sumsq", torch.float32, linear_residual_sumsq_shape(m, n))
    if m:
        backend().linear_residual(x, weight, tiles, residual, sumsq)


def qkv_rope_takes(rows: int, dtype: torch.dtype, in_features: int, head_dim: int, rotary_dim: int) -> bool:
    """Whether `qkv_rope` has a kernel for these sizes (else the caller runs `linear` and
    `rope_and_cache_write`)."""
    return bool(backend().qkv_rope_takes(rows, dtype, in_features, head_dim, rotary_dim))


def qkv_rope(x: torch.Tensor, weight: torch.Tensor, qkv: torch.Tensor, bias: Optional[torch.Tensor],
             positions: torch.Tensor, inv_freq: Optional[torch.Tensor], slots: Optional[torch.Tensor],
             cache: Optional[torch.Tensor], *, num_heads: int, num_kv_heads: int, head_dim: int, page_size: int,
             tiles: Optional[torch.Tensor] = None) -> None:
    """qkv = x @ weight^T, then everything `rope_and_cache_write` does, in one kernel: the
    projection of a decode step never leaves the registers between the product and the rotation.
    x T [n, k]; weight T [(num_heads + 2*num_kv_heads) * head_dim, k], the stacked query, key and
    value matrices (`tiles`: its tile-major copy); the other operands as in `rope_and_cache_write`,
    with inv_freq of head_dim/2 entries or None.  Only for sizes that `qkv_rope_takes`."""
    width = (num_heads + 2 * num_kv_heads) * head_dim
    _dense(x, "x", _ACT)
    _need(x.dim() == 2, "x: expected [rows, in]")
    n = x.shape[0]
    _dense(weight, "weight", x.dtype, (width, x.shape[1]))
    _check_tiles(tiles, weight, 1)
    _dense(qkv, "qkv", x.dtype, (n, width))
    rotary_dim = 0
    if inv_freq is not None:
        _dense(inv_freq, "inv_freq", torch.float32)
        _need(inv_freq.dim() == 1, "inv_freq: expected one axis")
        rotary_dim = 2 * inv_freq.shape[0]
    _need(qkv_rope_takes(n, x.dtype, x.shape[1], head_dim, rotary_dim or head_dim),
          "qkv_rope: no kernel for these sizes; run linear and rope_and_cache_write")
    if bias is not None:
        _dense(bias, "bias", torch.float32, (width,))
    _dense(positions, "positions", torch.int32, (n,))
    _need((slots is None) == (cache is None), "slots and cache go together")
    if cache is not None:
        _dense(slots, "slots", torch.int32, (n,))
        _dense(cache, "cache", x.dtype)
        _need(cache.dim() == 4 and tuple(cache.shape[1:]) == (2, num_kv_heads, page_size * head_dim),
              lambda: f"cache: shape {tuple(cache.shape)}, expected [pages, 2, {num_kv_heads}, {page_size * head_dim}]")
    if n:
        backend().qkv_rope(x, weight, tiles, qkv, bias, positions, inv_freq, slots, cache, num_heads, num_kv_heads,
                           head_dim, page_size)


def paged_attention(qkv: torch.Tensor, cache: torch.Tensor, block_tables: torch.Tensor,
                    token_segment: torch.Tensor, seg_q_start: torch.Tensor, seg_q_len: torch.Tensor,
                    seg_ctx_len: torch.Tensor, out: torch.Tensor, *, num_heads: int, num_kv_heads: int,
                    head_dim: int, page_size: int, scale: float, window: int = 0,
                    max_q_len: int = 0, max_ctx_len: int = 0, plan=None) -> None:
    """Softmax attention of every query over the keys of its own request in the paged cache.

    The batch is a row of segments; segment s holds tokens seg_q_start[s] .. +seg_q_len[s],
    the last seg_q_len[s] positions of a request that is seg_ctx_len[s] long after this
    step.  Token i of it is at position p = ctx_len - q_len + i and sees keys
    max(0, p - window + 1) .. p (window 0: from key 0).  Query head h uses key/value head
    h // (num_heads // num_kv_heads).  Scores are scaled by `scale`; scores, softmax and the
    weighted sum accumulate in float32.  qkv as in `rope_and_cache_write` (only the queries
    are read); block_tables int32 [S, max_pages]; out T [n, num_heads*head_dim].
    max_q_len / max_ctx_len are host-side bounds of the segment arrays (0: unknown).
    `plan`: what `plan_paged_attention` returned for these segments and sizes, or None.
    """
    width = (num_heads + 2 * num_kv_heads) * head_dim
    _dense(qkv, "qkv", _ACT)
    _need(qkv.dim() == 2 and qkv.shape[1] == width, lambda: f"qkv: shape {tuple(qkv.shape)}, expected [n, {width}]")
    n = qkv.shape[0]
    _need(num_heads % num_kv_heads == 0, "num_heads must be a multiple of num_kv_heads")
    _dense(cache, "cache", qkv.dtype)
    _need(cache.dim() == 4 and tuple(cache.shape[1:]) == (2, num_kv_heads, page_size * head_dim),
          lambda: f"cache: shape {tuple(cache.shape)}, expected [pages, 2, {num_kv_heads}, {page_size * head_dim}]")
    _dense(block_tables, "block_tables", torch.int32)
    _need(block_tables.dim() == 2, "block_tables: expected [segments, pages]")
    s = block_tables.shape[0]
    _dense(token_segment, "token_segment", torch.int32, (n,))
    for name, t in (("seg_q_start", seg_q_start), ("seg_q_len", seg_q_len), ("seg_ctx_len", seg_ctx_len)):
        _dense(t, name, torch.int32, (s,))
    _dense(out, "out", qkv.dtype, (n, num_heads * head_dim))
    _need(window >= 0, "window must not be negative")
    if n:
        backend().paged_attention(qkv, cache, block_tables, token_segment, seg_q_start, seg_q_len, seg_ctx_len,
                                  out, num_heads, num_kv_heads, head_dim, page_size, float(scale), int(window),
                                  int(max_q_len), int(max_ctx_len), plan)


def plan_paged_attention(host_q_len, host_ctx_len, *, num_heads: int, num_kv_heads: int, head_dim: int,
                         page_size: int, window: int, dtype: torch.dtype, device):
    """Cuts a step's attention into work items for the kernels that want them, once per step
    and attention shape (all layers of that shape share it).  Returns an opaque plan, or None
    when the kernel that will run needs none.  host_q_len / host_ctx_len: the segment arrays
    on the host."""
    return backend().plan_paged_attention(host_q_len, host_ctx_len, num_heads, num_kv_heads, head_dim, page_size,
                                          int(window), dtype, device)


def static_attention_plan(segments: int, *, num_heads: int, num_kv_heads: int, head_dim: int, page_size: int,
                          window: int, dtype: torch.dtype, device, max_context: int, max_total_keys: int):
    """The same for a captured graph of `segments` requests of one token each: a plan of fixed shape in
    device memory, with room for contexts of up to `max_context` keys and `max_total_keys` keys of all
    requests together, whose `update(host_q_len, host_ctx_len)` rewrites it in place before a replay.
    None when the kernel that will run needs no plan."""
    make = getattr(backend(), "static_attention_plan", None)
    if make is None:
        return None
    return make(int(segments), num_heads, num_kv_heads, head_dim, page_size, int(window), dtype, device,
                int(max_context), int(max_total_keys))


def linear_splits(rows: int, out_features: int, in_features: int, dtype: torch.dtype) -> int:
    """Into how many partial sums over the input axis the product kernel for these sizes splits
    its work (1: it does not).  A caller that can take the sum later (the next norm, the rotation)
    hands `linear` an output of shape [S, rows, out_features] and saves the pass that adds them."""
    return int(backend().linear_splits(rows, out_features, in_features, dtype))


def tiled_size(rows: int, in_features: int, dtype: torch.dtype = torch.bfloat16) -> int:
    """Elements of the tile-major copy of a [rows, in_features] weight (`tile_weight`)."""
    if dtype == torch.float32:
        return -(-rows // 16) * 16 * -(-in_features // 16) * 16
    return -(-rows // 16) * 16 * in_features


def tile_weight(weight: torch.Tensor, halves: int = 1) -> Optional[torch.Tensor]:
    """The tile-major copy of a weight [n, k] that the few-row product kernels stream: a wavefront's
    load is one contiguous KiB of it, and its walk along k one contiguous run.
    bfloat16 (k a multiple of 32): for each band of 16 rows (the last padded with zero rows) and each
    step of 32 keys, a tile of 1 KiB in which lane l = 16g + i of a wavefront finds
    w[16 * band + i][32 * step + 8g .. +8].  With halves = 2 (a stacked gate and up matrix) each half
    is tiled by itself, the gate's bands first.
    float32 (k a multiple of 4): for each band of 16 rows and each chunk of 16 keys (rows and keys
    beyond the weight are zeros) a tile of 1 KiB in which lane l = 16g + i finds
    w[16 * band + i][16 * chunk + 4g .. +4]; a stacked matrix is tiled as the one matrix it is.
    Returns a flat tensor, or None for weights the few-row kernels do not take."""
    _dense(weight, "weight", _ACT)
    _need(weight.dim() == 2 and halves in (1, 2) and weight.shape[0] % halves == 0, "weight: expected [out, in]")
    if weight.dtype == torch.float32:
        n, k = weight.shape
        if k % 4 != 0 or n == 0 or k < 4:
            return None
        tiles = torch.empty(tiled_size(n, k, torch.float32), dtype=weight.dtype, device=weight.device)
        backend().tile_weight(weight, tiles)
        return tiles
    n, k = weight.shape[0] // halves, weight.shape[1]
    if k % 32 != 0 or n == 0:
        return None
    size = tiled_size(n, k)
    tiles = torch.empty(halves * size, dtype=weight.dtype, device=weight.device)
    for h in range(halves):
        backend().tile_weight(weight[h * n:(h + 1) * n], tiles[h * size:(h + 1) * size])
    return tiles


def _check_tiles(tiles, weight, halves: int) -> None:
    if tiles is None:
        return
    if weight.dtype == torch.float32:
        _need(weight.shape[1] % 4 == 0, "tiles: float32 weights have them only with in_features % 4 == 0")
        _dense(tiles, "tiles", weight.dtype, (tiled_size(weight.shape[0], weight.shape[1], torch.float32),))
        return
    n, k = weight.shape[0] // halves, weight.shape[1]
    _dense(tiles, "tiles", weight.dtype, (halves * tiled_size(n, k),))
    _need(k % 32 == 0, "tiles: bfloat16 weights have them only with in_features % 32 == 0")


def linear(x: torch.Tensor, weight: torch.Tensor, out: torch.Tensor, tiles: Optional[torch.Tensor] = None) -> None:
    """out = x @ weight^T.  x T [m, k]; weight T [n, k]; out T or float32 [m, n], or float32
    [S, m, n] with S = linear_splits(m, n, k, T): then the S slices are partial sums whose sum in
    order is the product.  Products of bfloat16 accumulate in float32; float32 stays float32.
    `tiles` is `tile_weight(weight)`, the same numbers in the order the few-row kernels read
    fastest; with it they read that copy instead."""
    _dense(x, "x", _ACT)
    _need(x.dim() == 2, "x: expected [rows, in]")
    _dense(weight, "weight", x.dtype)
    _need(weight.dim() == 2 and weight.shape[1] == x.shape[1],
          lambda: f"weight: shape {tuple(weight.shape)}, expected [out, {x.shape[1]}]")
    _check_tiles(tiles, weight, 1)
    if out.dim() == 3:
        s = linear_splits(x.shape[0], weight.shape[0], x.shape[1], x.dtype)
        _dense(out, "out", torch.float32, (s, x.shape[0], weight.shape[0]))
        _need(s > 1, "out: a stack of partial sums where the product is not split")
    else:
        _dense(out, "out", (x.dtype, torch.float32), (x.shape[0], weight.shape[0]))
    if x.shape[0]:
        backend().linear(x, weight, out, tiles)


# the activations of a gated feed-forward and the numbers the kernels know them by (`common.h` holds
# the same table): a new one is a line here, a line and a case there
ACTIVATIONS = {"gelu_tanh": 0, "silu": 1}


def gated_activation(gate_up: torch.Tensor, out: torch.Tensor, activation: str) -> None:
    """out = act(gate_up[:, :I]) * gate_up[:, I:], in float32, cast to T.  gate_up T [n, 2I]."""
    _need(activation in ACTIVATIONS, lambda: f"activation {activation!r}: expected one of {sorted(ACTIVATIONS)}")
    _dense(gate_up, "gate_up", _ACT)
    _need(gate_up.dim() == 2 and gate_up.shape[1] % 2 == 0, "gate_up: expected [n, 2*intermediate]")
    _dense(out, "out", gate_up.dtype, (gate_up.shape[0], gate_up.shape[1] // 2))
    if gate_up.shape[0]:
        call("gated_activation", gate_up, out, activation)


class NormOnLoad:
    """The input of a product as something the product kernel computes while it reads it:
    rms_norm(residual) with the rows' sums of squares already known.  residual float32 [m, k];
    sumsq float32 [m, c] whose rows add up to the rows' sums of squares (`linear_residual` leaves
    it); weight float32 [k]; the result is what `rms_norm(residual, weight, eps, offset)` gives in
    dtype T."""

    def __init__(self, residual: torch.Tensor, sumsq: torch.Tensor, weight: torch.Tensor, eps: float, offset: float,
                 dtype: torch.dtype):
        _dense(residual, "residual", torch.float32)
        _need(residual.dim() == 2, "residual: expected [rows, hidden]")
        _dense(sumsq, "sumsq", torch.float32)
        _need(sumsq.dim() == 2 and sumsq.shape[0] == residual.shape[0] and sumsq.shape[1] >= 1,
              "sumsq: expected [rows, columns]")
        _dense(weight, "weight", torch.float32, (residual.shape[1],))
        self.residual, self.sumsq, self.weight = residual, sumsq, weight
        self.eps, self.offset, self.dtype = float(eps), float(offset), dtype

    @property
    def shape(self):
        return self.residual.shape


def gated_linear_norm_takes(rows: int, dtype: torch.dtype, in_features: int) -> bool:
    """Whether `gated_linear` can take its input as a `NormOnLoad` at these sizes."""
    return bool(backend().gated_linear_norm_takes(rows, dtype, in_features))


def gated_linear(x, weight: torch.Tensor, out: torch.Tensor, activation: str,
                 scratch: Optional[torch.Tensor], tiles: Optional[torch.Tensor] = None) -> None:
    """out = act(x @ Wg^T) * (x @ Wu^T) with weight = [Wg; Wu] stacked, T [2I, k]; x T [m, k];
    out T [m, I]; scratch T [m, 2I] may be used for the unfused product.  `tiles` is
    `tile_weight(weight, halves=2)`.  x may be a `NormOnLoad` where `gated_linear_norm_takes` says so:
    the norm is then applied as the kernel reads the residual stream (scratch is not used)."""
    _need(activation in ACTIVATIONS, lambda: f"activation {activation!r}: expected one of {sorted(ACTIVATIONS)}")
    if isinstance(x, NormOnLoad):
        _need(gated_linear_norm_takes(x.shape[0], x.dtype, x.shape[1]), "gated_linear: no kernel with the norm on load for these sizes")
        _dense(weight, "weight", x.dtype)
        _need(weight.dim() == 2 and weight.shape[1] == x.shape[1] and weight.shape[0] % 2 == 0,
              lambda: f"weight: shape {tuple(weight.shape)}, expected [2*intermediate, {x.shape[1]}]")
        _dense(out, "out", x.dtype, (x.shape[0], weight.shape[0] // 2))
        _check_tiles(tiles, weight, 2)
        if x.shape[0]:
            backend().gated_linear_norm(x, weight, out, activation, tiles)
        return
    _dense(x, "x", _ACT)
    _need(x.dim() == 2, "x: expected [rows, in]")
    _dense(weight, "weight", x.dtype)
    _need(weight.dim() == 2 and weight.shape[1] == x.shape[1] and weight.shape[0] % 2 == 0,
          lambda: f"weight: shape {tuple(weight.shape)}, expected [2*intermediate, {x.shape[1]}]")
    inter = weight.shape[0] // 2
    _dense(out, "out", x.dtype, (x.shape[0], inter))
    _dense(scratch, "scratch", x.dtype, (x.shape[0], 2 * inter))
    _check_tiles(tiles, weight, 2)
    if x.shape[0]:
        backend().gated_linear(x, weight, out, activation, scratch, tiles)


def argmax_rows(logits: torch.Tensor, out: torch.Tensor) -> None:
    """out[i] = index of the largest value of row i, the lowest index among equals.
    logits float32 [m, V]; out int32 [m]."""
    _dense(logits, "logits", torch.float32)
    _need(logits.dim() == 2 and logits.shape[1] > 0, "logits: expected [rows, vocab]")
    _dense(out, "out", torch.int32, (logits.shape[0],))
    if logits.shape[0]:
        backend().argmax_rows(logits, out)


def sample_rows(logits: torch.Tensor, params: torch.Tensor, seeds: torch.Tensor,
                penalty_ids: Optional[torch.Tensor], penalty_offsets: Optional[torch.Tensor],
                out_tokens: torch.Tensor, out_logprobs: torch.Tensor, truncations: bool = True) -> None:
    """Samples one token per row.

    logits float32 [m, V].  params float32 [m, 5]: temperature (0: greedy), top_k (0: off),
    top_p (1: off), min_p (0: off), repetition_penalty (1: off).  seeds int64 [m, 2]: the
    key and counter of the row's uniform draw.  penalty_ids int32 [P] with penalty_offsets
    int32 [m+1]: the ids the repetition penalty applies to, row by row (None: no row has
    any).  out_tokens int32 [m]; out_logprobs float32 [m]: log-probability of the token
    under the penalised, temperature-scaled distribution before truncation (temperature 1
    for greedy rows).  `truncations` may be False only if no row has top_k or top_p on: the
    kernels then skip the passes that find their thresholds.
    """
    _dense(logits, "logits", torch.float32)
    _need(logits.dim() == 2 and logits.shape[1] > 0, "logits: expected [rows, vocab]")
    m = logits.shape[0]
    _dense(params, "params", torch.float32, (m, 5))
    _dense(seeds, "seeds", torch.int64, (m, 2))
    _need((penalty_ids is None) == (penalty_offsets is None), "penalty_ids and penalty_offsets go together")
    if penalty_ids is not None:
        _dense(penalty_ids, "penalty_ids", torch.int32)
        _dense(penalty_offsets, "penalty_offsets", torch.int32, (m + 1,))
    _dense(out_tokens, "out_tokens", torch.int32, (m,))
    _dense(out_logprobs, "out_logprobs", torch.float32, (m,))
    if m:
        backend().sample_rows(logits, params, seeds, penalty_ids, penalty_offsets, out_tokens, out_logprobs,
                              truncations)


# ---- the framework's own operations that go through the same door as a part's ------------------
def _register_own() -> None:
    from ctypes import c_float, c_int, c_void_p
    p = pointer
    register_op("embed_lookup", entry_point="wllm_embed_lookup",
                argtypes=[c_void_p, c_void_p, c_int, c_float, c_void_p, c_int, c_int, c_int, c_void_p],
                launch=lambda fn, stream, ids, table, scale, out: fn(
                    p(ids), p(table), int(table.dtype == torch.bfloat16), scale, p(out), ids.shape[0], table.shape[1],
                    table.shape[0], stream))
    register_op("feed_tokens", entry_point="wllm_feed_tokens",
                argtypes=[c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_void_p],
                launch=lambda fn, stream, ids, dst, src, source: fn(
                    p(ids), p(dst), p(src), p(source), dst.shape[0], ids.shape[0], source.shape[0], stream))
    register_op("gated_activation", entry_point="wllm_gated_activation",
                argtypes=[c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_void_p],
                launch=lambda fn, stream, gate_up, out, activation: fn(
                    p(gate_up), p(out), int(gate_up.dtype == torch.bfloat16), ACTIVATIONS[activation], gate_up.shape[0],
                    out.shape[1], stream))


_register_own()
