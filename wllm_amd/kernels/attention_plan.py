"""How a step's attention is cut into work items for the matrix-core kernel.

For one request (segment) and one key/value head the query rows are the pairs (token, query
head of the group): rows = q_len * group.  A segment of at most 16 rows, and a segment of one token
whatever its group (a decoded token), is short: tiles of 16 rows (one, unless more than 16 query heads
share a key/value head) whose keys are split over workgroups in fixed chunks of `KEY_CHUNK` keys, the
partial results combined by a second kernel; chunk boundaries are multiples of the chunk size
counted from key 0, so they depend on the key index only.  Longer segments are cut into
workgroups of four tiles of 16 rows (prefill items).

A work item is 8 int32: segment, key/value head in the low 16 bits with the tile's number (its first
row / 16) in the high 16, the segment's number of new tokens, the place of
its first token among the step's tokens, first key, end key, partial slot (-1: the workgroup writes
the final result), the segment's context length: what the kernel needs of the segment comes with
the item, in the one read it begins with, and not from the segments' arrays in a second trip to memory.  A partial slot holds
one tile of 16 rows.  A reduce item is 8 int32: segment, key/value head, first partial slot, number
of splits, first row of the tile, slots between two splits, 2 unused.  A prefill item (long
segments, 64 rows each, for the kernel that stages keys and values through shared memory) is
8 int32: segment, key/value head, first row, first key, end key, partial slot (-1: final), 2
unused.  The keys of a block of rows are split over several prefill items when the step has too
few blocks to fill the compute units (a portion of a prompt late in a long context) or when they
span more pages than the kernel's shared copy of the block table holds; the pieces of a block are
equal and begin at multiples of 32 keys (`prefill_piece_length` chooses how long).  The prefill
items of a step are ordered by length, longest first, every second run of as many as the device has
compute units turned round: workgroups start in this order.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional

import numpy as np
import torch

KEY_CHUNK = 128
ROWS_PER_TILE = 16
ITEM_INTS = 8
PREFILL_TABLE_PAGES = 1024      # pages one prefill item may span (the kernel's shared block table)
PREFILL_MIN_PIECE = 16          # groups of 32 keys; shorter pieces cost more in partial results than they gain
WORKGROUP_SLOTS = 512           # prefill workgroups a device runs at once unless the caller knows better (two a compute unit)
PREFILL_ROWS = 64               # rows of a prefill item unless the kernel for the sizes at hand says otherwise


@dataclass
class AttentionPlan:
    items: torch.Tensor                 # int32 [num_items, 8] on the device
    reduce_items: Optional[torch.Tensor]  # int32 [num_reduce, 8] or None
    num_items: int
    num_reduce: int
    num_partial_slots: int
    partial_o: Optional[torch.Tensor] = None    # float32 [slots * 16 * head_dim]
    partial_ml: Optional[torch.Tensor] = None   # float32 [slots * 16 * 2]
    prefill_items: Optional[torch.Tensor] = None  # int32 [num_prefill, 8]
    num_prefill: int = 0
    prefill_rows: int = 64
    live_items: Optional[torch.Tensor] = None     # int32 [1] on the device: how many of `items` count (None: all)


class StaticAttentionPlan(AttentionPlan):
    """A plan of fixed shape for a captured graph: room for `segments * kv_heads * fixed_splits`
    work items in the same device tensors, whose contents `update` rewrites before each replay.
    The live items come first and their number lies in device memory behind them (`live_items`):
    the kernel reads it, so a step costs what its live items cost.  Partial slots are numbered
    over the live chunks only, so the partial buffers are as large as the most keys the cache
    pool can hold needs, not as the fixed shape."""

    def __init__(self, segments: int, group: int, num_kv_heads: int, window: int, fixed_splits: int,
                 max_slots: int, head_dim: int, device):
        # a live item of a segment with several chunks holds a partial slot; a segment with one has one item
        n_r = segments * num_kv_heads * row_tiles(1, group)
        max_slots = min(max_slots, n_r * fixed_splits)
        n_i = min(n_r * fixed_splits, max_slots + n_r)
        # the number of live items (and 7 unused), the reduce items, the items: a step copies the
        # front of it, up to the last live item
        self._host = torch.empty((1 + n_r + n_i) * ITEM_INTS, dtype=torch.int32, pin_memory=True)
        self._dev = torch.zeros_like(self._host, device=device)
        self._args = (group, num_kv_heads, window)
        self.max_slots = max_slots
        a, b = ITEM_INTS, (1 + n_r) * ITEM_INTS
        super().__init__(self._dev[b:].view(n_i, ITEM_INTS), self._dev[a:b].view(n_r, ITEM_INTS), n_i, n_r, max_slots,
                         torch.empty(max(1, max_slots) * ROWS_PER_TILE * head_dim, dtype=torch.float32, device=device),
                         torch.empty(max(1, max_slots) * ROWS_PER_TILE * 2, dtype=torch.float32, device=device))
        self.live_items = self._dev[:1]

    def update(self, q_len: np.ndarray, ctx_len: np.ndarray) -> None:
        group, nkv, window = self._args
        items, reduces, slots, prefill, _ = build_work_items(q_len, ctx_len, group, nkv, window)
        if prefill.shape[0]:
            raise ValueError("a captured decode graph holds segments of one token only")
        if slots > self.max_slots:
            raise ValueError(f"the step needs {slots} partial slots, the graph's plan has {self.max_slots}")
        if items.shape[0] > self.num_items or reduces.shape[0] > self.num_reduce:
            raise ValueError(f"the step needs {items.shape[0]} work items and {reduces.shape[0]} reduce items, "
                             f"the graph's plan has room for {self.num_items} and {self.num_reduce}")
        buf = self._host.numpy()
        buf[0] = items.shape[0]
        # a graph runs a reduce item for every (segment, key/value head); those beyond the segments
        # with several chunks stand for nothing
        a, b = ITEM_INTS, (1 + self.num_reduce) * ITEM_INTS
        buf[a:b].reshape(-1, ITEM_INTS)[reduces.shape[0]:, 0] = -1
        buf[a:a + reduces.size] = reduces.reshape(-1)
        buf[b:b + items.size] = items.reshape(-1)
        used = b + items.size
        self._dev[:used].copy_(self._host[:used], non_blocking=True)


def row_tiles(q_len: int, group: int) -> int:
    """Tiles of 16 rows of a short segment of `q_len` tokens."""
    return -(-(q_len * group) // ROWS_PER_TILE)


MAX_HEADS = 1 << 16     # an item packs the key/value head and the tile's number into 16 bits each
MAX_TILES = 1 << 15     # tiles of 16 rows a segment may have for one key/value head (the item's int32 stays positive)


def build_tile_items(q_len: np.ndarray, ctx_len: np.ndarray, group: int, num_kv_heads: int, window: int):
    """Every segment, whatever its length, as tiles of 16 rows with their keys in chunks of `KEY_CHUNK`
    counted from key 0 (the float32 kernel takes nothing else): a tile's chunks are those its rows can
    need, from the lowest key of its first row's window to its last row's position.  Returns (items
    [n, 8], reduce items [m, 8], partial slots) in the format of the short segments' items."""
    q_len = np.asarray(q_len, dtype=np.int64)
    ctx_len = np.asarray(ctx_len, dtype=np.int64)
    rows = q_len * group
    q_start = np.cumsum(q_len) - q_len
    nt = -(-rows // ROWS_PER_TILE)
    if nt.size and int(nt.max()) >= MAX_TILES:
        raise ValueError(f"a segment of {int(rows.max())} rows a key/value head: a work item numbers at most {MAX_TILES} tiles")
    seg_of = np.repeat(np.arange(q_len.size), nt)
    tile = np.arange(int(nt.sum())) - np.repeat(np.cumsum(nt) - nt, nt)
    row0 = tile * ROWS_PER_TILE
    first_pos = (ctx_len - q_len)[seg_of]
    last_row = np.minimum(rows[seg_of] - 1, row0 + ROWS_PER_TILE - 1)
    lo = np.maximum(0, first_pos + row0 // group - window + 1) if window > 0 else np.zeros_like(row0)
    hi = first_pos + last_row // group + 1
    c0 = lo // KEY_CHUNK
    ns = (hi - 1) // KEY_CHUNK - c0 + 1
    n_items = int(ns.sum())
    tile_of = np.repeat(np.arange(tile.size), ns)
    j = np.arange(n_items) - np.repeat(np.cumsum(ns) - ns, ns)
    chunk = c0[tile_of] + j
    split = ns > 1
    tile_slots = np.where(split, ns, 0)
    tile_base = np.cumsum(tile_slots) - tile_slots
    per_head = int(tile_slots.sum())
    kv = np.arange(num_kv_heads, dtype=np.int64)
    it = np.zeros((num_kv_heads, n_items, ITEM_INTS), dtype=np.int32)
    it[..., 0] = seg_of[tile_of][None, :]
    it[..., 1] = kv[:, None] | (tile[tile_of] << 16)[None, :]
    it[..., 2] = q_len[seg_of[tile_of]][None, :]
    it[..., 3] = q_start[seg_of[tile_of]][None, :]
    it[..., 4] = np.maximum(lo[tile_of], chunk * KEY_CHUNK)[None, :]
    it[..., 5] = np.minimum(hi[tile_of], (chunk + 1) * KEY_CHUNK)[None, :]
    it[..., 6] = np.where(split[tile_of][None, :], kv[:, None] * per_head + (tile_base[tile_of] + j)[None, :], -1)
    it[..., 7] = ctx_len[seg_of[tile_of]][None, :]
    st = np.nonzero(split)[0]
    rs = np.zeros((num_kv_heads, st.size, ITEM_INTS), dtype=np.int32)
    rs[..., 0] = seg_of[st][None, :]
    rs[..., 1] = kv[:, None]
    rs[..., 2] = kv[:, None] * per_head + tile_base[st][None, :]
    rs[..., 3] = ns[st][None, :]
    rs[..., 4] = row0[st][None, :]
    rs[..., 5] = 1
    return it.reshape(-1, ITEM_INTS), rs.reshape(-1, ITEM_INTS), per_head * num_kv_heads


def prefill_piece_length(span: np.ndarray, num_kv_heads: int, workgroup_slots: int, longest: int) -> int:
    """The most groups of 32 keys a prefill item gets, for blocks of rows that span `span` groups each
    (per key/value head).  The shortest length with which the items fill the workgroup slots of the
    device at most once, twice, ... (the fewest rounds that the longest allowed piece permits): every
    further item costs a partial result that is written and read again, and items that start together
    and are about equally long end together.  Never shorter than `PREFILL_MIN_PIECE` groups, below which
    a piece's partial result costs more than its share of the keys."""
    def count(length):
        return int((-(-span // length)).sum()) * num_kv_heads
    rounds = max(1, -(-count(longest) // workgroup_slots))
    lo, hi = 1, longest                      # the least length whose count fits
    while lo < hi:
        mid = (lo + hi) // 2
        if count(mid) <= rounds * workgroup_slots:
            hi = mid
        else:
            lo = mid + 1
    return min(longest, max(lo, PREFILL_MIN_PIECE))


def build_work_items(q_len: np.ndarray, ctx_len: np.ndarray, group: int, num_kv_heads: int, window: int,
                     page_size: int = 16, prefill_rows: int = PREFILL_ROWS, workgroup_slots: int = WORKGROUP_SLOTS,
                     tiles_only: bool = False):
    """Returns (items [n, 8], reduce_items [m, 8], partial slots, prefill items [p, 8], rows per
    prefill item) as int32 arrays.  `tiles_only`: no prefill items; long segments too are cut into
    tiles of 16 rows (`build_tile_items`)."""
    if tiles_only:
        if group * num_kv_heads >= MAX_HEADS:
            raise ValueError(f"{group * num_kv_heads} query heads: a work item has 16 bits for a head")
        items, reduces, slots = build_tile_items(q_len, ctx_len, group, num_kv_heads, window)
        return items, reduces, slots, np.zeros((0, ITEM_INTS), np.int32), prefill_rows
    q_len = np.asarray(q_len, dtype=np.int64)
    ctx_len = np.asarray(ctx_len, dtype=np.int64)
    rows = q_len * group
    q_start = np.cumsum(q_len) - q_len
    if group * num_kv_heads >= MAX_HEADS:
        raise ValueError(f"{group * num_kv_heads} query heads: a work item has 16 bits for a head")
    short = (rows <= ROWS_PER_TILE) | (q_len == 1)
    items, reduces = [], []
    slots = 0
    kv = np.arange(num_kv_heads, dtype=np.int64)
    # ---- short segments, vectorised over segments ----
    idx = np.nonzero(short)[0]
    if idx.size:
        first_pos = ctx_len[idx] - q_len[idx]
        lo = np.maximum(0, first_pos - window + 1) if window > 0 else np.zeros_like(first_pos)
        c0 = lo // KEY_CHUNK
        c1 = (ctx_len[idx] - 1) // KEY_CHUNK
        ns = c1 - c0 + 1
        width = int(ns.max())
        j = np.arange(width, dtype=np.int64)
        chunk = c0[:, None] + j[None, :]                       # [S, width]
        live = j[None, :] < ns[:, None]
        kb = np.maximum(lo[:, None], chunk * KEY_CHUNK)
        ke = np.minimum(ctx_len[idx][:, None], (chunk + 1) * KEY_CHUNK)
        single = ns == 1
        # tiles of 16 rows a segment has (one, unless a token's group has more than 16 heads)
        rt = -(-rows[idx] // ROWS_PER_TILE)
        T = int(rt.max())
        tile = np.arange(T, dtype=np.int64)
        tile_live = tile[None, :] < rt[:, None]                 # [S, T]
        # partial slots: one per (segment, kv head, tile, split) for segments that are split
        n_split_seg = np.where(single, 0, ns)
        seg_base = np.concatenate([[0], np.cumsum(n_split_seg * num_kv_heads * rt)])[:-1]
        S = idx.size
        it = np.zeros((S, num_kv_heads, T, width, ITEM_INTS), dtype=np.int32)
        it[..., 0] = np.where(live, idx[:, None], -1)[:, None, None, :]
        it[..., 1] = (kv[None, :, None] | (tile[None, None, :] << 16))[..., None]
        it[..., 2] = q_len[idx][:, None, None, None]
        it[..., 3] = q_start[idx][:, None, None, None]
        it[..., 4] = kb[:, None, None, :]
        it[..., 5] = ke[:, None, None, :]
        it[..., 7] = ctx_len[idx][:, None, None, None]
        first_slot = seg_base[:, None, None] + (kv[None, :, None] * rt[:, None, None] + tile[None, None, :]) \
            * n_split_seg[:, None, None]                        # [S, kv, T]
        it[..., 6] = np.where(single[:, None, None, None], -1, first_slot[..., None] + j[None, None, None, :])
        keep = np.broadcast_to(live[:, None, None, :] & tile_live[:, None, :, None], (S, num_kv_heads, T, width))
        items.append(it[keep].reshape(-1, ITEM_INTS))
        split_seg = ~single
        if split_seg.any():
            rs = np.zeros((S, num_kv_heads, T, ITEM_INTS), dtype=np.int32)
            rs[..., 0] = idx[:, None, None]
            rs[..., 1] = kv[None, :, None]
            rs[..., 2] = first_slot
            rs[..., 3] = ns[:, None, None]
            rs[..., 4] = tile[None, None, :] * ROWS_PER_TILE
            rs[..., 5] = 1
            keep_r = np.broadcast_to((split_seg[:, None] & tile_live)[:, None, :], (S, num_kv_heads, T))
            reduces.append(rs[keep_r].reshape(-1, ITEM_INTS))
        slots = int((n_split_seg * num_kv_heads * rt).sum())
    # ---- long segments: workgroups of 64 or 128 rows of one key/value head ----
    prefill = np.zeros((0, ITEM_INTS), np.int32)
    long_idx = np.nonzero(~short)[0]
    if long_idx.size:
        # the blocks of rows of all long segments, one after the other
        n_blocks = -(-rows[long_idx] // prefill_rows)
        seg_of = np.repeat(long_idx, n_blocks)
        rb = (np.arange(int(n_blocks.sum())) - np.repeat(np.cumsum(n_blocks) - n_blocks, n_blocks)) * prefill_rows
        first_pos = (ctx_len - q_len)[seg_of]
        hi = first_pos + np.minimum(rows[seg_of] - 1, rb + prefill_rows - 1) // group + 1
        lo = np.maximum(0, first_pos + rb // group - window + 1) if window > 0 else np.zeros_like(rb)
        # a block's keys are cut into equal pieces whose boundaries are multiples of 32 counted from the block's
        # first group of 32
        lo32 = lo // 32 * 32
        span = -(-(hi - lo32) // 32)                                                  # in groups of 32 keys
        # a piece that starts inside a page touches up to two pages more than its keys fill
        longest = max(KEY_CHUNK, (PREFILL_TABLE_PAGES - 2) * page_size // KEY_CHUNK * KEY_CHUNK) // 32
        ns = -(-span // prefill_piece_length(span, num_kv_heads, workgroup_slots, longest))
        piece = -(-span // ns)
        ns = -(-span // piece)
        tiles = prefill_rows // ROWS_PER_TILE
        n_items = int(ns.sum())
        block_of = np.repeat(np.arange(rb.size), ns)
        j = np.arange(n_items) - np.repeat(np.cumsum(ns) - ns, ns)
        split = ns > 1
        # slots of a split block: [split][tile], blocks one after the other, per key/value head
        block_slots = np.where(split, ns * tiles, 0)
        block_base = np.cumsum(block_slots) - block_slots
        per_head = int(block_slots.sum())
        it = np.zeros((num_kv_heads, n_items, ITEM_INTS), dtype=np.int32)
        it[..., 0] = seg_of[block_of][None, :]
        it[..., 1] = kv[:, None]
        it[..., 2] = rb[block_of][None, :]
        it[..., 3] = (lo32[block_of] + j * piece[block_of] * 32)[None, :]
        it[..., 4] = (lo32[block_of] + (j + 1) * piece[block_of] * 32)[None, :]
        slot = slots + kv[:, None] * per_head + (block_base[block_of] + j * tiles)[None, :]
        it[..., 5] = np.where(split[block_of][None, :], slot, -1)
        it = it.reshape(-1, ITEM_INTS)
        # The workgroups start in the order of the items, the first ones one on each compute unit, the next ones
        # beside them: the longest pieces come first, and each further run of `workgroup_slots / 2` turns round,
        # so that a long piece gets a short one for its neighbour and the last to start are the shortest.
        length = np.minimum(it[:, 4], hi[block_of][None, :].repeat(num_kv_heads, 0).reshape(-1)) - it[:, 3]
        order = np.argsort(-length, kind="stable")
        run = max(1, workgroup_slots // 2)
        turned = (np.arange(order.size) // run) % 2 == 1
        place = np.arange(order.size)
        run_first = place // run * run
        run_last = np.minimum(run_first + run, order.size) - 1
        prefill = it[order[np.where(turned, run_first + run_last - place, place)]]
        sb = np.nonzero(split)[0]
        if sb.size:
            t = np.arange(tiles, dtype=np.int64)
            first_row = rb[sb][:, None] + t[None, :] * ROWS_PER_TILE           # [blocks, tiles]
            live = first_row < rows[seg_of[sb]][:, None]
            rs = np.zeros((num_kv_heads, sb.size, tiles, ITEM_INTS), dtype=np.int32)
            rs[..., 0] = seg_of[sb][None, :, None]
            rs[..., 1] = kv[:, None, None]
            rs[..., 2] = slots + kv[:, None, None] * per_head + (block_base[sb][:, None] + t[None, :])[None]
            rs[..., 3] = ns[sb][None, :, None]
            rs[..., 4] = first_row[None]
            rs[..., 5] = tiles
            reduces.append(rs[:, live].reshape(-1, ITEM_INTS))
        slots += per_head * num_kv_heads
    items = np.concatenate(items) if items else np.zeros((0, ITEM_INTS), np.int32)
    reduces = np.concatenate(reduces) if reduces else np.zeros((0, ITEM_INTS), np.int32)
    return items, reduces, slots, prefill, prefill_rows
