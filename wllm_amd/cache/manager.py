"""The cache manager: keys and values in pages, a block table for each request,
and slots for per-request state of fixed size.

The reference has one pool and one block table per sequence for all layers
(src/wllm/engine/kv_cache.py:63-119,259-303).  Here the runs of layers
("schedule entries") that own a cache are sorted into groups by what they need
per token: entries that keep all keys of `h` heads of size `d` share a group,
entries that keep a window of them are another group.  Each group has its own
pool of pages and each request has one block table per group; a page id means
the same token slots in every entry of its group.

Pages are given back when a request is closed, and, in a group with a window,
as soon as every token of a page is out of reach of all later queries.  The
contract of `reserve` and `commit` is the reference's `reserve`/`advance`
(kv_cache.py:259-292): `reserve` makes room and says where the new tokens go
without moving the request's length; `commit` moves it after all layers wrote.
`reserve` is all-or-nothing across groups.

What a page holds is the need's to say (`page_shape`).  For keys and values
(`CacheNeed`) a page is [2, kv_heads, page_size * head_dim]: the keys as
[page_size, head_dim] and the values transposed, [head_dim, page_size], which
is the order the matrix-core attention kernels read them in.  A mixer that keeps
something else per token (`PagedNeed`: a compressed vector, an integer code)
gets pages of [page_size, *token_shape] in a dtype of its choice; the manager
treats both alike.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Optional

import numpy as np
import torch

from wllm_amd.cache.pages import OutOfPages, PageAccountingError, PagePool


_SET_ASIDE = "(set aside)"


class OutOfSlots(RuntimeError):
    """More live requests than state slots."""


@dataclass(frozen=True)
class CacheNeed:
    """What one schedule entry keeps per token: keys and values of
    `num_kv_heads` heads of `head_dim`; all of them (window None) or the last
    `window`.  Stored in the model's dtype."""
    num_kv_heads: int
    head_dim: int
    window: Optional[int] = None
    dtype = None

    def page_shape(self, page_size: int) -> tuple:
        return (2, self.num_kv_heads, page_size * self.head_dim)


@dataclass(frozen=True)
class PagedNeed:
    """Any other per-token payload: `token_shape` numbers of `dtype` (None: the
    model's) for every token, of all tokens (window None) or of the last `window`.
    A page is [page_size, *token_shape]."""
    token_shape: tuple
    window: Optional[int] = None
    dtype: Optional[torch.dtype] = None

    def page_shape(self, page_size: int) -> tuple:
        return (page_size,) + tuple(self.token_shape)


@dataclass(frozen=True)
class StateNeed:
    """Per-request state of fixed size: one tensor of `shape` and `dtype` per
    request, zeroed when the request is opened.  A mixer's `state_shape()` may
    return this, or a plain shape for float32."""
    shape: tuple
    dtype: torch.dtype = torch.float32


@dataclass
class LayerGroup:
    need: CacheNeed
    entries: list                      # schedule entries that own a cache here
    pool: PagePool
    storage: Optional[torch.Tensor]    # [len(entries), pages, *need.page_shape(page_size)]
    index_of_entry: dict = field(default_factory=dict)


@dataclass
class RequestCache:
    context_len: int = 0
    slot: int = -1
    # per group: page id at each page index of the request; -1 once given back
    tables: list = field(default_factory=list)
    # per group: first page index not yet given back
    first_live: list = field(default_factory=list)


class CacheManager:
    def __init__(self, needs: dict, page_size: int, num_pages, max_requests: int,
                 dtype: torch.dtype, device, state_shapes: Optional[dict] = None,
                 allocate_storage: bool = True, poison_freed_pages: bool = False):
        """`needs`: {schedule entry: need} for the entries that own a cache; a need is hashable
        and has `window` (or None), `page_shape(page_size)` and `dtype` (None: the model's):
        `CacheNeed`, `PagedNeed`.
        `num_pages`: pages of every group's pool (an int, or {need: int}).
        `state_shapes`: {schedule entry: shape or StateNeed} of fixed-size per-request state.
        `poison_freed_pages`: overwrite a page with NaN when it is given back, so
        that a read of a stale page shows in the results (for tests).
        """
        if page_size <= 0:
            raise ValueError(f"page_size must be positive, got {page_size}")
        if max_requests <= 0:
            raise ValueError(f"max_requests must be positive, got {max_requests}")
        self.page_size = page_size
        self.max_requests = max_requests
        self.dtype = dtype
        self.device = device
        self.poison_freed_pages = poison_freed_pages
        self.groups: list[LayerGroup] = []
        self.group_of_entry: dict = {}
        by_need: dict = {}
        for entry in sorted(needs):
            by_need.setdefault(needs[entry], []).append(entry)
        for need, entries in by_need.items():
            n = num_pages[need] if isinstance(num_pages, dict) else num_pages
            storage = None
            if allocate_storage:
                storage = torch.zeros(len(entries), n, *need.page_shape(page_size),
                                      dtype=getattr(need, "dtype", None) or dtype, device=device)
            g = LayerGroup(need, entries, PagePool(n), storage, {e: i for i, e in enumerate(entries)})
            for e in entries:
                self.group_of_entry[e] = len(self.groups)
            self.groups.append(g)
        self.requests: dict = {}
        self._set_aside: dict = {}
        self._free_slots = list(range(max_requests - 1, -1, -1))
        self.state: dict = {}
        for entry, need in (state_shapes or {}).items():
            if not isinstance(need, StateNeed):
                need = StateNeed(tuple(need))
            # one row more than there are requests: `padding_slot`, for the rows of a captured graph
            # that stand for no request (they read and write it, and nobody else does)
            self.state[entry] = torch.zeros((max_requests + 1,) + tuple(need.shape), dtype=need.dtype, device=device)

    @property
    def padding_slot(self) -> int:
        """The state row set aside for rows of a batch that belong to no request."""
        return self.max_requests

    # ---- requests ----------------------------------------------------------
    def open(self, request) -> int:
        """Registers a request and gives it a state slot (zeroed)."""
        if request in self.requests:
            raise KeyError(f"request {request!r} is already open")
        if not self._free_slots:
            raise OutOfSlots(f"all {self.max_requests} state slots are taken")
        slot = self._free_slots.pop()
        for t in self.state.values():
            t[slot].zero_()
        self.requests[request] = RequestCache(0, slot, [[] for _ in self.groups], [0 for _ in self.groups])
        return slot

    def is_open(self, request) -> bool:
        return request in self.requests

    def context_len(self, request) -> int:
        return self.requests[request].context_len

    def slot(self, request) -> int:
        return self.requests[request].slot

    def close(self, request) -> None:
        """Gives back every page and the state slot of a request."""
        rc = self.requests.pop(request)
        for gi, g in enumerate(self.groups):
            for page in rc.tables[gi]:
                if page >= 0:
                    self._release(g, page, request)
        self._free_slots.append(rc.slot)

    # ---- pages ---------------------------------------------------------------
    def pages_for(self, group_index: int, num_tokens: int, longest_portion: int = 1) -> int:
        """Upper bound of the pages a request of `num_tokens` holds at one time in a
        group, when it is fed in portions of at most `longest_portion` tokens."""
        ps = self.page_size
        need = self.groups[group_index].need
        total = -(-num_tokens // ps)
        if need.window is None:
            return total
        # a window's oldest key and the newest token of a portion can straddle pages
        return min(total, -(-(need.window + longest_portion) // ps) + 1)

    def new_pages_needed(self, request, num_new_tokens: int) -> list:
        """Per group, how many pages `reserve(request, num_new_tokens)` would take."""
        rc = self.requests[request]
        end = rc.context_len + num_new_tokens
        return [max(0, -(-end // self.page_size) - len(rc.tables[gi])) for gi in range(len(self.groups))]

    def num_free_pages(self, group_index: int = 0) -> int:
        return self.groups[group_index].pool.num_free

    def usable_pages(self, group_index: int) -> int:
        """Pages of a group that requests can ever hold: the pool without the pages set aside."""
        return self.groups[group_index].pool.num_pages - len(self._set_aside.get(group_index, []))

    def set_aside_page(self, group_index: int) -> int:
        """Takes one page of a group out of circulation for good (captured graphs point
        their padding rows at it) and returns its id."""
        page = self.groups[group_index].pool.allocate(_SET_ASIDE)
        self._set_aside.setdefault(group_index, []).append(page)
        return page

    def reserve(self, request, num_new_tokens: int) -> list:
        """Makes room for the next `num_new_tokens` tokens of a request in every
        group, or raises OutOfPages and leaves everything as it was.  Returns, per
        group, an int32 array of the flat slots (page * page_size + offset) the
        tokens go to.  Calling it again before `commit` gives the same answer.
        """
        rc = self.requests[request]
        ps = self.page_size
        start, end = rc.context_len, rc.context_len + num_new_tokens
        taken = []
        try:
            for gi, g in enumerate(self.groups):
                table = rc.tables[gi]
                while len(table) * ps < end:
                    page = g.pool.allocate(request)
                    table.append(page)
                    taken.append((gi, page))
        except OutOfPages:
            for gi, page in reversed(taken):
                popped = rc.tables[gi].pop()
                assert popped == page
                self.groups[gi].pool.free(page, request)
            raise
        pos = np.arange(start, end, dtype=np.int64)
        out = []
        for gi in range(len(self.groups)):
            table = np.asarray(rc.tables[gi], dtype=np.int64)
            pages = table[pos // ps] if num_new_tokens else pos
            if num_new_tokens and (pages < 0).any():
                raise PageAccountingError(f"request {request!r} writes to a page it gave back")
            out.append((pages * ps + pos % ps).astype(np.int32))
        return out

    def trim(self, request) -> None:
        """Gives back pages that `reserve` took beyond the request's committed length
        (after a step that did not run)."""
        rc = self.requests[request]
        keep = -(-rc.context_len // self.page_size)
        for gi, g in enumerate(self.groups):
            table = rc.tables[gi]
            while len(table) > keep:
                page = table.pop()
                if page >= 0:
                    self._release(g, page, request)

    def commit(self, request, num_new_tokens: int) -> None:
        """Moves the request's length after all layers wrote, then gives back the
        pages a window has passed: the next query is at position context_len and
        reaches back to context_len - window + 1."""
        rc = self.requests[request]
        rc.context_len += num_new_tokens
        for gi, g in enumerate(self.groups):
            w = g.need.window
            if w is None:
                continue
            first_needed = max(0, rc.context_len - w + 1) // self.page_size
            table = rc.tables[gi]
            while rc.first_live[gi] < min(first_needed, len(table)):
                i = rc.first_live[gi]
                self._release(g, table[i], request)
                table[i] = -1
                rc.first_live[gi] += 1

    def block_table(self, request, group_index: int) -> list:
        return self.requests[request].tables[group_index]

    def entry_storage(self, entry: int) -> torch.Tensor:
        """[pages, *page_shape] of one schedule entry."""
        g = self.groups[self.group_of_entry[entry]]
        return g.storage[g.index_of_entry[entry]]

    def _release(self, g: LayerGroup, page: int, request) -> None:
        g.pool.free(page, request)
        if self.poison_freed_pages and g.storage is not None:
            if g.storage.dtype.is_floating_point:
                g.storage[:, page] = float("nan")
            else:
                g.storage[:, page] = torch.iinfo(g.storage.dtype).min

    # ---- invariants ------------------------------------------------------------
    def check(self) -> None:
        """No page lost, held twice or held by a closed request; slots likewise."""
        for gi, g in enumerate(self.groups):
            g.pool.check()
            seen = {}
            for request, rc in self.requests.items():
                for page in rc.tables[gi]:
                    if page < 0:
                        continue
                    if page in seen:
                        raise PageAccountingError(f"page {page} is in the tables of {seen[page]!r} and {request!r}")
                    seen[page] = request
                    if g.pool.holder(page) != request:
                        raise PageAccountingError(f"page {page} in the table of {request!r} is held by {g.pool.holder(page)!r}")
            if set(seen) | set(self._set_aside.get(gi, [])) != set(g.pool.held_pages()):
                raise PageAccountingError("a held page is in no table")
        slots = [rc.slot for rc in self.requests.values()]
        if len(set(slots)) != len(slots) or set(slots) & set(self._free_slots):
            raise PageAccountingError("a state slot is held twice")
        if len(slots) + len(self._free_slots) != self.max_requests:
            raise PageAccountingError("a state slot is lost")
