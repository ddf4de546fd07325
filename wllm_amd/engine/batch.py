"""What one step runs on: a flat batch of segments and the tensors that describe it.

A segment is the next tokens of one request: a portion of its prompt, or the one
token it decoded last.  The reference never mixes the two (a prefill call takes
one sequence, src/wllm/models/llama.py:159-160,468; a decode call takes one token
of each, llama.py:535-539); here any number of both lie side by side in one
batch.  All index arrays of a step are packed into one int32 host buffer and go
to the device in one copy.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Optional

import numpy as np
import torch


@dataclass
class StepEntry:
    """A request's next tokens, and the places among them whose logits are wanted."""
    request: object
    tokens: list
    want: list = field(default_factory=list)
    # The last of `tokens` is not known on the host yet: it is row `feed_row` of the tensor of
    # sampled tokens that the step is given (`ModelRunner.step(..., feed_tokens=...)`), read on the
    # device.  The value in `tokens` is then a placeholder.
    feed_row: Optional[int] = None


@dataclass
class PageView:
    """The pages of one schedule entry as a mixer sees them."""
    storage: torch.Tensor          # [pages, *page shape]; keys and values: [pages, 2, kv_heads, page_size*head_dim]
    block_tables: torch.Tensor     # int32 [segments, max_pages]
    slots: torch.Tensor            # int32 [tokens]
    page_size: int
    writes: bool                   # False: this entry reads another entry's cache


class Workspace:
    """Named scratch tensors that live across steps and grow on demand, until `freeze`: a captured
    graph holds their addresses, so afterwards a request for more than there is raises."""

    def __init__(self, device):
        self.device = device
        self._flat: dict = {}
        self._frozen = False

    def freeze(self) -> None:
        self._frozen = True

    def get(self, name: str, shape: tuple, dtype: torch.dtype) -> torch.Tensor:
        count = 1
        for s in shape:
            count *= s
        key = (name, dtype)
        flat = self._flat.get(key)
        if flat is None or flat.numel() < count:
            if self._frozen:
                raise RuntimeError(f"scratch tensor {name!r} would have to grow to {count} elements, "
                                   "but a captured graph holds its address")
            flat = torch.empty(max(count, 1), dtype=dtype, device=self.device)
            self._flat[key] = flat
        return flat[:count].view(shape)


class StepContext:
    """Everything a part may ask about the step it runs in."""

    def __init__(self, *, n, num_segments, dtype, device, workspace, cache, schedule,
                 token_ids, positions, token_segment, seg_q_start, seg_q_len, seg_ctx_len,
                 state_slots, logit_rows, num_logit_rows, group_slots, group_block_tables,
                 host_q_start, host_q_len, host_ctx_len, host_state_slots, requests):
        self.n = n
        self.num_segments = num_segments
        self.dtype = dtype
        self.device = device
        self._workspace = workspace
        self._cache = cache
        self._schedule = schedule
        self.token_ids = token_ids
        self.positions = positions
        self.token_segment = token_segment
        self.seg_q_start = seg_q_start
        self.seg_q_len = seg_q_len
        self.seg_ctx_len = seg_ctx_len
        self.state_slots = state_slots
        self.logit_rows = logit_rows
        self.num_logit_rows = num_logit_rows
        self._group_slots = group_slots
        self._group_block_tables = group_block_tables
        # the same segment arrays on the host, for parts that loop over segments
        self.host_q_start = host_q_start
        self.host_q_len = host_q_len
        self.host_ctx_len = host_ctx_len
        self.host_state_slots = host_state_slots
        self.requests = requests
        self.max_q_len = int(host_q_len.max()) if num_segments else 0
        self.max_ctx_len = int(host_ctx_len.max()) if num_segments else 0
        self._plans: dict = {}             # key -> (plan, refresh)
        # set by a captured graph: its kernels hold the addresses of what a part makes for the step, so
        # a plan has a fixed shape, sized by these limits, and is rewritten in place before each replay
        self.captured = False
        self.capture_max_context = 0       # the longest context of a request the graph takes
        self.capture_max_tokens = 0        # the most tokens all its requests hold together (the pool's)

    def plan(self, key, build, refresh=None):
        """What a part prepares on the host for a step (work items, a routing table, the chunks of a
        scan), made once per step and `key` and shared by every layer that asks under the same key.
        `build(ctx)` makes it from the step's host arrays (`host_q_len`, `host_ctx_len`, ...) and may
        return None.  In a captured graph (`ctx.captured`) `build` runs once, when the graph is first
        run, and makes a plan of fixed shape in device memory sized by `capture_max_context` and
        `capture_max_tokens`; `refresh(plan, ctx)` then rewrites its contents in place before every
        replay, the first included.  A part whose plan needs a refresh and gives none cannot be
        captured."""
        if key not in self._plans:
            made = build(self)
            self._plans[key] = (made, refresh)
            if self.captured and made is not None and refresh is not None:
                refresh(made, self)
        return self._plans[key][0]

    def refresh_plans(self) -> None:
        """Before a replay of the captured graph: every plan takes the step's contents."""
        for made, refresh in self._plans.values():
            if made is not None and refresh is not None:
                refresh(made, self)

    def buffer(self, name: str, shape: tuple, dtype: torch.dtype) -> torch.Tensor:
        return self._workspace.get(name, shape, dtype)

    def pages(self, entry: int) -> PageView:
        owner = self._schedule[entry].reads_cache_of
        writes = owner is None
        owner = entry if writes else owner
        g = self._cache.group_of_entry[owner]
        return PageView(self._cache.entry_storage(owner), self._group_block_tables[g], self._group_slots[g],
                        self._cache.page_size, writes)

    def state(self, entry: int) -> Optional[torch.Tensor]:
        """[max_requests, *shape] state of a schedule entry (float32 unless the mixer asked for
        another dtype); row state_slots[s] belongs to segment s."""
        return self._cache.state.get(entry)
