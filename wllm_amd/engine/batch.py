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
        self._attention_plans: dict = {}
        # set by a captured graph: plans of fixed shape, refreshed in place before each replay
        self.static_plans = False
        self.static_max_context = 0
        self.static_max_total_keys = 0

    def attention_plan(self, *, num_heads: int, num_kv_heads: int, head_dim: int, page_size: int, window: int):
        """The step's work items for attention of this shape; made once, shared by all layers."""
        from wllm_amd.kernels import ops
        key = (num_heads, num_kv_heads, head_dim, page_size, window)
        if key not in self._attention_plans and self.static_plans:
            plan = ops.backend().static_attention_plan(
                self.num_segments, num_heads, num_kv_heads, head_dim, page_size, window, self.dtype, self.device,
                self.static_max_context, self.static_max_total_keys)
            if plan is not None:
                plan.update(self.host_q_len, self.host_ctx_len)
            self._attention_plans[key] = plan
        if key not in self._attention_plans:
            self._attention_plans[key] = ops.plan_paged_attention(
                self.host_q_len, self.host_ctx_len, num_heads=num_heads, num_kv_heads=num_kv_heads,
                head_dim=head_dim, page_size=page_size, window=window, dtype=self.dtype, device=self.device)
        return self._attention_plans[key]

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
