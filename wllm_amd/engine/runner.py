"""The step function: a batch of (request, its next tokens) in, logits at the wanted
places out.

`ModelRunner.step` runs only the tokens it is given, as one batch, from the cache
that earlier steps left.  It asks the cache manager for room for every entry
first (all or nothing: a step that does not fit raises `OutOfPages` before
anything ran), builds the index tensors, runs the model and commits the new
lengths.  It is the only way tokens reach the model: the scheduler, the replay
tool and the benchmark all call it.
"""
from __future__ import annotations

from typing import Optional

import numpy as np
import torch

from wllm_amd.cache.manager import CacheManager
from wllm_amd.cache.pages import OutOfPages
from wllm_amd.engine.batch import StepContext, StepEntry, Workspace
from wllm_amd.kernels import ops
from wllm_amd.kernels.staging import pack_int32


class StepError(ValueError):
    """A step's entries are inconsistent with each other or with the cache."""


class ModelRunner:
    def __init__(self, model, cache: CacheManager):
        self.model = model
        self.cache = cache
        self.device = model.device
        self.workspace = Workspace(self.device)
        self.steps_run = 0
        self.tokens_run = 0
        self.graphs: dict = {}             # bucket -> {longest context -> DecodeGraph}
        self.graph_buckets: tuple = ()
        self.graph_contexts: tuple = ()    # ascending; the last is graph_max_context
        self.graph_max_context = 0
        self.dummy_pages: list = []
        self.graph_steps = 0

    def enable_graphs(self, buckets=(1, 2, 4, 8, 16, 32, 48, 64, 128, 256), max_context=None, contexts=None) -> None:
        """Decode-only steps of up to max(buckets) requests replay a captured graph of the
        smallest bucket that holds them; the largest number of requests the cache admits, if it
        is below max(buckets), is a bucket too, so that a full batch of any size has its graph.
        A bucket has a graph for each class of context lengths (the longest, a half of it, a
        quarter, down to about a thousand tokens): a graph's attention runs as many workgroups
        as its longest context needs, live or not, and its block tables are as wide.  Graphs
        are captured when a step first needs them (`contexts` names other classes).  One page per
        group is set aside for padding rows."""
        if self.graph_buckets:
            return
        if not self.model.graph_capturable():
            raise ValueError("a part of this model reads the step's arrays on the host; its steps cannot be captured")
        limit = min(self.model.plan.max_positions, min(g.pool.num_pages - 1 for g in self.cache.groups) * self.cache.page_size)
        self.graph_max_context = min(max_context or limit, limit)
        if contexts is None:
            contexts = [self.graph_max_context]
            while contexts[-1] > 1024:
                contexts.append(-(-contexts[-1] // (2 * self.cache.page_size)) * self.cache.page_size)
        self.graph_contexts = tuple(sorted({c for c in contexts if c < self.graph_max_context} | {self.graph_max_context}))
        most = self.cache.max_requests
        self.graph_buckets = tuple(sorted({b for b in buckets if b <= most} | ({most} if most <= max(buckets) else set())))
        self.dummy_pages = [self.cache.set_aside_page(gi) for gi in range(len(self.cache.groups))]

    def _graph_for(self, entries: list):
        if not self.graph_buckets or len(entries) > self.graph_buckets[-1]:
            return None
        longest = 0
        for e in entries:
            if len(e.tokens) != 1 or list(e.want) != [0]:
                return None
            longest = max(longest, self.cache.context_len(e.request) + 1)
        if longest > self.graph_max_context:
            return None
        bucket = next(b for b in self.graph_buckets if b >= len(entries))
        context = next(c for c in self.graph_contexts if c >= longest)
        of_bucket = self.graphs.setdefault(bucket, {})
        if context not in of_bucket:
            from wllm_amd.engine.graphs import DecodeGraph

            # the graphs of a bucket run one at a time and need scratch tensors of the same shapes
            shared = next(iter(of_bucket.values())).workspace if of_bucket else None
            of_bucket[context] = DecodeGraph(self, bucket, context, workspace=shared)
        return of_bucket[context]

    @classmethod
    def create(cls, model, *, num_pages: int, page_size: int, max_requests: int, **cache_options):
        cache = CacheManager(model.cache_needs(), page_size, num_pages, max_requests, model.dtype, model.device,
                             state_shapes=model.state_shapes(), **cache_options)
        return cls(model, cache)

    def open(self, request) -> None:
        self.cache.open(request)

    def close(self, request) -> None:
        self.cache.close(request)

    def step(self, entries: list, feed_tokens: Optional[torch.Tensor] = None) -> torch.Tensor:
        """Returns float32 logits [wanted, vocab] in the order of the entries and of
        each entry's `want`.  The tensor is a view of a buffer the next step reuses.
        `feed_tokens` (int32, on the device) holds the tokens of entries with a `feed_row`: the
        output of a sampling that the host has not read yet."""
        if any(e.feed_row is not None for e in entries):
            if feed_tokens is None:
                raise StepError("an entry names a feed_row but the step was given no feed_tokens")
        else:
            feed_tokens = None
        graph = self._graph_for(entries) if entries else None
        if graph is not None:
            self._validate(entries)
            reserved = self._reserve(entries)
            logits = graph.run(entries, reserved, feed_tokens)
            self.graph_steps += 1
        else:
            ctx = self.prepare(entries)
            if feed_tokens is not None:
                ops.feed_tokens(ctx.token_ids, ctx.feed_dst, ctx.feed_src, feed_tokens)
            logits = self.model.forward(ctx)
        self.commit(entries)
        return logits

    def commit(self, entries: list) -> None:
        """Moves the requests' lengths after all layers wrote."""
        for e in entries:
            self.cache.commit(e.request, len(e.tokens))
        self.steps_run += 1
        self.tokens_run += sum(len(e.tokens) for e in entries)

    def prepare(self, entries: list) -> StepContext:
        """Checks the entries, takes room for them in the cache (all or none) and builds
        the step's index tensors."""
        self._validate(entries)
        cache = self.cache
        reserved = self._reserve(entries)
        return self._build_context(entries, reserved)

    def _validate(self, entries: list) -> None:
        cache = self.cache
        max_pos = self.model.plan.max_positions
        seen = set()
        for e in entries:
            if e.request in seen:
                raise StepError(f"request {e.request!r} appears twice in one step")
            seen.add(e.request)
            if not cache.is_open(e.request):
                raise StepError(f"request {e.request!r} is not open")
            if len(e.tokens) == 0:
                raise StepError(f"request {e.request!r} brings no tokens")
            if cache.context_len(e.request) + len(e.tokens) > max_pos:
                raise StepError(f"request {e.request!r} would reach {cache.context_len(e.request) + len(e.tokens)} "
                                f"tokens; the model allows {max_pos}")
            if e.feed_row is not None and e.feed_row < 0:
                raise StepError(f"request {e.request!r}: feed_row {e.feed_row} is negative")
            for w in e.want:
                if not 0 <= w < len(e.tokens):
                    raise StepError(f"request {e.request!r}: wanted place {w} is not among its {len(e.tokens)} tokens")
            vocab = self.model.plan.embedding.vocab_size
            if min(e.tokens) < 0 or max(e.tokens) >= vocab:
                raise StepError(f"request {e.request!r}: token id outside 0..{vocab - 1}")

    def _reserve(self, entries: list) -> list:
        """Room for every entry, or for none."""
        cache = self.cache
        reserved = []
        try:
            for e in entries:
                reserved.append(cache.reserve(e.request, len(e.tokens)))
        except OutOfPages:
            for e in entries[:len(reserved) + 1]:
                cache.trim(e.request)
            raise
        return reserved

    def _build_context(self, entries: list, reserved: list) -> StepContext:
        cache = self.cache
        num_groups = len(cache.groups)
        s = len(entries)
        q_len = np.array([len(e.tokens) for e in entries], dtype=np.int32)
        q_start = np.zeros(s, dtype=np.int32)
        if s:
            q_start[1:] = np.cumsum(q_len)[:-1]
        n = int(q_len.sum())
        old_len = np.array([cache.context_len(e.request) for e in entries], dtype=np.int32)
        ctx_len = old_len + q_len
        token_ids = np.concatenate([np.asarray(e.tokens, dtype=np.int64) for e in entries]) if s else np.zeros(0, np.int64)
        token_ids = token_ids.astype(np.int32)
        token_segment = np.repeat(np.arange(s, dtype=np.int32), q_len)
        positions = (np.arange(n, dtype=np.int32) - q_start[token_segment] + old_len[token_segment]).astype(np.int32)
        logit_rows = np.array([q_start[i] + w for i, e in enumerate(entries) for w in e.want], dtype=np.int32)
        state_slots = np.array([cache.slot(e.request) for e in entries], dtype=np.int32)
        group_slots, group_tables = [], []
        for g in range(num_groups):
            group_slots.append(np.concatenate([r[g] for r in reserved]) if s else np.zeros(0, np.int32))
            tables = [cache.block_table(e.request, g) for e in entries]
            width = max((len(t) for t in tables), default=1)
            bt = np.zeros((s, max(width, 1)), dtype=np.int32)
            for i, t in enumerate(tables):
                # a page given back (-1) lies outside every window that is still read
                bt[i, :len(t)] = np.maximum(np.asarray(t, dtype=np.int32), 0)
            group_tables.append(bt)
        fed = [i for i, e in enumerate(entries) if e.feed_row is not None]
        feed_dst = np.array([q_start[i] + q_len[i] - 1 for i in fed], dtype=np.int32)
        feed_src = np.array([entries[i].feed_row for i in fed], dtype=np.int32)
        arrays = [token_ids, positions, token_segment, q_start, q_len, ctx_len, state_slots, logit_rows]
        arrays += group_slots + group_tables + [feed_dst, feed_src]
        dev = pack_int32(arrays, self.device)
        ctx = StepContext(
            n=n, num_segments=s, dtype=self.model.dtype, device=self.device, workspace=self.workspace,
            cache=cache, schedule=self.model.plan.schedule,
            token_ids=dev[0], positions=dev[1], token_segment=dev[2], seg_q_start=dev[3], seg_q_len=dev[4],
            seg_ctx_len=dev[5], state_slots=dev[6], logit_rows=dev[7], num_logit_rows=int(logit_rows.size),
            group_slots=dev[8:8 + num_groups], group_block_tables=dev[8 + num_groups:8 + 2 * num_groups],
            host_q_start=q_start, host_q_len=q_len, host_ctx_len=ctx_len, host_state_slots=state_slots,
            requests=[e.request for e in entries])
        ctx.feed_dst, ctx.feed_src = dev[8 + 2 * num_groups], dev[9 + 2 * num_groups]
        return ctx
