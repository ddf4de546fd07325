"""Captured HIP graphs for decode steps.

A decode step (every request brings one token and wants its logits) launches a few hundred
small kernels; issued one by one from Python they cost more host time than GPU time (the
reference counts about 880 launches of 8 microseconds in a 30 ms step,
src/wllm/engine/cuda_graph_decoder.py:5-11, and captures one CUDA graph per batch-size
bucket, :66-134).  Here a graph is captured per bucket and class of context lengths (its
attention kernel's grid and its block tables are as large as its longest context needs, so
short contexts get graphs of their own).  A graph owns everything whose
address its kernels hold: a packed int32 buffer with all index arrays of the step (ids,
positions, slots, block tables of fixed width, attention work items of fixed count), its
scratch tensors and its logits.  A step fills the pinned host copy of the buffer, copies it
to the device in one transfer and replays.  Rows beyond the live requests are padding: a
request of one token on a page reserved for that purpose (the reference pads with permanent
scratch sequences, cuda_graph_decoder.py:72-87).

No memset node is recorded: buffers are cleared, where they must be, by kernels.
"""
from __future__ import annotations

import gc

import numpy as np
import torch

from wllm_amd.engine.batch import StepContext, Workspace
from wllm_amd.kernels import ops


def capture(body):
    """Captures what `body()` launches into a new graph; returns (graph, body's result).

    No garbage collection while the stream is capturing: a collector run that frees an object with
    device resources of its own (an event, pinned memory, another graph) makes a call the capture
    does not allow, and the process aborts.  The collector is switched back on afterwards if it was
    on, also when the body raises."""
    graph = torch.cuda.CUDAGraph()
    collecting = gc.isenabled()
    gc.disable()
    try:
        with torch.cuda.graph(graph):
            result = body()
    finally:
        if collecting:
            gc.enable()
    return graph, result


class DecodeGraph:
    def __init__(self, runner, bucket: int, max_context: int, workspace=None):
        self.runner = runner
        self.bucket = bucket
        self.max_context = max_context
        cache, model = runner.cache, runner.model
        self.device = runner.device
        self.page_size = cache.page_size
        self.num_groups = len(cache.groups)
        self.table_width = -(-max_context // cache.page_size)
        b = bucket
        # layout of the packed buffer: eight arrays of b, then per group slots [b] and tables [b, width]
        # and two arrays of b that say which token ids come from the device (`feed_row`)
        sizes = [b] * 8 + [b] * self.num_groups + [b * self.table_width] * self.num_groups + [b] * 2
        self._offsets = np.concatenate([[0], np.cumsum(sizes)]).astype(np.int64)
        total = int(self._offsets[-1])
        self.host = torch.zeros(total, dtype=torch.int32, pin_memory=True)
        self.dev = torch.zeros(total, dtype=torch.int32, device=self.device)
        self.np = self.host.numpy()
        v = [self.dev[self._offsets[i]:self._offsets[i + 1]] for i in range(len(sizes))]
        g = self.num_groups
        self._feed_dst, self._feed_src = v[8 + 2 * g], v[9 + 2 * g]
        self.workspace = workspace if workspace is not None else Workspace(self.device)
        self.ctx = StepContext(
            n=b, num_segments=b, dtype=model.dtype, device=self.device, workspace=self.workspace, cache=cache,
            schedule=model.plan.schedule, token_ids=v[0], positions=v[1], token_segment=v[2], seg_q_start=v[3],
            seg_q_len=v[4], seg_ctx_len=v[5], state_slots=v[6], logit_rows=v[7], num_logit_rows=b,
            group_slots=v[8:8 + g], group_block_tables=[t.view(b, self.table_width) for t in v[8 + g:8 + 2 * g]],
            host_q_start=np.arange(b, dtype=np.int32), host_q_len=np.ones(b, dtype=np.int32),
            host_ctx_len=np.ones(b, dtype=np.int32), host_state_slots=np.zeros(b, dtype=np.int32),
            requests=[None] * b)
        self.ctx.max_q_len, self.ctx.max_ctx_len = 1, max_context
        self.ctx.captured = True
        self.ctx.capture_max_context = max_context
        self.ctx.capture_max_tokens = max(g_.pool.num_pages for g_ in cache.groups) * cache.page_size
        self.graph = None
        self.logits = None
        self._copied = torch.cuda.Event()
        self._in_flight = False

    def _field(self, i: int) -> np.ndarray:
        return self.np[self._offsets[i]:self._offsets[i + 1]]

    def fill(self, entries: list, reserved: list) -> None:
        """Writes the step's arrays into the pinned buffer; rows beyond the entries are padding."""
        cache, b, n = self.runner.cache, self.bucket, len(entries)
        g = self.num_groups
        if self._in_flight:
            self._copied.synchronize()      # the last transfer out of the pinned buffer is over
        old = np.fromiter((cache.context_len(e.request) for e in entries), dtype=np.int32, count=n)
        ids, pos, seg, q0, ql, cl, st, rows = (self._field(i) for i in range(8))
        ids[:n] = [e.tokens[0] for e in entries]
        ids[n:] = 0
        pos[:n] = old
        pos[n:] = 0
        seg[:] = np.arange(b)
        q0[:] = np.arange(b)
        ql[:] = 1
        cl[:n] = old + 1
        cl[n:] = 1
        st[:n] = [cache.slot(e.request) for e in entries]
        st[n:] = cache.padding_slot         # a state row that belongs to no request
        rows[:] = np.arange(b)
        for gi in range(g):
            slots = self._field(8 + gi)
            table = self._field(8 + g + gi).reshape(b, self.table_width)
            dummy = self.runner.dummy_pages[gi]
            slots[n:] = dummy * self.page_size
            table[n:, 0] = dummy
            for i, e in enumerate(entries):
                slots[i] = reserved[i][gi][0]
                t = cache.block_table(e.request, gi)
                table[i, :len(t)] = np.maximum(np.asarray(t, dtype=np.int32), 0)
        feed_dst, feed_src = self._field(8 + 2 * g), self._field(9 + 2 * g)
        feed_dst[:] = -1
        feed_src[:] = 0
        for i, e in enumerate(entries):
            if e.feed_row is not None:
                feed_dst[i], feed_src[i] = i, e.feed_row
        self.ctx.host_ctx_len = cl.copy()
        self.ctx.host_state_slots = st.copy()
        self.ctx.requests = [e.request for e in entries] + [None] * (b - n)
        self.ctx.refresh_plans()
        self.dev.copy_(self.host, non_blocking=True)
        self._copied.record()
        self._in_flight = True

    def run(self, entries: list, reserved: list, feed_tokens=None) -> torch.Tensor:
        if self.graph is None:
            # Once eagerly, so that scratch tensors and plans come into being and lazy library state
            # settles, with every row a padding row: the run before the capture must leave no trace in
            # a request's pages or state (a mixer that updates a state would update it twice).
            self.fill([], [])
            self.runner.model.forward(self.ctx)
            torch.cuda.synchronize()
            self.graph, self.logits = capture(lambda: self.runner.model.forward(self.ctx))
            self.workspace.freeze()
        self.fill(entries, reserved)
        if feed_tokens is not None:
            # outside the captured graph: the tensor of sampled tokens is not the graph's own
            ops.feed_tokens(self.ctx.token_ids, self._feed_dst, self._feed_src, feed_tokens)
        self.graph.replay()
        return self.logits[:len(entries)]
