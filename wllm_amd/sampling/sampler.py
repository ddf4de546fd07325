"""The sampler: one token per row of logits, on the GPU.

Rows that are all greedy and unpenalised take the argmax kernel.  Otherwise one
kernel does what the reference's `sample` does step by step
(src/wllm/engine/sampling.py:101-143); see `wllm_amd/csrc/sampling.hip` for the
order and for the two deliberate differences (a per-row counter-based random draw,
order-independent sums).  A row's uniform number is Philox4x32-10 with the row's
seed as key and the index of the output token as counter.
"""
from __future__ import annotations

from typing import Optional, Sequence

import numpy as np
import torch

from wllm_amd.kernels import ops
from wllm_amd.kernels.staging import pack_words
from wllm_amd.sampling.params import SamplingParams


class Sampler:
    def __init__(self, device, default_seed: int = 0):
        self.device = device
        self.default_seed = default_seed

    def seed_of(self, params: SamplingParams, request_index: int) -> int:
        """The key of a request's draws: its own seed, or one derived from the
        sampler's seed and the order in which requests were added."""
        if params.seed is not None:
            return int(params.seed) & 0x7FFF_FFFF_FFFF_FFFF
        return (self.default_seed * 0x9E3779B97F4A7C15 + request_index * 0xBF58476D1CE4E5B9 + 1) & 0x7FFF_FFFF_FFFF_FFFF

    def sample(self, logits: torch.Tensor, params: Sequence[SamplingParams], seeds: Sequence[int],
               counters: Sequence[int], generated: Optional[Sequence[Sequence[int]]] = None,
               want_logprobs: bool = True):
        """logits float32 [m, V] (overwritten where a repetition penalty applies).
        Returns (tokens, logprobs) as Python lists; logprobs is None if they are not
        wanted and every row is greedy and unpenalised."""
        return self.finish(self.start(logits, params, seeds, counters, generated, want_logprobs))

    def start(self, logits: torch.Tensor, params: Sequence[SamplingParams], seeds: Sequence[int],
              counters: Sequence[int], generated: Optional[Sequence[Sequence[int]]] = None,
              want_logprobs: bool = True) -> "PendingSample":
        """Enqueues the sampling and the copy of its results to the host and returns without
        waiting.  `PendingSample.tokens` stays on the device: a step started before the results are
        read takes its token ids from there."""
        m = logits.shape[0]
        assert len(params) == m and len(seeds) == m and len(counters) == m
        tokens = torch.empty(m, dtype=torch.int32, device=logits.device)
        plain_greedy = all(p.greedy and p.repetition_penalty == 1.0 for p in params)
        if plain_greedy and not want_logprobs:
            ops.argmax_rows(logits, tokens)
            return PendingSample(tokens, None)
        table = np.array([[p.temperature, p.top_k, p.top_p, p.min_p, p.repetition_penalty] for p in params],
                         dtype=np.float32)
        keys = np.array([[s, c] for s, c in zip(seeds, counters)], dtype=np.int64)
        # one copy from page-locked memory carries every per-row number, so the host goes on while
        # the step's kernels still run
        arrays = [keys, table]
        if generated is not None and any(p.repetition_penalty != 1.0 for p in params):
            # the penalty applies once per distinct generated id (sampling.py:55)
            lists = [sorted(set(g)) if p.repetition_penalty != 1.0 else [] for g, p in zip(generated, params)]
            offsets = np.zeros(m + 1, dtype=np.int32)
            offsets[1:] = np.cumsum([len(x) for x in lists])
            flat = np.array([t for x in lists for t in x], dtype=np.int32)
            if flat.size:
                arrays += [flat, offsets]
        on_device = pack_words(arrays, logits.device)
        pen_ids, pen_off = (on_device[2], on_device[3]) if len(on_device) == 4 else (None, None)
        logprobs = torch.empty(m, dtype=torch.float32, device=logits.device)
        truncations = any(not p.greedy and (p.top_k > 0 or p.top_p < 1.0) for p in params)
        ops.sample_rows(logits, on_device[1], on_device[0], pen_ids, pen_off, tokens, logprobs, truncations=truncations)
        return PendingSample(tokens, logprobs)

    @staticmethod
    def finish(pending: "PendingSample"):
        """Waits for a started sampling (and for nothing enqueued after it) and returns
        (tokens, logprobs) as Python lists."""
        return pending.read()


class PendingSample:
    """A sampling whose results are on their way to the host."""

    def __init__(self, tokens: torch.Tensor, logprobs: Optional[torch.Tensor]):
        self.tokens = tokens                # int32 [m] on the device
        self.logprobs = logprobs
        self._host_tokens = self._host_logprobs = self._event = None
        if tokens.is_cuda:
            # into pinned memory, with an event after the copies: reading them later does not wait
            # for work that was enqueued after this sampling
            self._host_tokens = torch.empty(tokens.shape, dtype=tokens.dtype, pin_memory=True)
            self._host_tokens.copy_(tokens, non_blocking=True)
            if logprobs is not None:
                self._host_logprobs = torch.empty(logprobs.shape, dtype=logprobs.dtype, pin_memory=True)
                self._host_logprobs.copy_(logprobs, non_blocking=True)
            self._event = torch.cuda.Event()
            self._event.record()

    def read(self):
        if self._event is None:
            return self.tokens.tolist(), (self.logprobs.tolist() if self.logprobs is not None else None)
        self._event.synchronize()
        return (self._host_tokens.tolist(),
                self._host_logprobs.tolist() if self._host_logprobs is not None else None)
