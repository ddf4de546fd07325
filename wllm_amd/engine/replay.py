"""Trace replay: given token ids fed through the model step by step, logits out.

A trace is a sequence of steps; a step is
    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}
All entries of a step are one batch.  A request is opened when its id is first
seen and closed, its pages and slot given back, when a step's `end` names it.
Nothing is sampled.  The replayer drives the same `ModelRunner.step` and cache
manager as generation does; it has no forward pass of its own.
"""
from __future__ import annotations

from typing import Optional

import torch

from wllm_amd.engine.batch import StepEntry
from wllm_amd.engine.runner import ModelRunner


class TraceError(ValueError):
    """A trace step is malformed."""


def pages_for_max_tokens(max_tokens: int, page_size: int, live_requests: int = 4) -> int:
    """`max_tokens` is the most tokens live requests hold at any time, each request's
    count rounded up to a multiple of 64; a pool of that many tokens' pages holds them
    when the page size divides 64, and a larger page rounds up to itself."""
    if page_size <= 0 or max_tokens <= 0:
        raise ValueError("max_tokens and page_size must be positive")
    if 64 % page_size == 0:
        return -(-max_tokens // page_size)
    return -(-max_tokens // page_size) + live_requests


class TraceReplayer:
    def __init__(self, runner: ModelRunner):
        self.runner = runner

    def run_step(self, step: dict) -> Optional[torch.Tensor]:
        """Runs one step; returns float32 logits [wanted, vocab] or None if nothing is wanted."""
        if not isinstance(step, dict) or "entries" not in step:
            raise TraceError("a step is an object with 'entries'")
        entries = []
        for raw in step["entries"]:
            try:
                rid, tokens = raw["id"], [int(t) for t in raw["tokens"]]
                want = [int(w) for w in raw.get("want", [])]
            except (KeyError, TypeError, ValueError) as e:
                raise TraceError(f"malformed entry {raw!r}: {e}") from e
            if not self.runner.cache.is_open(rid):
                self.runner.open(rid)
            entries.append(StepEntry(rid, tokens, want))
        logits = self.runner.step(entries) if entries else None
        wanted = sum(len(e.want) for e in entries)
        result = logits.clone() if (logits is not None and wanted) else None
        for rid in step.get("end", []) or []:
            if self.runner.cache.is_open(rid):
                self.runner.close(rid)
        return result
