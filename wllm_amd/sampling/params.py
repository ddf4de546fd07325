"""Sampling parameters, with the reference's names, meanings and defaults
(src/wllm/engine/sampling.py:22-29): temperature 0.0 is greedy; top_k 0, top_p 1.0,
min_p 0.0 and repetition_penalty 1.0 switch their step off.  `seed` is honoured here
(the reference declares it and never uses it, src/wllm/api/server.py:76-81): with a
seed, a request's tokens are the same whatever else is in the batch."""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional


@dataclass(frozen=True)
class SamplingParams:
    temperature: float = 0.0
    top_k: int = 0
    top_p: float = 1.0
    min_p: float = 0.0
    repetition_penalty: float = 1.0
    seed: Optional[int] = None

    def __post_init__(self):
        if not self.temperature >= 0.0:
            raise ValueError(f"temperature must not be negative, got {self.temperature}")
        if self.top_k < 0:
            raise ValueError(f"top_k must not be negative, got {self.top_k}")
        if not 0.0 < self.top_p <= 1.0:
            raise ValueError(f"top_p must lie in (0, 1], got {self.top_p}")
        if not 0.0 <= self.min_p <= 1.0:
            raise ValueError(f"min_p must lie in [0, 1], got {self.min_p}")
        if not self.repetition_penalty > 0.0:
            raise ValueError(f"repetition_penalty must be positive, got {self.repetition_penalty}")

    @property
    def greedy(self) -> bool:
        return self.temperature == 0.0
