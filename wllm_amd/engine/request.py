"""A request and its life: waiting, prefilling, running, finished.

The states and the finishing rules are the reference's (src/wllm/engine/sequence.py:13-59):
a request finishes when it samples its end-of-sequence token or one of its stop tokens
(the token is kept in the output) or has `max_new_tokens` outputs; a prefill alone can
finish it.  One thing is organised differently: a request is one list of tokens, prompt
then outputs, with a count of how many of them are in the cache.  Feeding a prompt
portion, decoding, and recomputing after a preemption are then the same act: feed the
next tokens that are not in the cache yet, and sample when the last one has been fed.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from enum import Enum
from typing import Optional

from wllm_amd.sampling.params import SamplingParams


class RequestStatus(Enum):
    WAITING = "waiting"
    PREFILLING = "prefilling"
    RUNNING = "running"
    FINISHED = "finished"


@dataclass
class Request:
    request_id: object
    prompt_token_ids: list
    max_new_tokens: int
    eos_token_id: Optional[int] = None
    stop_token_ids: frozenset = frozenset()
    sampling_params: SamplingParams = field(default_factory=SamplingParams)
    output_token_ids: list = field(default_factory=list)
    logprobs: list = field(default_factory=list)
    status: RequestStatus = RequestStatus.WAITING
    finish_reason: Optional[str] = None
    num_computed: int = 0           # tokens of prompt + outputs that are in the cache
    num_preemptions: int = 0
    arrival_index: int = 0
    seed: int = 0
    num_unread: int = 0             # outputs that were sampled on the device and have not been read yet

    @property
    def num_prompt_tokens(self) -> int:
        return len(self.prompt_token_ids)

    @property
    def num_tokens(self) -> int:
        return len(self.prompt_token_ids) + len(self.output_token_ids)

    @property
    def total_len_estimate(self) -> int:
        """The most tokens the request can ever hold (sequence.py:39-44)."""
        return self.num_prompt_tokens + self.max_new_tokens

    def tokens(self, begin: int, end: int) -> list:
        p = self.prompt_token_ids
        if end <= len(p):
            return p[begin:end]
        return (p[begin:] if begin < len(p) else []) + self.output_token_ids[max(0, begin - len(p)):end - len(p)]

    def is_finished(self) -> bool:
        return self.status == RequestStatus.FINISHED

    def is_complete(self) -> bool:
        """Finished, and every output has its value."""
        return self.status == RequestStatus.FINISHED and self.num_unread == 0

    def append_token(self, token: int, logprob: Optional[float]) -> None:
        """sequence.py:53-59."""
        self.output_token_ids.append(int(token))
        self.logprobs.append(logprob)
        if self.ends_with(token):
            self.status, self.finish_reason = RequestStatus.FINISHED, "stop"
        elif len(self.output_token_ids) >= self.max_new_tokens:
            self.status, self.finish_reason = RequestStatus.FINISHED, "length"

    def ends_with(self, token: int) -> bool:
        """Whether sampling this token ends the request whatever its length."""
        return (self.eos_token_id is not None and token == self.eos_token_id) or token in self.stop_token_ids

    def append_placeholder(self) -> int:
        """Room for a token that has been sampled on the device and not been read yet; returns its
        index among the outputs.  Only the length rule can be applied before the value is known."""
        self.output_token_ids.append(0)
        self.logprobs.append(None)
        self.num_unread += 1
        if len(self.output_token_ids) >= self.max_new_tokens:
            self.status, self.finish_reason = RequestStatus.FINISHED, "length"
        return len(self.output_token_ids) - 1
