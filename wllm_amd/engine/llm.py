"""The Python entry point: token ids in, token ids out.

The reference has no such class; programmatic use there is a `Scheduler` over a model
and a cache, `add_request` and `run_to_completion`
(tests/test_gemma_architecture.py:119-122), with the server's options
(src/wllm/cli.py:21-56, src/wllm/api/server.py:124-145) as constructor arguments.
`LLM` bundles exactly that and keeps the reference's names for the options it has:
`num_blocks`, `block_size`, `dtype`, `max_prefill_tokens_per_step`.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional, Sequence, Union

from wllm_amd.engine.request import Request
from wllm_amd.engine.runner import ModelRunner
from wllm_amd.engine.scheduler import Scheduler
from wllm_amd.parts.model import load_model
from wllm_amd.sampling.params import SamplingParams


@dataclass
class RequestOutput:
    request_id: object
    prompt_token_ids: list
    token_ids: list
    logprobs: list
    finish_reason: Optional[str]
    num_preemptions: int = 0


class LLM:
    def __init__(self, model: str, dtype: str = "bfloat16", device: str = "cuda", num_blocks: int = 256,
                 block_size: int = 16, max_prefill_tokens_per_step: Optional[int] = None, max_requests: int = 64,
                 admission: str = "pledged", seed: int = 0, hip_graphs: bool = False,
                 decode_weight_copy: Optional[bool] = None, lookahead: bool = True,
                 step_row_multiple: Optional[int] = 256):
        """`model`: a folder with config.json and model.safetensors.  `num_blocks` pages of
        `block_size` tokens make the cache pool.  `max_prefill_tokens_per_step` enables
        chunked prefill.  `hip_graphs` replays captured graphs for decode-only steps.
        `decode_weight_copy` keeps a second copy of the matrices in the order the decode
        kernels read fastest (default: yes; costs the matrices' memory once more).
        `lookahead` starts each step before the tokens of the step before it have been read, so the
        GPU does not wait for the host between steps; what is generated is the same.
        `step_row_multiple`: under chunked prefill a portion that the budget cuts is shortened so that
        the step's rows are a multiple of this (the library's products of many rows work in tiles of
        256 rows: 530 rows cost a fifth more than 512); None leaves portions as the budget cuts them."""
        self.model = load_model(model, dtype, device, tiled_copies=decode_weight_copy)
        self.runner = ModelRunner.create(self.model, num_pages=num_blocks, page_size=block_size,
                                         max_requests=max_requests)
        if hip_graphs:
            self.runner.enable_graphs()
        self.scheduler = Scheduler(self.runner, max_prefill_tokens_per_step, admission=admission, seed=seed,
                                   lookahead=lookahead, row_multiple=step_row_multiple)
        self._next_id = 0

    def generate(self, prompt_token_ids: Sequence[Sequence[int]],
                 sampling_params: Union[None, SamplingParams, Sequence[SamplingParams]] = None,
                 max_new_tokens: Union[int, Sequence[int]] = 16, eos_token_id: Optional[int] = None,
                 stop_token_ids: Sequence[int] = ()) -> list:
        """Generates for all prompts together (continuous batching) and returns one
        `RequestOutput` per prompt, in the order of the prompts."""
        n = len(prompt_token_ids)
        if sampling_params is None or isinstance(sampling_params, SamplingParams):
            sampling_params = [sampling_params or SamplingParams()] * n
        if isinstance(max_new_tokens, int):
            max_new_tokens = [max_new_tokens] * n
        if len(sampling_params) != n or len(max_new_tokens) != n:
            raise ValueError("one SamplingParams and one max_new_tokens per prompt, or one for all")
        requests = []
        for prompt, sp, mx in zip(prompt_token_ids, sampling_params, max_new_tokens):
            r = Request(self._next_id, [int(t) for t in prompt], int(mx), eos_token_id,
                        frozenset(int(t) for t in stop_token_ids), sp)
            self._next_id += 1
            requests.append(r)
        for r in requests:
            self.scheduler.add_request(r)
        self.scheduler.run_to_completion()
        return [RequestOutput(r.request_id, r.prompt_token_ids, list(r.output_token_ids), list(r.logprobs),
                              r.finish_reason, r.num_preemptions) for r in requests]
