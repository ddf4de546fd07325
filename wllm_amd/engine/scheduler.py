"""The scheduler: admits requests, cuts prompts into portions under a token budget,
decodes, finishes and frees.

It keeps the reference's policy (src/wllm/engine/scheduler.py:178-274,384-506):
first come, first served, never skipping the head of the queue; a request is admitted
if the pages its prompt and all its outputs can ever need fit into what is free minus
what running requests are still pledged; the budget `max_prefill_tokens_per_step`
counts prompt tokens only (decoded tokens are free) and is shared first by the requests
already prefilling, in order, then by new admissions; the token that ends a prompt is
sampled from the portion that completes it, and that request does not decode in the same
step, so every request gets at most one token per step; pages are given back at the end
of the step in which a request finished.

What differs.  One step is one batch: the portions and the decoded tokens run together
in one call of the step function (the reference runs each portion alone and then one
decode batch, scheduler.py:465-498).  "Used" pages are the pages a request really holds
(the reference counts a prefilling request's whole prompt as used though only part is
allocated, scheduler.py:17-21,186-189).  A request that can never fit is refused when it
is added instead of waiting for ever.

When pages run out.  With the pledge accounting they cannot: every admitted request has
its worst case set aside.  With `admission="prompt_only"` (only the prompt must fit at
admission) they can, and then the step function raises `OutOfPages` before anything ran;
the scheduler takes the request admitted last (scheduler.py:424), gives back its pages
and puts it at the front of the queue (scheduler.py:293-305), and tries the step again
without it.  The preempted request keeps the tokens it generated and recomputes prompt
and outputs when it is admitted again (the reference drops the outputs,
scheduler.py:303), so that a seeded request gives the same tokens with or without a
preemption.

Looking ahead.  With `lookahead=True` a step is started before the tokens of the step before it
have been read: the sampled tokens stay on the device, the next step takes them from there
(`StepEntry.feed_row`), and the host reads them while that step runs, so the GPU does not wait
for the host between steps.  Whether a request ended on its end-of-sequence or a stop token is
then known one step late: the request has been given one more token, which is dropped, and its
pages go back one step later.  What each request generates is the same.  A request whose
sampling needs the tokens it generated (a repetition penalty) is never run ahead.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Optional

from wllm_amd.cache.pages import OutOfPages
from wllm_amd.engine.batch import StepEntry
from wllm_amd.engine.request import Request, RequestStatus
from wllm_amd.sampling.sampler import Sampler


class RequestRefused(ValueError):
    """A request that can never run: too long for the model or for the page pool."""


@dataclass
class _StartedStep:
    """A step whose sampling has been enqueued and not been read."""
    sampled: list                       # the requests that sample in it, in the order of its logits rows
    places: list                        # for each, the index among its outputs that the token will fill
    pending: object                     # the sampler's handle: tokens on the device, on their way to the host
    dropped: set = field(default_factory=set)     # rows whose request ended before this step's token counted


class Scheduler:
    def __init__(self, runner, max_prefill_tokens_per_step: Optional[int] = None, admission: str = "pledged",
                 seed: int = 0, compute_logprobs: bool = True, lookahead: bool = False,
                 row_multiple: Optional[int] = None):
        if admission not in ("pledged", "prompt_only"):
            raise ValueError(f"admission {admission!r}: expected 'pledged' or 'prompt_only'")
        if max_prefill_tokens_per_step is not None and max_prefill_tokens_per_step <= 0:
            raise ValueError("max_prefill_tokens_per_step must be positive or None")
        self.runner = runner
        self.cache = runner.cache
        self.max_prefill_tokens_per_step = max_prefill_tokens_per_step
        # A step's rows (decoded tokens and prompt tokens) are trimmed to a multiple of this where a
        # portion is cut by the budget anyway: the library's products of many rows work in tiles of
        # rows, and a step of 530 rows costs as much as one of 768.
        self.row_multiple = row_multiple
        self.admission = admission
        self.compute_logprobs = compute_logprobs
        self.sampler = Sampler(runner.device, seed)
        self.lookahead = lookahead
        self._started: Optional[_StartedStep] = None      # the step that has been started and not been read
        self.waiting: list = []
        self.running: list = []           # PREFILLING and RUNNING, in the order of admission
        self._arrivals = 0
        self.stats = {"steps": 0, "prefill_tokens": 0, "decode_tokens": 0, "preemptions": 0,
                      "admission_waits": 0, "peak_pages": 0}

    # ---- requests ------------------------------------------------------------------
    def add_request(self, request: Request) -> None:
        if request.num_prompt_tokens == 0:
            raise RequestRefused(f"request {request.request_id!r} has an empty prompt")
        if request.max_new_tokens <= 0:
            raise RequestRefused(f"request {request.request_id!r}: max_new_tokens must be positive")
        limit = self.runner.model.plan.max_positions
        # the last sampled token is never fed, so it needs no position
        if request.total_len_estimate - 1 > limit:
            raise RequestRefused(f"request {request.request_id!r} may reach {request.total_len_estimate - 1} "
                                 f"positions; the model allows {limit}")
        for gi, g in enumerate(self.cache.groups):
            need = self.cache.pages_for(gi, request.total_len_estimate, self._longest_portion(request))
            usable = self.cache.usable_pages(gi)
            if need > usable:
                raise RequestRefused(f"request {request.request_id!r} needs {need} pages; the pool has {usable} "
                                     f"that a request can ever hold")
        request.arrival_index = self._arrivals
        request.seed = self.sampler.seed_of(request.sampling_params, self._arrivals)
        self._arrivals += 1
        request.status = RequestStatus.WAITING
        self.waiting.append(request)

    def has_unfinished_requests(self) -> bool:
        return bool(self.waiting or self.running or self._started is not None)

    def cancel(self, request_id) -> None:
        """Running: give back its pages; waiting: drop it; unknown: nothing (scheduler.py:158-176)."""
        if self._started is not None:
            for row, r in enumerate(self._started.sampled):
                if r.request_id == request_id and row not in self._started.dropped:
                    self._started.dropped.add(row)
                    r.num_unread -= 1
                    del r.output_token_ids[self._started.places[row]:], r.logprobs[self._started.places[row]:]
        for i, r in enumerate(self.running):
            if r.request_id == request_id:
                self.cache.close(request_id)
                self.running.pop(i)
                return
        for i, r in enumerate(self.waiting):
            if r.request_id == request_id:
                self.waiting.pop(i)
                return

    # ---- admission ----------------------------------------------------------------
    def _longest_portion(self, request: Request) -> int:
        return self.max_prefill_tokens_per_step or max(1, request.total_len_estimate)

    def _pledged(self, gi: int) -> int:
        """Pages running requests may still take beyond what they hold (scheduler.py:181-190)."""
        if self.admission != "pledged":
            return 0
        total = 0
        for r in self.running:
            worst = self.cache.pages_for(gi, r.total_len_estimate, self._longest_portion(r))
            held = sum(1 for p in self.cache.block_table(r.request_id, gi) if p >= 0)
            total += max(0, worst - held)
        return total

    def _fits(self, request: Request) -> bool:
        for gi in range(len(self.cache.groups)):
            if self.admission == "pledged":
                needed = self.cache.pages_for(gi, request.total_len_estimate, self._longest_portion(request))
            else:
                needed = self.cache.pages_for(gi, request.num_tokens, self._longest_portion(request))
            if needed > self.cache.num_free_pages(gi) - self._pledged(gi):
                return False
        return len(self.running) < self.cache.max_requests

    # ---- one step -------------------------------------------------------------------
    def _plan(self) -> list:
        """[(request, how many tokens to feed)] of this step: decodes of all running
        requests, then portions under the budget."""
        plan = []
        for r in self.running:
            if r.status == RequestStatus.RUNNING:
                plan.append((r, 1))
        budget = self.max_prefill_tokens_per_step
        unlimited = budget is None
        for r in self.running:
            if r.status != RequestStatus.PREFILLING:
                continue
            if not unlimited and budget <= 0:
                break
            remaining = r.num_tokens - r.num_computed
            take = remaining if unlimited else min(budget, remaining)
            plan.append((r, take))
            if not unlimited:
                budget -= take
        while self.waiting and (unlimited or budget > 0):
            r = self.waiting[0]
            if not self._fits(r):
                if not self.running:
                    # nothing holds a page that could come back: waiting would be for ever
                    self.waiting.pop(0)
                    raise RequestRefused(f"request {r.request_id!r} does not fit into the free pages although no "
                                         f"request is running; it can never be admitted")
                self.stats["admission_waits"] += 1
                break       # first come, first served: the head is not skipped
            self.waiting.pop(0)
            self.cache.open(r.request_id)
            r.status = RequestStatus.PREFILLING
            r.num_computed = 0
            self.running.append(r)
            remaining = r.num_tokens
            take = remaining if unlimited else min(budget, remaining)
            plan.append((r, take))
            if not unlimited:
                budget -= take
        if self.row_multiple and not unlimited and plan:
            rows = sum(n for _, n in plan)
            extra = rows % self.row_multiple
            r, take = plan[-1]
            cut_by_budget = r.status == RequestStatus.PREFILLING and r.num_tokens - r.num_computed > take
            if rows > self.row_multiple and extra and cut_by_budget and take - extra >= max(2, take // 2):
                plan[-1] = (r, take - extra)
        return plan

    def _preempt(self, request: Request) -> None:
        self.running.remove(request)
        self.cache.close(request.request_id)
        request.status = RequestStatus.WAITING
        request.num_computed = 0
        request.num_preemptions += 1
        self.waiting.insert(0, request)
        self.stats["preemptions"] += 1

    def step(self) -> list:
        """One batch.  Returns the requests that got a token."""
        if self._started is None:
            self._started = self._start(None)
            if self._started is None:
                return []
        current = self._started
        self._started = self._start(current) if self.lookahead and self._may_run_ahead(current) else None
        return self._finish(current)

    @staticmethod
    def _may_run_ahead(step: _StartedStep) -> bool:
        """Not past a request whose next sampling needs the token that has not been read."""
        return all(r.sampling_params.repetition_penalty == 1.0 for r in step.sampled)

    def _start(self, before: Optional[_StartedStep]) -> Optional[_StartedStep]:
        """Plans a step, runs it and enqueues its sampling; nothing is read.  `before` is the step
        that has been started and not been read: its tokens are taken from the device."""
        unread = {}
        if before is not None:
            unread = {id(r): row for row, r in enumerate(before.sampled) if row not in before.dropped}
        plan = self._plan()
        logits = None
        while plan:
            entries = []
            for r, take in plan:
                completes = r.num_computed + take == r.num_tokens
                # the last output of a request sampled in `before` is a placeholder on the host
                feed = unread.get(id(r)) if completes and r.output_token_ids else None
                entries.append(StepEntry(r.request_id, r.tokens(r.num_computed, r.num_computed + take),
                                         [take - 1] if completes else [], feed_row=feed))
            try:
                if any(e.feed_row is not None for e in entries):
                    logits = self.runner.step(entries, before.pending.tokens)
                else:
                    logits = self.runner.step(entries)
                break
            except OutOfPages:
                victim = self.running[-1]
                if len(self.running) == 1:
                    raise
                self._preempt(victim)
                plan = [(r, take) for r, take in plan if r is not victim]
        if not plan:
            return None
        self.stats["steps"] += 1
        held = sum(g.pool.num_pages - g.pool.num_free for g in self.cache.groups)
        self.stats["peak_pages"] = max(self.stats["peak_pages"], held)
        sampled = []
        for r, take in plan:
            if r.status == RequestStatus.RUNNING:
                self.stats["decode_tokens"] += take
            else:
                self.stats["prefill_tokens"] += take
            r.num_computed += take
            if r.num_computed == r.num_tokens:
                sampled.append(r)
        started = _StartedStep(sampled, [], None)
        if sampled:
            started.pending = self.sampler.start(
                logits, [r.sampling_params for r in sampled], [r.seed for r in sampled],
                [len(r.output_token_ids) for r in sampled], [r.output_token_ids for r in sampled],
                want_logprobs=self.compute_logprobs)
            for r in sampled:
                r.status = RequestStatus.RUNNING
                started.places.append(r.append_placeholder())       # may end the request by its length
        for r in [r for r in self.running if r.is_finished()]:
            self.cache.close(r.request_id)
        self.running = [r for r in self.running if not r.is_finished()]
        return started

    def _finish(self, step: _StartedStep) -> list:
        """Reads a started step's tokens and applies the rules that need their values."""
        if not step.sampled:
            return []
        tokens, logprobs = self.sampler.finish(step.pending)
        got = []
        for row, r in enumerate(step.sampled):
            if row in step.dropped:
                continue
            place = step.places[row]
            r.num_unread -= 1
            r.output_token_ids[place] = int(tokens[row])
            r.logprobs[place] = logprobs[row] if logprobs is not None else None
            got.append(r)
            if r.ends_with(tokens[row]):
                # sequence.py:53-59: the stop rules come before the length rule
                r.status, r.finish_reason = RequestStatus.FINISHED, "stop"
                # The request may have been run ahead: that token does not count, whether or not it
                # was the one that filled the request's length (and closed it in the step run ahead).
                ahead = self._started
                if ahead is not None:
                    for row2, r2 in enumerate(ahead.sampled):
                        if r2 is r and row2 not in ahead.dropped:
                            ahead.dropped.add(row2)
                            r.num_unread -= 1
                del r.output_token_ids[place + 1:], r.logprobs[place + 1:]
                if r in self.running:           # not there if its length had closed it already
                    self.running.remove(r)
                    self.cache.close(r.request_id)
                elif r in self.waiting:         # preempted after it was sampled
                    self.waiting.remove(r)
        return got

    def run_to_completion(self, max_steps: int = 1_000_000) -> list:
        """Steps until nothing is left (scheduler.py:500-506).  Ending with requests unfinished is an
        error, not a result."""
        finished = []
        for _ in range(max_steps):
            if not self.has_unfinished_requests():
                return finished
            finished.extend(r for r in self.step() if r.is_complete())
        if self.has_unfinished_requests():
            left = [r.request_id for r in self.running + self.waiting]
            raise RuntimeError(f"{max_steps} steps did not finish requests {left!r}")
        return finished
