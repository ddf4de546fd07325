"""The scheduler's decisions, on the CPU: the kernels are replaced by their plain
emulation, the model is a tiny random one, and the tokens are compared with the plain
implementation's full recomputation."""
import pytest
import torch

from helpers import assert_varied, random_ids
from kernel_emulation import EmulatedKernels
from plain import gemma_plain
from wllm_amd.cache import OutOfPages
from wllm_amd.engine import ModelRunner, Request, RequestRefused, RequestStatus, Scheduler
from wllm_amd.kernels import ops
from wllm_amd.parts import load_model
from wllm_amd.sampling import SamplingParams


@pytest.fixture(autouse=True)
def emulated():
    with ops.use_backend(EmulatedKernels()):
        yield


@pytest.fixture(scope="module")
def tiny(varied_folders):
    # weights large enough that greedy decoding does not just repeat the last prompt token
    folder = varied_folders["AV"]
    with ops.use_backend(EmulatedKernels()):
        model = load_model(folder, "float32", "cpu")
    cfg = gemma_plain.read_config(folder)
    w = gemma_plain.read_weights(folder, torch.float32)
    return model, cfg, w


def make(model, num_pages=64, page_size=4, max_requests=8, **kw):
    runner = ModelRunner.create(model, num_pages=num_pages, page_size=page_size, max_requests=max_requests)
    return Scheduler(runner, **kw)


def prompts_of(lengths, seed=0):
    return [random_ids(seed + 17 * i, n, 512) for i, n in enumerate(lengths)]


def test_batched_generation_equals_each_request_alone_and_the_plain_implementation(tiny):
    # the reference's continuous-batching test (tests/test_scheduler.py:53-91) and its paged-serving
    # test (tests/test_gemma_architecture.py:106-124): prompts 7/16/23, 8 greedy tokens, pages of 4
    model, cfg, w = tiny
    prompts = prompts_of([7, 16, 23])
    s = make(model)
    for i, p in enumerate(prompts):
        s.add_request(Request(i, p, 8))
    together = {r.request_id: r.output_token_ids for r in s.run_to_completion()}
    for i, p in enumerate(prompts):
        alone = make(model)
        alone.add_request(Request(0, p, 8))
        assert alone.run_to_completion()[0].output_token_ids == together[i]
        assert gemma_plain.generate_greedy(cfg, w, p, 8) == together[i]
        assert_varied(together[i])
    s.cache.check()
    assert s.cache.num_free_pages(0) == 64


def test_chunked_prefill_gives_the_same_tokens_and_takes_the_steps_it_should(tiny):
    # tests/test_chunked_prefill_scheduler.py:47-152: budget 8 takes at least len // 8 steps;
    # budget 6 gives the tokens of the unchunked run; a long prompt is PREFILLING after one step
    model, cfg, w = tiny
    prompt = prompts_of([50])[0]
    plain = gemma_plain.generate_greedy(cfg, w, prompt, 5)
    for budget in (None, 6, 8, 1):
        s = make(model, max_prefill_tokens_per_step=budget)
        r = Request(0, prompt, 5)
        s.add_request(r)
        s.step()
        if budget is not None:
            assert r.status == RequestStatus.PREFILLING and r.output_token_ids == []
            assert r.num_computed == budget
        s.run_to_completion()
        assert r.output_token_ids == plain
        if budget:
            assert s.stats["steps"] >= 50 // budget + 4
            assert s.stats["prefill_tokens"] == 50 and s.stats["decode_tokens"] == 4


def test_portions_run_beside_decoded_tokens_in_one_batch(tiny):
    model, cfg, w = tiny
    short, long_ = prompts_of([5, 40])
    s = make(model, max_prefill_tokens_per_step=8)
    seen = []
    real_step = s.runner.step
    s.runner.step = lambda entries: (seen.append([(e.request, len(e.tokens), list(e.want)) for e in entries]), real_step(entries))[1]
    s.add_request(Request("short", short, 10))
    s.step()                       # short is prefilled whole (5 <= 8) and gets its first token
    s.add_request(Request("long", long_, 3))
    s.run_to_completion()
    mixed = [b for b in seen if len(b) == 2 and {n for _, n, _ in b} != {1}]
    assert mixed, "some step held a decoded token and a prompt portion"
    assert mixed[0] == [("short", 1, [0]), ("long", 8, [])], "decodes first, then the portion; no logits inside a prompt"
    # the budget counts prompt tokens only: the decode rides free
    assert all(sum(n for _, n, _ in b if n > 1) <= 8 for b in seen)
    # first token comes from the portion that completes the prompt; that request does not decode in the same step
    last_portion = [b for b in seen if any(rid == "long" and n > 1 for rid, n, _ in b)][-1]
    assert [x for x in last_portion if x[0] == "long"] == [("long", 8, [7])]


def test_first_come_first_served_admission_with_pledged_pages(tiny):
    # tests/test_scheduler.py:94-112: two pages of 16; two requests of 10 + 20 need two pages each
    model, _, _ = tiny
    s = make(model, num_pages=2, page_size=16)
    a, b = Request("a", prompts_of([10])[0], 20), Request("b", prompts_of([10], 5)[0], 20)
    s.add_request(a)
    s.add_request(b)
    s.step()
    assert a.status == RequestStatus.RUNNING and b.status == RequestStatus.WAITING
    assert s.stats["admission_waits"] >= 1
    done = s.run_to_completion()
    assert [r.request_id for r in done] == ["a", "b"], "b runs once a's pages are back"
    assert len(a.output_token_ids) == 20 and len(b.output_token_ids) == 20
    assert s.stats["preemptions"] == 0


def test_head_of_the_queue_is_not_skipped(tiny):
    model, _, _ = tiny
    s = make(model, num_pages=6, page_size=4)
    s.add_request(Request("running", prompts_of([8])[0], 8))        # 4 pages pledged
    s.step()
    s.add_request(Request("big", prompts_of([12], 3)[0], 8))         # 5 pages: does not fit beside it
    s.add_request(Request("small", prompts_of([2], 4)[0], 2))        # 1 page: would fit, but waits its turn
    s.step()
    assert [r.request_id for r in s.waiting] == ["big", "small"]


def test_requests_that_can_never_run_are_refused(tiny):
    model, _, _ = tiny
    s = make(model, num_pages=4, page_size=4)
    with pytest.raises(RequestRefused, match="pages"):
        s.add_request(Request(0, prompts_of([10])[0], 10))
    with pytest.raises(RequestRefused, match="positions"):
        make(model, num_pages=64).add_request(Request(0, prompts_of([100])[0], 40))   # max_position 128
    with pytest.raises(RequestRefused):
        s.add_request(Request(1, [], 3))


def test_running_out_of_pages_preempts_the_request_admitted_last(tiny):
    """Only the prompt must fit at admission; decoding then runs the pool dry.  The victim gives
    its pages back, goes to the front of the queue with its outputs kept, recomputes, and ends
    with the tokens it would have had."""
    model, cfg, w = tiny
    prompts = prompts_of([8, 8, 8])
    expected = [gemma_plain.generate_greedy(cfg, w, p, 12) for p in prompts]
    s = make(model, num_pages=10, page_size=4, admission="prompt_only")
    reqs = [Request(i, p, 12) for i, p in enumerate(prompts)]
    for r in reqs:
        s.add_request(r)
    first_victim = None
    for _ in range(200):
        if not s.has_unfinished_requests():
            break
        before = s.stats["preemptions"]
        free_before = s.cache.num_free_pages(0)
        s.step()
        if s.stats["preemptions"] > before and first_victim is None:
            first_victim = s.waiting[0]
            assert first_victim.request_id == 2, "the request admitted last is the victim"
            assert first_victim.status == RequestStatus.WAITING and first_victim.num_computed == 0
            assert len(first_victim.output_token_ids) > 0, "what it generated is kept"
            assert not s.cache.is_open(2)
        s.cache.check()
    assert s.stats["preemptions"] >= 1 and first_victim is not None
    assert [r.output_token_ids for r in reqs] == expected
    assert s.cache.num_free_pages(0) == 10


def test_out_of_pages_with_one_request_left_is_an_error_not_a_loop(tiny):
    model, _, _ = tiny
    s = make(model, num_pages=4, page_size=4)
    r = Request(0, prompts_of([6])[0], 6)
    s.add_request(r)
    s.step()
    # take the free pages away behind the scheduler's back (the reference's test drains the
    # allocator by hand, tests/test_scheduler.py:133-137)
    pool = s.cache.groups[0].pool
    while pool.num_free:
        pool.allocate("thief")
    with pytest.raises(OutOfPages):
        for _ in range(10):
            s.step()


def test_cancel(tiny):
    # tests/test_scheduler.py:150-184
    model, _, _ = tiny
    s = make(model, num_pages=8, page_size=16)
    s.add_request(Request("a", prompts_of([10])[0], 20))
    s.step()
    assert s.cache.num_free_pages(0) == 7
    s.cancel("a")
    assert s.cache.num_free_pages(0) == 8 and not s.running
    s.add_request(Request("b", prompts_of([10])[0], 20))
    s.cancel("b")
    assert not s.waiting
    s.cancel("nobody")


def test_finishing_rules(tiny):
    # src/wllm/engine/sequence.py:53-59
    model, cfg, w = tiny
    prompt = prompts_of([9])[0]
    plain = gemma_plain.generate_greedy(cfg, w, prompt, 6)
    assert len(set(plain[:3])) == 3, "the stops below are in the middle of what is generated"
    s = make(model)
    one = Request("one", prompt, 1)
    s.add_request(one)
    s.step()
    assert one.is_finished() and one.output_token_ids == plain[:1] and one.finish_reason == "length"
    assert not s.running and s.cache.num_free_pages(0) == 64, "a prefill alone can finish a request"
    eos = Request("eos", prompt, 6, eos_token_id=plain[2])
    stop = Request("stop", prompt, 6, stop_token_ids=frozenset([plain[1]]))
    s.add_request(eos)
    s.add_request(stop)
    s.run_to_completion()
    cut = plain.index(plain[2]) + 1
    assert eos.output_token_ids == plain[:cut] and eos.finish_reason == "stop", "the end token is kept"
    assert stop.output_token_ids == plain[:plain.index(plain[1]) + 1]


def test_seeded_sampling_does_not_depend_on_the_batch(tiny):
    model, _, _ = tiny
    prompts = prompts_of([5, 31, 12])
    params = [SamplingParams(temperature=0.8, seed=100 + i) for i in range(3)]
    s = make(model, max_prefill_tokens_per_step=16)
    reqs = [Request(i, p, 6, sampling_params=sp) for i, (p, sp) in enumerate(zip(prompts, params))]
    for r in reqs:
        s.add_request(r)
    s.run_to_completion()
    for r, p, sp in zip(reqs, prompts, params):
        alone = make(model)
        a = Request("x", p, 6, sampling_params=sp)
        alone.add_request(a)
        alone.run_to_completion()
        assert a.output_token_ids == r.output_token_ids
        assert all(lp is not None and lp <= 0 for lp in r.logprobs)
    greedy = make(model)
    g = Request("g", prompts[1], 6)
    greedy.add_request(g)
    greedy.run_to_completion()
    assert g.output_token_ids != reqs[1].output_token_ids, "temperature 0.8 does not give the greedy tokens here"


def test_every_admitted_request_finishes_and_no_page_is_lost(tiny):
    model, _, _ = tiny
    g = torch.Generator().manual_seed(5)
    for admission in ("pledged", "prompt_only"):
        s = make(model, num_pages=24, page_size=4, max_requests=4, max_prefill_tokens_per_step=10,
                 admission=admission)
        reqs = []
        for i in range(10):
            n = int(torch.randint(1, 40, (1,), generator=g))
            mx = int(torch.randint(1, 20, (1,), generator=g))
            reqs.append(Request(i, random_ids(i, n, 512), mx))
            s.add_request(reqs[-1])
        steps = 0
        while s.has_unfinished_requests():
            s.step()
            s.cache.check()
            assert len(s.running) <= 4
            steps += 1
            assert steps < 2000
        assert all(r.is_finished() and len(r.output_token_ids) == r.max_new_tokens for r in reqs)
        assert s.cache.num_free_pages(0) == 24 and not s.cache.requests


def _workload(seed, count=9):
    """Requests of mixed lengths; a third stop on a token that greedy decoding will produce."""
    g = torch.Generator().manual_seed(seed)
    reqs = []
    for i in range(count):
        n = int(torch.randint(1, 40, (1,), generator=g))
        mx = int(torch.randint(1, 16, (1,), generator=g))
        kind = i % 3
        sp = SamplingParams(temperature=0.9, top_k=20, seed=7 + i) if kind == 1 else SamplingParams()
        reqs.append(dict(request_id=i, prompt_token_ids=random_ids(seed * 100 + i, n, 512), max_new_tokens=mx,
                         sampling_params=sp))
    return reqs


@pytest.mark.parametrize("admission,pages", [("pledged", 40), ("prompt_only", 16)])
def test_looking_ahead_gives_every_request_the_same_tokens(tiny, admission, pages):
    """A step started before the step before it was read: the tokens come from the device, stops on
    an end token are seen one step late and the extra token is dropped."""
    model, _, _ = tiny
    specs = _workload(3)
    results = {}
    for lookahead in (False, True):
        # first without stop tokens, to learn what is generated; then stop in the middle of that
        plain_run = make(model, num_pages=pages, page_size=4, max_requests=4, max_prefill_tokens_per_step=10,
                         admission=admission, lookahead=lookahead)
        first = [Request(**spec) for spec in specs]
        for r in first:
            plain_run.add_request(r)
        done = plain_run.run_to_completion()
        assert sorted(r.request_id for r in done) == list(range(len(specs))), "each request is handed back once, complete"
        assert all(r.is_complete() for r in done)
        s = make(model, num_pages=pages, page_size=4, max_requests=4, max_prefill_tokens_per_step=10,
                 admission=admission, lookahead=lookahead)
        reqs = []
        for spec, done in zip(specs, first):
            out = done.output_token_ids
            extra = {}
            if spec["request_id"] % 3 == 0 and len(out) >= 3:
                extra = dict(eos_token_id=out[len(out) // 2])
            elif spec["request_id"] % 3 == 2 and len(out) >= 2:
                extra = dict(stop_token_ids=frozenset([out[-2]]))
            reqs.append(Request(**spec, **extra))
            s.add_request(reqs[-1])
        steps = 0
        while s.has_unfinished_requests():
            s.step()
            s.cache.check()
            steps += 1
            assert steps < 3000
        assert all(r.is_finished() for r in reqs)
        assert s.cache.num_free_pages(0) == pages and not s.cache.requests, "every page came back"
        for r in reqs:
            assert len(r.output_token_ids) == len(r.logprobs) <= r.max_new_tokens
            if r.finish_reason == "stop":
                assert r.ends_with(r.output_token_ids[-1]) and not any(r.ends_with(t) for t in r.output_token_ids[:-1])
        results[lookahead] = ([r.output_token_ids for r in reqs], [r.finish_reason for r in reqs],
                              [r.output_token_ids for r in first], s.stats["preemptions"])
    assert results[True][:3] == results[False][:3]
    assert any(reason == "stop" for reason in results[True][1]), "the workload has requests that stop early"
    assert any(reason == "stop" and len(out) > 1 for out, reason in zip(*results[True][:2])), "and not only at once"
    for out in results[True][2]:
        assert_varied(out, least=3)
    if admission == "prompt_only":
        assert results[True][3] > 0, "the small pool forces preemptions"


@pytest.mark.parametrize("sampled", [False, True])
def test_a_stop_at_any_output_index_ends_the_request_there_with_and_without_looking_ahead(tiny, sampled):
    """The token that stops a request may come at any place among its outputs, the last but one
    (where the step run ahead has already filled the request's length and closed it) and the last
    included: the request ends with that token and "stop", and every page comes back."""
    model, _, _ = tiny
    prompt = prompts_of([11], 4)[0]
    sp = SamplingParams(temperature=1.0, seed=77) if sampled else SamplingParams()
    max_new = 6
    free = make(model, lookahead=False)
    r = Request("free", prompt, max_new, sampling_params=sp)
    free.add_request(r)
    free.run_to_completion()
    out = list(r.output_token_ids)
    assert len(set(out)) == max_new, f"every output token is its own stop: {out}"
    for index in range(max_new):
        for lookahead in (False, True):
            for other in (False, True):      # alone, and beside a request that keeps the batch going
                s = make(model, lookahead=lookahead)
                stop = Request("stop", prompt, max_new, sampling_params=sp, stop_token_ids=frozenset([out[index]]))
                s.add_request(stop)
                if other:
                    s.add_request(Request("other", prompts_of([5], 3)[0], 12))
                s.run_to_completion()
                assert stop.output_token_ids == out[:index + 1], (index, lookahead, other)
                assert stop.finish_reason == "stop" and len(stop.logprobs) == index + 1 and stop.num_unread == 0
                s.cache.check()
                assert s.cache.num_free_pages(0) == 64 and not s.cache.requests


def test_a_request_that_needs_the_page_set_aside_for_graphs_is_refused_when_added(tiny):
    """Captured graphs keep one page per group for their padding rows; a request that would need
    every page of the pool can then never be admitted and is refused at once instead of waiting
    for ever (the reference's scheduler would spin to its step limit, scheduler.py:228-236,500-506)."""
    model, _, _ = tiny
    s = make(model, num_pages=8, page_size=4)
    s.runner.enable_graphs()
    assert s.cache.usable_pages(0) == 7
    with pytest.raises(RequestRefused, match="pages"):
        s.add_request(Request("all", prompts_of([24])[0], 8))      # 32 tokens: 8 pages
    fits = Request("fits", prompts_of([20])[0], 8)                  # 28 tokens: 7 pages
    s.add_request(fits)
    assert not s.waiting[0].is_finished()


def test_a_request_at_the_head_of_the_queue_that_can_never_fit_is_an_error_not_a_wait(tiny):
    """Nothing runs, so no page can come back, and the head of the queue does not fit: the step
    raises and names the request; the requests behind it are served afterwards."""
    model, cfg, w = tiny
    s = make(model, num_pages=6, page_size=4)
    pool = s.cache.groups[0].pool
    for _ in range(3):
        pool.allocate("thief")        # pages lost behind the scheduler's back
    s.add_request(Request("big", prompts_of([14])[0], 6))           # 5 pages of 3 free
    small = Request("small", prompts_of([4], 2)[0], 4)
    s.add_request(small)
    with pytest.raises(RequestRefused, match="'big'"):
        s.run_to_completion(max_steps=50)
    assert [r.request_id for r in s.waiting] == ["small"]
    s.run_to_completion()
    assert small.output_token_ids == gemma_plain.generate_greedy(cfg, w, small.prompt_token_ids, 4)


def test_run_to_completion_does_not_return_with_requests_unfinished(tiny):
    model, _, _ = tiny
    s = make(model)
    s.add_request(Request("long", prompts_of([9])[0], 30))
    with pytest.raises(RuntimeError, match="did not finish"):
        s.run_to_completion(max_steps=5)
    s.run_to_completion()
    assert not s.has_unfinished_requests()


def test_looking_ahead_starts_the_next_step_before_the_tokens_are_read(tiny):
    model, cfg, w = tiny
    prompt = prompts_of([9])[0]
    s = make(model, lookahead=True)
    fed = []
    real_step = s.runner.step
    def spy(entries, feed_tokens=None):
        fed.append([e.feed_row for e in entries])
        return real_step(entries, feed_tokens)
    s.runner.step = spy
    r = Request("r", prompt, 5)
    s.add_request(r)
    got = s.step()
    # the prompt's step and the first decode step have both been started; only the first was read
    assert len(fed) == 2 and fed[1] == [0] and got == [r]
    assert len(r.output_token_ids) == 2 and r.logprobs[1] is None, "the second token is a placeholder still"
    s.run_to_completion()
    assert r.output_token_ids == gemma_plain.generate_greedy(cfg, w, prompt, 5)
    assert [rows for rows in fed[1:]] == [[0]] * 4, "four decode steps, each fed from the device"


def test_a_repetition_penalty_is_never_run_ahead(tiny):
    model, _, _ = tiny
    prompt = prompts_of([12])[0]
    outs = []
    for lookahead in (False, True):
        s = make(model, lookahead=lookahead)
        r = Request("p", prompt, 8, sampling_params=SamplingParams(repetition_penalty=1.3))
        s.add_request(r)
        while s.has_unfinished_requests():
            s.step()
            assert s._started is None, "a penalised request waits for its tokens"
        outs.append(r.output_token_ids)
    assert outs[0] == outs[1]


def test_a_steps_rows_are_trimmed_to_the_products_tiles_where_the_budget_cuts_anyway(tiny):
    """With `row_multiple`, a portion that the budget cuts is shortened so that the step's rows
    (decoded tokens and prompt tokens) are a multiple of it; a portion that ends its prompt is not,
    and the tokens are the same either way."""
    model, cfg, w = tiny
    prompts = prompts_of([5, 6, 7, 90])
    outs = {}
    for multiple in (None, 8):
        s = make(model, num_pages=96, max_prefill_tokens_per_step=16, row_multiple=multiple)
        seen = []
        real_step = s.runner.step
        s.runner.step = lambda entries, *a, real=real_step, log=seen: (
            log.append([len(e.tokens) for e in entries]), real(entries, *a))[1]
        for i, p in enumerate(prompts[:3]):
            s.add_request(Request(i, p, 30))
        s.step()
        s.step()                                    # three requests decode
        s.add_request(Request(3, prompts[3], 4))
        done = s.run_to_completion()
        outs[multiple] = {r.request_id: r.output_token_ids for r in done}
        mixed = [b for b in seen if max(b) > 1 and b.count(1) == 3]
        assert mixed, "portions of the long prompt ran beside three decoded tokens"
        if multiple is None:
            assert mixed[0] == [1, 1, 1, 16]
        else:
            # 3 + 16 rows would be 19: the portion gives 3 up; the last portion (90 = 13 * 6 + 12) ends
            # the prompt and is left alone
            assert mixed[0] == [1, 1, 1, 13] and all(sum(b) % 8 == 0 for b in mixed[:-1])
            assert sum(b[-1] for b in mixed) == 90 and sum(mixed[-1]) % 8 != 0
    assert outs[None] == outs[8]
