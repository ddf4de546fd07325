"""Decode steps of many requests against the plain implementation: 17 to 130 live requests of unequal
lengths in one step, kernel by kernel and replayed from captured graphs of the default batch-size
buckets (with padding rows on the page set aside for them, and a drop of the live count across a
bucket's edge), and the mixed family with 24 live requests.  These are the shapes of a serving
batch: product kernels for 17 to 64 rows, the library's products above that, attention plans of
hundreds of work items in which requests of one and of several key chunks lie side by side.

The reference tests its graph decoder padded up to the next bucket against eager decoding
(tests/test_cuda_graph_decoder.py:74-100); here both are compared with the plain implementation."""
import numpy as np
import pytest
import torch

from helpers import (TINY, assert_varied, compare_replay, plain_for, max_live_tokens, random_ids, replay_and_collect,
                     trace_mixed)
from plain import gemma_plain
from wllm_amd.engine import LLM, ModelRunner
from wllm_amd.engine.replay import TraceReplayer, pages_for_max_tokens
from wllm_amd.parts import load_model

pytestmark = pytest.mark.gpu
_PLAIN = {}      # what the requests are compared with, made once per (model, requests, dtype)


def plain_of(key, cfg, folder, requests, dtype):
    if (key, dtype) not in _PLAIN:
        _PLAIN[(key, dtype)] = plain_for(cfg, folder, requests, dtype)
    return _PLAIN[(key, dtype)]
DECODED = 8
# live requests -> how many end half way, so that the count crosses the edge of a bucket of
# (1, 2, 4, 8, 16, 32, 48, 64, 128, 256): 17 -> 15, 48 -> 30, 64 -> 47, 65 -> 63, 130 -> 127
DROPS = {17: 2, 48: 18, 64: 17, 65: 2, 130: 3}


def many_requests(name: str, count: int, longest: int) -> dict:
    vocab = TINY[name]["config"].vocab_size
    rng = np.random.default_rng(count)
    lengths = rng.integers(3, longest + 1, size=count)
    lengths[:3] = (3, longest, longest // 2)          # the shortest and the longest are there
    return {f"r{i}": random_ids(1000 * count + i, int(n) + DECODED, vocab) for i, n in enumerate(lengths)}


def decode_trace(requests: dict, drop: int, prompts_per_step: int = 16) -> list:
    """Prompts whole, several in a step; then every live request decodes one token a step, and after
    half of the decode steps `drop` requests are ended."""
    rids = list(requests)
    steps = []
    for i in range(0, len(rids), prompts_per_step):
        entries = []
        for rid in rids[i:i + prompts_per_step]:
            n = len(requests[rid]) - DECODED
            entries.append({"id": rid, "tokens": requests[rid][:n], "want": [n - 1]})
        steps.append({"step": len(steps), "entries": entries, "end": []})
    live = list(rids)
    for d in range(DECODED):
        entries = [{"id": rid, "tokens": [requests[rid][len(requests[rid]) - DECODED + d]], "want": [0]} for rid in live]
        ended = []
        if d == DECODED // 2 - 1:
            ended = live[1::max(1, len(live) // drop)][:drop]
        if d == DECODED - 1:
            ended = list(live)
        steps.append({"step": len(steps), "entries": entries, "end": ended})
        live = [rid for rid in live if rid not in ended]
    return steps


@pytest.fixture(scope="module")
def models(model_folders):
    return {(name, dtype): load_model(model_folders[name], dtype, "cuda") for name in ("A", "M")
            for dtype in ("float32", "bfloat16")}


@pytest.fixture(scope="module")
def plain_models(model_folders):
    return {name: (gemma_plain.read_config(model_folders[name]), model_folders[name]) for name in ("A", "M")}


@pytest.mark.parametrize("graphs", [False, True])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("count", list(DROPS))
@pytest.mark.parametrize("name", ["A", "M"])
def test_decode_steps_of_many_requests(models, plain_models, name, count, dtype, graphs):
    longest = {"A": 100, "M": 200}[name]
    requests = many_requests(name, count, longest)
    cfg, folder = plain_models[name]
    plain = plain_of((name, count), cfg, folder, requests, dtype)
    trace = decode_trace(requests, DROPS[count])
    page_size = TINY[name]["page_size"]
    pages = pages_for_max_tokens(max_live_tokens(trace, round_to=page_size), page_size) + (1 if graphs else 0)
    runner = ModelRunner.create(models[(name, dtype)], num_pages=pages, page_size=page_size, max_requests=256,
                                poison_freed_pages=True)
    if graphs:
        runner.enable_graphs()
        assert runner.graph_buckets == (1, 2, 4, 8, 16, 32, 48, 64, 128, 256)
    got = replay_and_collect(TraceReplayer(runner), trace)
    runner.cache.check()
    assert len(got) == count + count * (DECODED // 2) + (count - DROPS[count]) * (DECODED // 2)
    if graphs:
        after = count - DROPS[count]
        used = sorted(runner.graphs)
        assert runner.graph_steps == DECODED
        assert used == sorted({next(b for b in runner.graph_buckets if b >= n) for n in (count, after)}), used
        assert used[-1] > count or count in runner.graph_buckets, "padding rows, unless the batch fills its bucket"
    worst = compare_replay(got, plain, dtype)
    print(f"{name} {dtype} {count} live, graphs {graphs}: worst error {worst:.3f} x bound")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_mixed_steps_of_24_live_requests(models, plain_models, dtype):
    """Portions of some requests beside decoded tokens of others, 24 live at a time, pages handed out again."""
    vocab = TINY["M"]["config"].vocab_size
    rng = np.random.default_rng(5)
    requests = {f"r{i}": random_ids(300 + i, int(n), vocab) for i, n in enumerate(rng.integers(20, 150, size=40))}
    cfg, folder = plain_models["M"]
    plain = plain_of("mixed24", cfg, folder, requests, dtype)
    trace = trace_mixed(requests, seed=3, live=24)
    assert max(len(s["entries"]) for s in trace) >= 20
    pages = pages_for_max_tokens(max_live_tokens(trace, round_to=16), 16)
    runner = ModelRunner.create(models[("M", dtype)], num_pages=pages, page_size=16, max_requests=24, poison_freed_pages=True)
    got = replay_and_collect(TraceReplayer(runner), trace)
    runner.cache.check()
    assert len(got) == sum(len(t) for t in requests.values())
    compare_replay(got, plain, dtype)


def test_forty_requests_generate_what_the_plain_implementation_generates(varied_folders):
    """Continuous batching of 40 requests through the entry point, float32: prompt portions beside
    decoding requests, then decode steps of all 32 admitted requests from captured graphs of the default
    buckets, steps started ahead, the last 8 requests admitted as others finish; every request's greedy
    tokens equal the plain implementation's full recomputation."""
    folder = varied_folders["MV"]
    cfg = gemma_plain.read_config(folder)
    w = gemma_plain.read_weights(folder, torch.float32)
    rng = np.random.default_rng(11)
    prompts = [random_ids(500 + i, int(n), cfg["vocab_size"]) for i, n in enumerate(rng.integers(3, 60, size=40))]
    news = [int(n) for n in rng.integers(24, 40, size=40)]
    llm = LLM(folder, dtype="float32", num_blocks=400, block_size=16, max_prefill_tokens_per_step=96, max_requests=32,
              hip_graphs=True, lookahead=True)
    outs = llm.generate(prompts, max_new_tokens=news)
    llm.runner.cache.check()
    assert llm.runner.graph_steps > 10 and max(llm.runner.graphs) == 32, sorted(llm.runner.graphs)
    for p, n, o in zip(prompts, news, outs):
        assert o.token_ids == gemma_plain.generate_greedy(cfg, w, p, n)
        assert o.finish_reason == "length"
    assert_varied([t for o in outs[:6] for t in o.token_ids], least=8)
