"""The engine's bookkeeping (cache, batching, step function) on the CPU.

The kernels are replaced by their plain emulation, so what is compared with the
plain implementation here is everything around the kernels: block tables, slot
arithmetic, positions, segment arrays, page reuse, the order of layers.
"""
import pytest
import torch

from helpers import (TINY, compare_with_plain, max_live_tokens, random_ids, replay_and_collect, trace_mixed,
                     trace_portions, trace_tail, trace_whole)
from kernel_emulation import EmulatedKernels
from plain import gemma_plain
from wllm_amd.engine import ModelRunner
from wllm_amd.engine.replay import TraceReplayer, pages_for_max_tokens
from wllm_amd.kernels import ops
from wllm_amd.parts import load_model

LENGTHS = {"A": [40, 57, 72, 33, 90, 64], "B": [45, 97, 64, 130, 51, 80], "C": [37, 66, 49, 100, 41], "M": [70, 130, 48, 97, 33],
           "S": [50, 33, 120, 64, 77], "W": [60, 140, 33, 90, 75], "P": [44, 150, 61, 36, 100]}
FAMILIES = {"whole": trace_whole, "tail": trace_tail, "portions": trace_portions, "mixed": trace_mixed}


def _requests(name):
    vocab = TINY[name]["config"].vocab_size
    return {f"r{i}": random_ids(100 * i + len(name), n, vocab) for i, n in enumerate(LENGTHS[name])}


@pytest.fixture(scope="module")
def plain_logits(model_folders):
    out = {}
    for name, folder in model_folders.items():
        cfg = gemma_plain.read_config(folder)
        w = gemma_plain.read_weights(folder, torch.float32)
        out[name] = {rid: gemma_plain.forward_logits(cfg, w, toks) for rid, toks in _requests(name).items()}
    return out


@pytest.mark.parametrize("family", list(FAMILIES))
@pytest.mark.parametrize("name", list(TINY))
def test_replay_matches_plain_float32(model_folders, plain_logits, name, family):
    requests = _requests(name)
    trace = FAMILIES[family](requests)
    page_size = TINY[name]["page_size"]
    with ops.use_backend(EmulatedKernels()):
        model = load_model(model_folders[name], "float32", "cpu")
        pages = pages_for_max_tokens(max_live_tokens(trace), page_size)
        runner = ModelRunner.create(model, num_pages=pages, page_size=page_size, max_requests=4,
                                    poison_freed_pages=True)
        got = replay_and_collect(TraceReplayer(runner), trace)
        runner.cache.check()
        assert not runner.cache.requests, "every request was ended"
        assert all(g.pool.num_free == g.pool.num_pages for g in runner.cache.groups)
    assert len(got) == sum(len(t) for t in requests.values())
    compare_with_plain(got, plain_logits[name], atol=2e-5, rtol=1e-4)


def test_mixed_trace_reuses_pages(model_folders):
    requests = _requests("A")
    trace = trace_mixed(requests)
    pages = pages_for_max_tokens(max_live_tokens(trace), 4)
    total = sum(-(-len(t) // 4) for t in requests.values())
    assert pages < total, "the pool is smaller than what all requests need together"
    assert max(len(s["entries"]) for s in trace) == 4
    assert any(len(e["tokens"]) > 1 for s in trace for e in s["entries"] if len(s["entries"]) > 1)
    assert any(len(e["tokens"]) == 1 for s in trace for e in s["entries"] if len(s["entries"]) > 1)


def test_partial_sums_of_split_products_reach_the_consumers(model_folders, plain_logits):
    """With a product kernel that splits its sums, the stacks must be added by the next norm and by
    the rotation: same logits."""
    requests = _requests("C")
    trace = trace_mixed(requests)
    emu = EmulatedKernels(splits=3)
    with ops.use_backend(emu):
        model = load_model(model_folders["C"], "float32", "cpu")
        runner = ModelRunner.create(model, num_pages=pages_for_max_tokens(max_live_tokens(trace), 16), page_size=16,
                                    max_requests=4)
        got = replay_and_collect(TraceReplayer(runner), trace)
    compare_with_plain(got, plain_logits["C"], atol=2e-5, rtol=1e-4)


def test_the_garbage_collector_is_off_while_a_graph_is_captured(monkeypatch):
    """A collector run inside a capture that frees an object with device resources aborts the
    process; `capture` switches the collector off for the capture and back on after it, also when
    the captured body raises, and leaves it off if it was off."""
    import contextlib
    import gc

    from wllm_amd.engine import graphs

    seen = []

    class StandInGraph:
        pass

    @contextlib.contextmanager
    def stand_in_capture(graph):
        assert isinstance(graph, StandInGraph)
        seen.append(("enter", gc.isenabled()))
        yield
        seen.append(("exit", gc.isenabled()))

    monkeypatch.setattr(torch.cuda, "CUDAGraph", StandInGraph)
    monkeypatch.setattr(torch.cuda, "graph", stand_in_capture)
    assert gc.isenabled()

    graph, result = graphs.capture(lambda: (seen.append(("body", gc.isenabled())), 42)[1])
    assert isinstance(graph, StandInGraph) and result == 42
    assert seen == [("enter", False), ("body", False), ("exit", False)] and gc.isenabled()

    def failing():
        assert not gc.isenabled()
        raise KeyError("inside the capture")

    with pytest.raises(KeyError):
        graphs.capture(failing)
    assert gc.isenabled(), "switched back on after a body that raised"

    gc.disable()
    try:
        graphs.capture(lambda: None)
        assert not gc.isenabled(), "a collector that was off stays off"
    finally:
        gc.enable()
