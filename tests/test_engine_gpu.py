"""The engine on the GPU against the plain implementation: every family of traces, in
float32 and in bfloat16, on all tiny configurations."""
import pytest
import torch

from helpers import (TINY, compare_with_plain, max_live_tokens, random_ids, replay_and_collect, trace_mixed,
                     trace_portions, trace_tail, trace_whole)
from plain import gemma_plain
from wllm_amd.engine import ModelRunner
from wllm_amd.engine.replay import TraceReplayer, pages_for_max_tokens
from wllm_amd.parts import load_model

pytestmark = pytest.mark.gpu

LENGTHS = {"A": [40, 57, 72, 33, 90, 64], "B": [45, 97, 64, 130, 51, 80], "C": [37, 66, 49, 100, 41], "M": [70, 130, 48, 97, 33]}
FAMILIES = {"whole": trace_whole, "tail": trace_tail, "portions": trace_portions, "mixed": trace_mixed}
# float32: the engine and the oracle differ by the order of float32 sums only.
# bfloat16: activations between kernels are rounded to 8 bits of mantissa; logits of
# these models are O(0.1..1), and errors of a few 1e-3 per rounding pile up over the layers.
TOLERANCE = {"float32": dict(atol=2e-5, rtol=1e-4), "bfloat16": dict(atol=1e-2, rtol=1e-2)}


def _requests(name):
    vocab = TINY[name]["config"].vocab_size
    return {f"r{i}": random_ids(100 * i + len(name), n, vocab) for i, n in enumerate(LENGTHS[name])}


@pytest.fixture(scope="module")
def plain_logits(model_folders):
    out = {}
    for name, folder in model_folders.items():
        cfg = gemma_plain.read_config(folder)
        w = gemma_plain.read_weights(folder, torch.float32)
        out[name] = {}
        for dtype, rounding in (("float32", None), ("bfloat16", torch.bfloat16)):
            out[name][dtype] = {rid: gemma_plain.forward_logits(cfg, w, toks, scale_rounding=rounding)
                                for rid, toks in _requests(name).items()}
    return out


@pytest.fixture(scope="module")
def models(model_folders):
    return {(name, dtype): load_model(folder, dtype, "cuda")
            for name, folder in model_folders.items() for dtype in ("float32", "bfloat16")}


@pytest.mark.parametrize("family", list(FAMILIES))
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", list(TINY))
def test_replay_matches_plain(models, plain_logits, name, dtype, family):
    requests = _requests(name)
    trace = FAMILIES[family](requests)
    page_size = TINY[name]["page_size"]
    pages = pages_for_max_tokens(max_live_tokens(trace), page_size)
    runner = ModelRunner.create(models[(name, dtype)], num_pages=pages, page_size=page_size, max_requests=4,
                                poison_freed_pages=True)
    got = replay_and_collect(TraceReplayer(runner), trace)
    runner.cache.check()
    assert len(got) == sum(len(t) for t in requests.values())
    worst = compare_with_plain(got, plain_logits[name][dtype], **TOLERANCE[dtype])
    print(f"{name} {dtype} {family}: worst error {worst:.3f} x tolerance")
