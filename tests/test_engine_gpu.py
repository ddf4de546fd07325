"""The engine on the GPU against the plain implementation: every family of traces, in
float32 and in bfloat16, on all tiny configurations."""
import pytest
import torch

from helpers import (TINY, compare_replay, compare_with_plain, max_live_tokens, plain_for, random_ids, replay_and_collect, trace_mixed,
                     trace_portions, trace_tail, trace_whole)
from plain import gemma_plain
from wllm_amd.engine import ModelRunner
from wllm_amd.engine.replay import TraceReplayer, pages_for_max_tokens
from wllm_amd.parts import load_model

pytestmark = pytest.mark.gpu

LENGTHS = {"A": [40, 57, 72, 33, 90, 64], "B": [45, 97, 64, 130, 51, 80], "C": [37, 66, 49, 100, 41], "M": [70, 130, 48, 97, 33],
           "S": [50, 33, 120, 64, 77], "W": [60, 140, 33, 90, 75], "P": [44, 150, 61, 36, 100]}
FAMILIES = {"whole": trace_whole, "tail": trace_tail, "portions": trace_portions, "mixed": trace_mixed}
# float32: the engine and the plain implementation differ by the order of float32 sums only.
# bfloat16: a row may be as far from the exact logits as a small multiple of what the plain
# implementation is when it rounds like the reference's bfloat16 model (helpers.compare_with_bfloat16_bound).


def _requests(name):
    vocab = TINY[name]["config"].vocab_size
    return {f"r{i}": random_ids(100 * i + len(name), n, vocab) for i, n in enumerate(LENGTHS[name])}


@pytest.fixture(scope="module")
def plain_logits(model_folders):
    out = {}
    for name, folder in model_folders.items():
        cfg = gemma_plain.read_config(folder)
        out[name] = {dtype: plain_for(cfg, folder, _requests(name), dtype) for dtype in ("float32", "bfloat16")}
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
    worst = compare_replay(got, plain_logits[name][dtype], dtype)
    print(f"{name} {dtype} {family}: worst error {worst:.3f} x bound")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_sharp_attention_over_hundreds_of_keys(model_folders, tmp_path_factory, dtype):
    """Random weights of the usual size give nearly flat attention, which hides a lost or doubled key.
    Here the query and key projections are scaled up until each query puts almost all its weight on
    one or two keys, often far back, over sequences of several hundred tokens cut at page and chunk
    edges; a wrong key then changes the logits by far more than the tolerance."""
    import os
    from wllm_amd.weights import Checkpoint, write_safetensors
    src = model_folders["M"]
    folder = str(tmp_path_factory.mktemp("sharp"))
    ck = Checkpoint(src)
    tensors = {n: ck.tensor(n) for n in ck.names()}
    ck.close()
    for n in tensors:
        if n.endswith(("q_proj.weight", "k_proj.weight")):
            tensors[n] = (tensors[n].float() * 6.0).to(torch.bfloat16)
    write_safetensors(os.path.join(folder, "model.safetensors"), tensors)
    with open(os.path.join(src, "config.json")) as f, open(os.path.join(folder, "config.json"), "w") as g:
        g.write(f.read())
    cfg = gemma_plain.read_config(folder)
    w = gemma_plain.read_weights(folder, torch.float32)
    requests = {"a": random_ids(71, 400, 1000), "b": random_ids(72, 333, 1000), "c": random_ids(73, 257, 1000)}
    plain = plain_for(cfg, folder, requests, dtype)
    # the attention really is sharp: the largest probability of a late query is far from 1/400
    h = gemma_plain.rms_norm_one_plus_w(gemma_plain.embed(torch.tensor(requests["a"]), w["model.embed_tokens.weight"], 128),
                                        w["model.layers.0.input_layernorm.weight"], 1e-6)
    q = (h @ w["model.layers.0.self_attn.q_proj.weight"].T).view(400, 8, 64)
    k = (h @ w["model.layers.0.self_attn.k_proj.weight"].T).view(400, 2, 64)
    probs = torch.softmax((q[-1, 0] @ k[:, 0].T) / 8.0, -1)
    assert probs.max() > 0.2
    model = load_model(folder, dtype, "cuda")
    # In bfloat16 the rounding of queries and keys (8 bits) is multiplied by scores of magnitude 20 before
    # the exponential; the rounded plain implementation has that too, so the bound follows it.  float32
    # sums of scores this large differ a little more than the usual ones by their order.
    for family in (trace_whole, trace_portions, trace_mixed, lambda r: trace_tail(r, tail=40)):
        trace = family(requests)
        pages = pages_for_max_tokens(max_live_tokens(trace), 16)
        runner = ModelRunner.create(model, num_pages=pages, page_size=16, max_requests=4, poison_freed_pages=True)
        got = replay_and_collect(TraceReplayer(runner), trace)
        if dtype == "float32":
            compare_with_plain(got, plain, atol=5e-5, rtol=2e-4)
        else:
            compare_replay(got, plain, dtype)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name,kind", [("A", "no_contributions"), ("C", "no_contributions"), ("A", "one_feed_forward"),
                                       ("B", "one_feed_forward"), ("C", "bias_only_queries_and_keys"),
                                       ("A", "one_attention"), ("B", "one_attention"), ("C", "one_attention")])
def test_models_whose_logits_a_formula_gives(model_folders, tmp_path, name, kind, dtype):
    """The folders that pin the plain implementation's wiring (layers that contribute nothing; one
    feed-forward alone; one attention alone; queries and keys that are rotated biases), through the engine: whole prompts,
    the last tokens one by one, and portions."""
    from helpers import degenerate_folder
    folder = degenerate_folder(model_folders[name], str(tmp_path / kind), kind)
    cfg = gemma_plain.read_config(folder)
    requests = {f"r{i}": random_ids(7 * i + 1, n, cfg["vocab_size"]) for i, n in enumerate([21, 40])}
    plain = plain_for(cfg, folder, requests, dtype)
    model = load_model(folder, dtype, "cuda")
    page_size = TINY[name]["page_size"]
    for family in (trace_whole, lambda r: trace_tail(r, tail=8), trace_portions):
        trace = family(requests)
        runner = ModelRunner.create(model, num_pages=pages_for_max_tokens(max_live_tokens(trace), page_size),
                                    page_size=page_size, max_requests=4, poison_freed_pages=True)
        compare_replay(replay_and_collect(TraceReplayer(runner), trace), plain, dtype)
