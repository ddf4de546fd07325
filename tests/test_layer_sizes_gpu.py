"""The engine at the layer sizes of the models it is measured on: the widths, head counts, head
size 256 and inner sizes of Gemma-2B (one key head for eight query heads) and of Gemma-7B
(sixteen heads with keys of their own, heads * head size != width), with fewer layers and a small
vocabulary so that the plain implementation stays fast.  The prompts are long enough for the
attention's work to be cut along the keys (several pieces of 128 keys in decode steps, a late
portion of a prompt split over workgroups).

float32 is held to the tolerance of the tiny configurations, bfloat16 to the bound that the plain
implementation's own rounded run sets for each row (helpers.compare_with_bfloat16_bound), as
everywhere."""
import pytest
import torch

from helpers import compare_replay, max_live_tokens, plain_for, random_ids, replay_and_collect, trace_mixed, trace_portions, trace_tail, trace_whole
from plain import gemma_plain
from wllm_amd.architectures import GemmaConfig
from wllm_amd.engine import ModelRunner
from wllm_amd.engine.replay import TraceReplayer, pages_for_max_tokens
from wllm_amd.parts import load_model, write_random_model_folder

pytestmark = pytest.mark.gpu

SIZES = {
    "gemma_2b_layers": GemmaConfig(vocab_size=2000, hidden_size=2048, intermediate_size=16384, num_hidden_layers=2,
                                   num_attention_heads=8, num_key_value_heads=1, head_dim=256, rms_norm_eps=1e-6,
                                   rope_theta=10000.0, max_position_embeddings=8192, tie_word_embeddings=True),
    "gemma_7b_layers": GemmaConfig(vocab_size=1500, hidden_size=3072, intermediate_size=24576, num_hidden_layers=1,
                                   num_attention_heads=16, num_key_value_heads=16, head_dim=256, rms_norm_eps=1e-6,
                                   rope_theta=10000.0, max_position_embeddings=8192, tie_word_embeddings=True),
}
LENGTHS = [300, 70, 650, 161]
PAGE_SIZE = 16


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    root = tmp_path_factory.mktemp("layer_sizes")
    return {name: write_random_model_folder(str(root / name), c, seed=21 + i, std=0.02, norm_std=0.1)
            for i, (name, c) in enumerate(SIZES.items())}


@pytest.fixture(scope="module")
def plain_logits(folders):
    out = {}
    for name, folder in folders.items():
        cfg = gemma_plain.read_config(folder)
        out[name] = {dtype: plain_for(cfg, folder, _requests(name), dtype) for dtype in ("float32", "bfloat16")}
    return out


def _requests(name):
    return {f"r{i}": random_ids(17 * i + len(name), n, SIZES[name].vocab_size) for i, n in enumerate(LENGTHS)}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", list(SIZES))
def test_layer_sizes_of_the_measured_models(folders, plain_logits, name, dtype):
    requests = _requests(name)
    plain = plain_logits[name][dtype]
    model = load_model(folders[name], dtype, "cuda")
    for family in (trace_whole, trace_tail, trace_portions, trace_mixed):
        trace = family(requests)
        pages = pages_for_max_tokens(max_live_tokens(trace), PAGE_SIZE)
        runner = ModelRunner.create(model, num_pages=pages, page_size=PAGE_SIZE, max_requests=4, poison_freed_pages=True)
        got = replay_and_collect(TraceReplayer(runner), trace)
        runner.cache.check()
        assert len(got) == sum(LENGTHS)
        worst = compare_replay(got, plain, dtype)
        print(f"{name} {dtype} {family.__name__}: worst {worst:.3f} x bound")
