"""The engine at the layer sizes of the models it is measured on: the widths, head counts, head
size 256 and inner sizes of Gemma-2B (one key head for eight query heads) and of Gemma-7B
(sixteen heads with keys of their own, heads * head size != width), with fewer layers and a small
vocabulary so that the plain implementation stays fast.  The prompts are long enough for the
attention's work to be cut along the keys (several pieces of 128 keys in decode steps, a late
portion of a prompt split over workgroups).

float32 is held to the tolerance of the tiny configurations.  The bfloat16 bound here is a second line
behind the tiny configurations' element-wise one: it shows a wrong page, key or head, not a rounding
made at another point than the plain implementation makes it.  In bfloat16 an activation of these
widths is the sum of thousands of rounded terms, so single logits stray further than in the tiny
models; the measure is each position's error against the length of its logits vector, which a
missed key, a wrong page or a wrong head would raise to the order of one."""
import pytest
import torch

from helpers import max_live_tokens, random_ids, replay_and_collect, trace_mixed, trace_portions, trace_tail, trace_whole
from plain import gemma_plain
from wllm_amd.config import GemmaConfig
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
FLOAT32 = dict(atol=2e-5, rtol=1e-4)
# eight bits of mantissa: a rounding is 2^-9 of a value on average; a position's logits carry those of a
# handful of activations a layer
BFLOAT16_ROW_ERROR = 0.01


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
        w = gemma_plain.read_weights(folder, torch.float32)
        requests = _requests(name)
        out[name] = {rounding: {rid: gemma_plain.forward_logits(cfg, w, toks, scale_rounding=rounding)
                                for rid, toks in requests.items()} for rounding in (None, torch.bfloat16)}
    return out


def _requests(name):
    return {f"r{i}": random_ids(17 * i + len(name), n, SIZES[name].vocab_size) for i, n in enumerate(LENGTHS)}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", list(SIZES))
def test_layer_sizes_of_the_measured_models(folders, plain_logits, name, dtype):
    requests = _requests(name)
    plain = plain_logits[name][torch.bfloat16 if dtype == "bfloat16" else None]
    model = load_model(folders[name], dtype, "cuda")
    for family in (trace_whole, trace_tail, trace_portions, trace_mixed):
        trace = family(requests)
        pages = pages_for_max_tokens(max_live_tokens(trace), PAGE_SIZE)
        runner = ModelRunner.create(model, num_pages=pages, page_size=PAGE_SIZE, max_requests=4, poison_freed_pages=True)
        got = replay_and_collect(TraceReplayer(runner), trace)
        runner.cache.check()
        assert len(got) == sum(LENGTHS)
        worst = 0.0
        for (rid, pos), row in sorted(got.items()):
            ref = plain[rid][pos].double()
            row = row.double()
            assert torch.isfinite(row).all(), f"{family.__name__}: request {rid!r} position {pos}: logits are not finite"
            if dtype == "float32":
                err = ((row - ref).abs() / (FLOAT32["atol"] + FLOAT32["rtol"] * ref.abs())).max().item()
                assert err <= 1.0, f"{family.__name__}: request {rid!r} position {pos}: {err:.2f} x tolerance"
            else:
                err = ((row - ref).norm() / ref.norm()).item()
                assert err <= BFLOAT16_ROW_ERROR, f"{family.__name__}: request {rid!r} position {pos}: row error {err:.4f}"
            worst = max(worst, err)
        print(f"{name} {dtype} {family.__name__}: worst {worst:.4f}")
