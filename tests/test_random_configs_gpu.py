"""Configurations drawn at random from what the configuration type allows: head sizes in steps of 16 up to
256, any number of heads and groups, widths, inner sizes and vocabularies that are no power of two (or no
multiple of 4), one to three layers, every eps and rotation base, tied or not, with or without biases, pages
of 4 to 64 tokens.  Each goes through the four ways of cutting its requests into steps, in float32 and in
bfloat16, and has to follow the plain implementation."""
import random

import pytest
import torch

from helpers import (compare_with_plain, max_live_tokens, random_ids, replay_and_collect, trace_mixed, trace_portions,
                     trace_tail, trace_whole)
from plain import gemma_plain
from wllm_amd.config import GemmaConfig
from wllm_amd.engine import ModelRunner
from wllm_amd.engine.replay import TraceReplayer, pages_for_max_tokens
from wllm_amd.parts import load_model, write_random_model_folder

pytestmark = pytest.mark.gpu

TOLERANCE = {"float32": dict(atol=2e-5, rtol=1e-4), "bfloat16": dict(atol=1e-2, rtol=1e-2)}
CASES = 12


def draw(case):
    rng = random.Random(7000 + case)
    kv = rng.choice([1, 1, 2, 3, 4])
    raw = dict(
        architectures=["GemmaForCausalLM"],
        vocab_size=rng.choice([61, 97, 128, 255, 300, 513, 1000, 1031, 2048, 4099]),
        hidden_size=rng.choice([24, 36, 50, 64, 70, 88, 100, 128, 136, 200, 256, 264]),
        intermediate_size=rng.choice([40, 66, 96, 130, 160, 200, 256, 344, 512]),
        num_hidden_layers=rng.choice([1, 2, 3]),
        num_attention_heads=kv * rng.choice([1, 1, 2, 3, 4, 5, 8]),
        num_key_value_heads=kv,
        head_dim=rng.choice([16, 32, 48, 64, 80, 96, 112, 128, 160, 192, 256]),
        rms_norm_eps=rng.choice([1e-6, 1e-5, 1e-4, 3e-3]),
        rope_theta=rng.choice([10000.0, 300.0, 1e6, 50.0]),
        max_position_embeddings=512,
        tie_word_embeddings=rng.random() < 0.7,
        attention_bias=rng.random() < 0.3,
    )
    page_size = rng.choice([16, 16, 16, 4, 8, 32, 12, 64])
    lengths = [rng.randint(33, 150) for _ in range(4)]
    return GemmaConfig.from_dict(raw), page_size, lengths


@pytest.mark.parametrize("case", range(CASES))
def test_a_random_configuration_follows_the_plain_implementation(tmp_path, case):
    config, page_size, lengths = draw(case)
    folder = write_random_model_folder(str(tmp_path / "model"), config, seed=100 + case, std=0.04, norm_std=0.1)
    requests = {f"r{i}": random_ids(17 * i + case, n, config.vocab_size) for i, n in enumerate(lengths)}
    plain_cfg = gemma_plain.read_config(folder)
    weights = gemma_plain.read_weights(folder, torch.float32)
    for dtype in ("float32", "bfloat16"):
        rounding = torch.bfloat16 if dtype == "bfloat16" else None
        plain = {rid: gemma_plain.forward_logits(plain_cfg, weights, toks, scale_rounding=rounding)
                 for rid, toks in requests.items()}
        model = load_model(folder, dtype, "cuda")
        for family in (trace_whole, trace_tail, trace_portions, trace_mixed):
            trace = family(requests)
            pages = pages_for_max_tokens(max_live_tokens(trace), page_size)
            runner = ModelRunner.create(model, num_pages=pages, page_size=page_size, max_requests=4,
                                        poison_freed_pages=True)
            got = replay_and_collect(TraceReplayer(runner), trace)
            runner.cache.check()
            assert len(got) == sum(lengths), (config, family.__name__, dtype)
            compare_with_plain(got, plain, **TOLERANCE[dtype])
