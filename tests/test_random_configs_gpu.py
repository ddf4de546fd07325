"""Configurations drawn at random from what the configuration type allows: head sizes in steps of 16 up to
256, any number of heads and groups, widths, inner sizes and vocabularies that are no power of two (or no
multiple of 4), one to three layers, every eps and rotation base, tied or not, with or without biases, pages
of 4 to 64 tokens, weights of std 0.05 and norm weights of std 0.2.  Each goes through the four ways of
cutting its requests into steps, in float32 and in bfloat16, and has to follow the plain implementation:
float32 within the order of its sums, bfloat16 within the bound that the plain implementation's own
rounded run sets (helpers.compare_with_bfloat16_bound).  28 of the draws are ones on which a hand-set
bfloat16 tolerance of 1e-2 once failed by up to a half; the others are drawn afresh."""
import random

import pytest
import torch

from helpers import (compare_replay, max_live_tokens, plain_for, random_ids, replay_and_collect, trace_mixed, trace_portions,
                     trace_tail, trace_whole)
from plain import gemma_plain
from wllm_amd.architectures import GemmaConfig
from wllm_amd.engine import ModelRunner
from wllm_amd.engine.replay import TraceReplayer, pages_for_max_tokens
from wllm_amd.parts import load_model, write_random_model_folder

pytestmark = pytest.mark.gpu

# draws that a hand-set tolerance once failed on, as (generator, case) pairs, and twenty more
ONCE_FAILED = [(1, 4), (1, 13), (1, 21), (1, 28), (1, 29), (2, 6), (2, 7), (2, 20), (2, 23), (2, 24), (2, 29), (2, 40),
               (2, 43), (2, 49), (2, 56), (2, 57), (2, 58), (3, 4), (3, 9), (3, 10), (3, 11), (3, 23), (3, 33), (3, 42),
               (3, 43), (3, 51), (3, 55), (3, 57)]
CASES = ONCE_FAILED + [(7, c) for c in range(20)]


def draw(generator, case):
    rng = random.Random(generator * 1000 + case)
    head_dim = rng.choice([16, 32, 48, 64, 80, 96, 112, 128, 160, 192, 256])
    kv = rng.choice([1, 1, 2, 3, 4])
    group = rng.choice([1, 1, 2, 3, 4, 5, 8])
    raw = dict(
        architectures=["GemmaForCausalLM"],
        head_dim=head_dim,
        num_key_value_heads=kv,
        num_attention_heads=kv * group,
        hidden_size=rng.choice([24, 36, 50, 64, 70, 88, 100, 128, 136, 200, 256, 264]),
        intermediate_size=rng.choice([40, 66, 96, 130, 160, 200, 256, 344, 512]),
        vocab_size=rng.choice([61, 97, 128, 255, 300, 513, 1000, 1031, 2048, 4099]),
        num_hidden_layers=rng.choice([1, 2, 3]),
        rms_norm_eps=rng.choice([1e-6, 1e-5, 1e-4, 3e-3]),
        rope_theta=rng.choice([10000.0, 300.0, 1e6, 50.0]),
        max_position_embeddings=512,
        tie_word_embeddings=rng.random() < 0.7,
        attention_bias=rng.random() < 0.3,
    )
    page_size = rng.choice([16, 16, 16, 4, 8, 32, 12, 64])
    lengths = [rng.randint(33, 180) for _ in range(4)]
    return GemmaConfig.from_dict(raw), page_size, lengths


@pytest.mark.parametrize("generator,case", CASES)
def test_a_random_configuration_follows_the_plain_implementation(tmp_path, generator, case):
    config, page_size, lengths = draw(generator, case)
    folder = write_random_model_folder(str(tmp_path / "model"), config, seed=case + 11, std=0.05, norm_std=0.2)
    requests = {f"r{i}": random_ids(17 * i + case, n, config.vocab_size) for i, n in enumerate(lengths)}
    plain_cfg = gemma_plain.read_config(folder)
    for dtype in ("float32", "bfloat16"):
        plain = plain_for(plain_cfg, folder, requests, dtype)
        model = load_model(folder, dtype, "cuda")
        for family in (trace_whole, trace_tail, trace_portions, trace_mixed):
            trace = family(requests)
            pages = pages_for_max_tokens(max_live_tokens(trace), page_size)
            runner = ModelRunner.create(model, num_pages=pages, page_size=page_size, max_requests=4,
                                        poison_freed_pages=True)
            got = replay_and_collect(TraceReplayer(runner), trace)
            runner.cache.check()
            assert len(got) == sum(lengths), (config, family.__name__, dtype)
            compare_replay(got, plain, dtype)
