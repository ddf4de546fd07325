"""Sizes the tiny configurations of the other tests do not have: head sizes in steps of 16 from 16
to 144, widths and inner sizes that are no multiple of 32 (or of 4), an odd vocabulary, pages of
4 to 32 tokens.  Whatever kernel a size selects, or refuses so that a general one runs, the
logits follow the plain implementation: whole prompts, the last tokens one by one, portions of
changing size, and mixed portions with pages handed out again, in float32 and in bfloat16."""
import pytest
import torch

from helpers import (compare_replay, plain_for, max_live_tokens, random_ids, replay_and_collect, trace_mixed, trace_portions,
                     trace_tail, trace_whole)
from plain import gemma_plain
from wllm_amd.architectures import GemmaConfig
from wllm_amd.engine import ModelRunner
from wllm_amd.engine.replay import TraceReplayer, pages_for_max_tokens
from wllm_amd.parts import load_model, write_random_model_folder

pytestmark = pytest.mark.gpu


def cfg(vocab, hidden, inter, layers, heads, kv, head_dim, eps=1e-6, theta=10000.0, tie=True):
    return GemmaConfig(vocab_size=vocab, hidden_size=hidden, intermediate_size=inter, num_hidden_layers=layers,
                       num_attention_heads=heads, num_key_value_heads=kv, head_dim=head_dim, rms_norm_eps=eps,
                       rope_theta=theta, max_position_embeddings=256, tie_word_embeddings=tie)


ODD = {
    "head16": (cfg(97, 40, 72, 2, 3, 3, 16), 4),
    "head48": (cfg(1001, 104, 136, 2, 4, 2, 48, eps=1e-5, theta=300.0), 16),
    "head80": (cfg(513, 72, 200, 1, 2, 1, 80, tie=False), 32),
    "head112": (cfg(260, 96, 160, 2, 3, 1, 112), 8),
    "head128_pages12": (cfg(333, 64, 96, 2, 2, 2, 128), 12),
    "head144": (cfg(150, 50, 66, 1, 2, 2, 144, eps=1e-4), 16),
    "width_not_4": (cfg(211, 70, 90, 2, 5, 1, 32), 8),
}
LENGTHS = [37, 70, 33, 52]


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    root = tmp_path_factory.mktemp("odd")
    return {name: write_random_model_folder(str(root / name), c, seed=7 + i, std=0.04, norm_std=0.1)
            for i, (name, (c, _)) in enumerate(ODD.items())}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", list(ODD))
def test_odd_sizes_follow_the_plain_implementation(folders, name, dtype):
    config, page_size = ODD[name]
    requests = {f"r{i}": random_ids(31 * i + len(name), n, config.vocab_size) for i, n in enumerate(LENGTHS)}
    plain_cfg = gemma_plain.read_config(folders[name])
    plain = plain_for(plain_cfg, folders[name], requests, dtype)
    model = load_model(folders[name], dtype, "cuda")
    for family in (trace_whole, trace_tail, trace_portions, trace_mixed):
        trace = family(requests)
        pages = pages_for_max_tokens(max_live_tokens(trace), page_size)
        runner = ModelRunner.create(model, num_pages=pages, page_size=page_size, max_requests=4,
                                    poison_freed_pages=True)
        got = replay_and_collect(TraceReplayer(runner), trace)
        runner.cache.check()
        assert len(got) == sum(LENGTHS)
        compare_replay(got, plain, dtype)
