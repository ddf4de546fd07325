"""Shared by the tests: the tiny configurations, trace building and comparison."""
from __future__ import annotations

import numpy as np
import torch

from wllm_amd.architectures import GemmaConfig
from wllm_amd.parts import write_random_model_folder

# Two tiny configurations that differ in every size and option, a third with
# biases and an untied head, a fourth whose head size and page size are the
# ones the matrix-core attention kernels take, a fifth without grouped heads, a sixth with more
# query heads a key/value head than a tile of rows holds, and a seventh with pages of 6 tokens.
TINY = {
    "A": dict(config=GemmaConfig(vocab_size=512, hidden_size=64, intermediate_size=256, num_hidden_layers=2,
                                 num_attention_heads=4, num_key_value_heads=1, head_dim=32, rms_norm_eps=1e-6,
                                 rope_theta=10000.0, max_position_embeddings=128, tie_word_embeddings=True),
              seed=11, std=0.02, norm_std=0.1, page_size=4),
    "B": dict(config=GemmaConfig(vocab_size=777, hidden_size=96, intermediate_size=384, num_hidden_layers=3,
                                 num_attention_heads=6, num_key_value_heads=6, head_dim=24, rms_norm_eps=1e-5,
                                 rope_theta=500.0, max_position_embeddings=256, tie_word_embeddings=True),
              seed=22, std=0.03, norm_std=0.05, page_size=8),
    "C": dict(config=GemmaConfig(vocab_size=301, hidden_size=80, intermediate_size=112, num_hidden_layers=2,
                                 num_attention_heads=6, num_key_value_heads=2, head_dim=20, rms_norm_eps=1e-4,
                                 rope_theta=77.0, max_position_embeddings=192, tie_word_embeddings=False,
                                 attention_bias=True),
              seed=33, std=0.05, norm_std=0.2, page_size=16),
    "M": dict(config=GemmaConfig(vocab_size=1000, hidden_size=128, intermediate_size=320, num_hidden_layers=2,
                                 num_attention_heads=8, num_key_value_heads=2, head_dim=64, rms_norm_eps=1e-6,
                                 rope_theta=10000.0, max_position_embeddings=512, tie_word_embeddings=True),
              seed=44, std=0.04, norm_std=0.1, page_size=16),
    # every query head with its own key/value head, a head size the matrix-core kernels take, and
    # heads * head_dim (160) unlike the width (96): the arrangement of the 7B sizes
    "S": dict(config=GemmaConfig(vocab_size=1200, hidden_size=96, intermediate_size=192, num_hidden_layers=2,
                                 num_attention_heads=5, num_key_value_heads=5, head_dim=32, rms_norm_eps=1e-6,
                                 rope_theta=10000.0, max_position_embeddings=256, tie_word_embeddings=True),
              seed=55, std=0.04, norm_std=0.1, page_size=8),
    # 32 query heads on one key/value head: a decoded token's rows fill two tiles of 16
    "W": dict(config=GemmaConfig(vocab_size=640, hidden_size=64, intermediate_size=160, num_hidden_layers=2,
                                 num_attention_heads=32, num_key_value_heads=1, head_dim=32, rms_norm_eps=1e-6,
                                 rope_theta=10000.0, max_position_embeddings=256, tie_word_embeddings=True),
              seed=66, std=0.04, norm_std=0.1, page_size=8),
    # pages of 6 tokens (no multiple of 4), 20 query heads on two key/value heads
    "P": dict(config=GemmaConfig(vocab_size=450, hidden_size=72, intermediate_size=200, num_hidden_layers=2,
                                 num_attention_heads=20, num_key_value_heads=2, head_dim=32, rms_norm_eps=1e-5,
                                 rope_theta=3000.0, max_position_embeddings=256, tie_word_embeddings=True),
              seed=77, std=0.04, norm_std=0.1, page_size=6),
}


# Greedy decoding of the configurations above repeats the last prompt token for ever: with weights
# this small the tied head's logit of a token for itself beats everything the context adds.  Tests
# that compare generated tokens use these instead: the same sizes with weights large enough that
# the context decides, so that a wrong key, page or position changes the tokens.
VARIED = {"AV": dict(TINY["A"], std=0.3), "MV": dict(TINY["M"], std=0.3), "WV": dict(TINY["W"], std=0.3)}


def assert_varied(tokens: list, least: int = 4) -> None:
    """The generated tokens are not one token repeated (a test of token equality would be empty)."""
    assert len(set(tokens)) >= min(least, len(tokens)), f"the generated tokens hardly vary: {tokens}"


def write_tiny(name: str, folder: str) -> str:
    t = TINY[name] if name in TINY else VARIED[name]
    return write_random_model_folder(folder, t["config"], t["seed"], std=t["std"], norm_std=t["norm_std"])


def degenerate_folder(src: str, out: str, kind: str) -> str:
    """A copy of a model folder with some weights set to zero, so that the logits reduce to a formula
    a test writes out by hand (through the framework's safetensors writer, not the model):
    "no_contributions": every o_proj and down_proj zero and the layers' norm weights zero, so each
        layer adds nothing: logits = final_norm(E[ids] * sqrt(H)) @ head^T;
    "one_feed_forward": as above, but layer 0's down_proj and post-attention norm weight are kept:
        logits = final_norm(x + mlp(norm(x))) @ head^T with x = E[ids] * sqrt(H);
    "one_attention": every down_proj zero, every o_proj but layer 0's zero, the norm weights of the other
        layers zero (layer 0 keeps both of its own, so that taking the wrong one shows):
        logits = final_norm(x + attention(input_norm(x))) @ head^T;
    "bias_only_queries_and_keys": q_proj and k_proj weights zero (the folder must have biases): queries
        and keys are the rotated biases."""
    import os
    from wllm_amd.weights import Checkpoint, write_safetensors
    ck = Checkpoint(src)
    tensors = {n: ck.tensor(n).clone() for n in ck.names()}
    ck.close()
    for n, t in tensors.items():
        if kind in ("no_contributions", "one_feed_forward"):
            keep = kind == "one_feed_forward" and ".layers.0." in n
            if n.endswith("o_proj.weight") or (n.endswith("down_proj.weight") and not keep):
                t.zero_()
            if n.endswith("input_layernorm.weight") or (n.endswith("post_attention_layernorm.weight") and not keep):
                t.zero_()
        elif kind == "one_attention":
            first = ".layers.0." in n
            if n.endswith("down_proj.weight") or (n.endswith("o_proj.weight") and not first):
                t.zero_()
            if n.endswith(("input_layernorm.weight", "post_attention_layernorm.weight")) and not first:
                t.zero_()
        elif kind == "bias_only_queries_and_keys":
            if n.endswith(("q_proj.weight", "k_proj.weight")):
                t.zero_()
        else:
            raise ValueError(kind)
    os.makedirs(out, exist_ok=True)
    write_safetensors(os.path.join(out, "model.safetensors"), tensors)
    with open(os.path.join(src, "config.json")) as f, open(os.path.join(out, "config.json"), "w") as g:
        g.write(f.read())
    return out


def random_ids(seed: int, length: int, vocab: int) -> list:
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (length,), generator=g).tolist()


# ---- traces ------------------------------------------------------------------

def trace_whole(requests: dict) -> list:
    """Each request alone, all its tokens in one step, every logit wanted."""
    return [{"step": i, "entries": [{"id": rid, "tokens": toks, "want": list(range(len(toks)))}], "end": [rid]}
            for i, (rid, toks) in enumerate(requests.items())]


def trace_tail(requests: dict, tail: int = 32) -> list:
    """All but the last `tail` tokens in one step, then the rest one by one."""
    steps = []
    for rid, toks in requests.items():
        head = max(1, len(toks) - tail)
        steps.append({"step": len(steps), "entries": [{"id": rid, "tokens": toks[:head], "want": list(range(head))}], "end": []})
        for p in range(head, len(toks)):
            steps.append({"step": len(steps), "entries": [{"id": rid, "tokens": [toks[p]], "want": [0]}],
                          "end": [rid] if p == len(toks) - 1 else []})
        if head == len(toks):
            steps[-1]["end"] = [rid]
    return steps


def trace_portions(requests: dict, sizes=(16, 5, 2, 11, 2, 7, 3, 2, 9)) -> list:
    """Consecutive portions of changing size, down to two tokens."""
    steps = []
    for rid, toks in requests.items():
        p, k = 0, 0
        while p < len(toks):
            size = min(sizes[k % len(sizes)], len(toks) - p)
            k += 1
            last = p + size == len(toks)
            steps.append({"step": len(steps), "entries": [{"id": rid, "tokens": toks[p:p + size], "want": list(range(size))}],
                          "end": [rid] if last else []})
            p += size
    return steps


def trace_mixed(requests: dict, seed: int = 0, live: int = 4, prompt_fraction: float = 0.6,
                portion_sizes=(2, 3, 5, 8, 13)) -> list:
    """Up to `live` requests at a time: portions of some beside single tokens of
    others; a request is sometimes left out of a step; finished requests are ended
    and new ones start, so their pages are handed out again."""
    rng = np.random.default_rng(seed)
    waiting = list(requests.items())
    running = {}      # rid -> (tokens, fed, prompt_len)
    steps = []
    while waiting or running:
        while waiting and len(running) < live:
            rid, toks = waiting.pop(0)
            running[rid] = [toks, 0, max(2, int(len(toks) * prompt_fraction))]
        entries, ended = [], []
        for rid in list(running):
            toks, fed, plen = running[rid]
            if len(running) > 1 and rng.random() < 0.2:
                continue  # left out of this step
            if fed < plen:
                size = int(min(rng.choice(portion_sizes), plen - fed))
                if plen - fed - size == 1:
                    size += 1   # never leave a portion of one token: that is a decode
            else:
                size = 1
            entries.append({"id": rid, "tokens": toks[fed:fed + size], "want": list(range(size))})
            running[rid][1] = fed + size
            if fed + size == len(toks):
                ended.append(rid)
                del running[rid]
        if entries:
            steps.append({"step": len(steps), "entries": entries, "end": ended})
    return steps


def max_live_tokens(trace: list, round_to: int = 64) -> int:
    """The most tokens live requests hold at any time, each rounded up to `round_to`."""
    held, worst = {}, 0
    for step in trace:
        for e in step["entries"]:
            held[e["id"]] = held.get(e["id"], 0) + len(e["tokens"])
        worst = max(worst, sum(-(-v // round_to) * round_to for v in held.values()))
        for rid in step["end"]:
            held.pop(rid, None)
    return worst


def replay_and_collect(replayer, trace: list) -> dict:
    """Runs a trace; returns {(request, position): logits row (float32 CPU)}."""
    fed, out = {}, {}
    for step in trace:
        logits = replayer.run_step(step)
        row = 0
        for e in step["entries"]:
            base = fed.get(e["id"], 0)
            for w in e["want"]:
                out[(e["id"], base + w)] = logits[row].float().cpu()
                row += 1
            fed[e["id"]] = base + len(e["tokens"])
        for rid in step["end"]:
            fed.pop(rid, None)
    return out


def compare_with_plain(collected: dict, plain: dict, atol: float, rtol: float) -> float:
    """Every collected row against the plain implementation's row of the same request
    and position; returns the worst error in units of the tolerance.  The first wrong
    place is named."""
    worst = 0.0
    for (rid, pos) in sorted(collected, key=lambda k: (str(k[0]), k[1])):
        got, ref = collected[(rid, pos)].double(), plain[rid][pos].double()
        assert torch.isfinite(got).all(), f"request {rid!r} position {pos}: logits are not finite"
        err = ((got - ref).abs() / (atol + rtol * ref.abs())).max().item()
        assert err <= 1.0, (f"request {rid!r} position {pos}: worst error {err:.2f} x tolerance "
                            f"(max abs diff {(got - ref).abs().max().item():.3e}, ref max {ref.abs().max().item():.3e})")
        worst = max(worst, err)
    return worst


# ---- the bound of the bfloat16 comparisons -------------------------------------------------------
#
# Not a number chosen until the cases pass: the measure is how far the reference's own bfloat16
# model is from the exact result.  The plain implementation runs in float64 as it is (`exact`) and
# again rounding to bfloat16 wherever the reference's bfloat16 model holds a tensor (see
# tests/plain/gemma_plain.py).  One rounded run is one draw of the rounding's noise; a second draw comes
# from the same run with all positions moved by a constant (the exact logits do not change, which
# tests/test_plain_implementation.py holds; every rounding falls differently).  `REALISATIONS` such
# runs give, per row, the farthest that the reference's rounding strays, in the root mean square
# over the row and in its largest element; the engine's row may be RMS_FACTOR and MAX_FACTOR times
# as far from `exact`.
#
# The factors are what a further draw of the reference's own rounding needs: over ten models (eight
# drawn at random with weights of std 0.05 and norm weights of 0.2, and a model whose attention is
# sharpened until single keys decide, where the noise of a row is a few large roundings and no sum of
# many small ones) a fifth and sixth realisation came as far as 1.85 times the farthest of four in
# the root mean square and 2.20 times in the largest element.  The engine rounds at fewer places than
# the reference (its residual stream and its logits are float32): its worst rows were 2.03 and 2.01
# times in the sharp model (whole prompts, whose queries and keys are rounded once by the library's
# product and once after the rotation) and 1.14 and 1.30 times in the others.  A lost key, a wrong page
# or a wrong head is no rounding and lands many bounds away where a test is made to show it
# (tests/test_plain_implementation.py holds that with this bound).
BF16_REALISATIONS = (0, 37, 64, 101)      # shifts of all positions
BF16_RMS_FACTOR = 2.5
BF16_MAX_FACTOR = 3.0
BF16_HALF_ULP = 2.0 ** -9       # rows that every realisation hits by luck still allow one rounding of the logits


def plain_exact_and_rounded(cfg: dict, weights64: dict, tokens, realisations=BF16_REALISATIONS):
    """(exact, [rounded, ...]) float64 logits of one request: see above.  `weights64`: the folder's
    tensors in float64."""
    from plain import gemma_plain
    exact = gemma_plain.forward_logits(cfg, weights64, tokens)
    rounded = [gemma_plain.forward_logits(cfg, weights64, tokens, positions=torch.arange(len(tokens)) + shift,
                                          round_to=torch.bfloat16) for shift in realisations]
    return exact, rounded


def bfloat16_row_errors(got: torch.Tensor, exact: torch.Tensor, rounded: list):
    """A row's error in units of its bound: (root mean square, largest element).  `rounded`: the row
    in each realisation of the reference's rounding."""
    got, exact = got.double(), exact.double()
    floor = exact.pow(2).mean().sqrt().item() * BF16_HALF_ULP
    far_rms = max((r.double() - exact).pow(2).mean().sqrt().item() for r in rounded)
    far_top = max((r.double() - exact).abs().max().item() for r in rounded)
    rms = (got - exact).pow(2).mean().sqrt().item() / (BF16_RMS_FACTOR * max(far_rms, floor))
    top = (got - exact).abs().max().item() / (BF16_MAX_FACTOR * max(far_top, floor))
    return rms, top


def compare_with_bfloat16_bound(collected: dict, plain: dict) -> float:
    """Every collected row against (exact, realisations) of `plain[request]`; returns the worst error in
    units of the bound and names the first row beyond it."""
    worst = 0.0
    for (rid, pos) in sorted(collected, key=lambda k: (str(k[0]), k[1])):
        got = collected[(rid, pos)]
        exact, rounded = plain[rid]
        assert torch.isfinite(got).all(), f"request {rid!r} position {pos}: logits are not finite"
        rms, top = bfloat16_row_errors(got, exact[pos], [r[pos] for r in rounded])
        assert rms <= 1.0 and top <= 1.0, (
            f"request {rid!r} position {pos}: {rms:.2f} x the bound in the root mean square, {top:.2f} x in the largest "
            f"element (the rounded plain rows are up to {max((r[pos] - exact[pos]).abs().max().item() for r in rounded):.3e} "
            f"from the exact one, this row {(got.double() - exact[pos]).abs().max().item():.3e})")
        worst = max(worst, rms, top)
    return worst


def plain_for(cfg: dict, folder: str, requests: dict, dtype: str) -> dict:
    """What a replay in `dtype` is compared with: float32 logits, or (exact, rounded) pairs for bfloat16."""
    from plain import gemma_plain
    if dtype == "float32":
        w = gemma_plain.read_weights(folder, torch.float32)
        return {rid: gemma_plain.forward_logits(cfg, w, t) for rid, t in requests.items()}
    w = gemma_plain.read_weights(folder, torch.float64)
    return {rid: plain_exact_and_rounded(cfg, w, t) for rid, t in requests.items()}


FLOAT32_TOLERANCE = dict(atol=2e-5, rtol=1e-4)       # the engine and the plain implementation differ by the order of float32 sums


def compare_replay(collected: dict, plain: dict, dtype: str) -> float:
    if dtype == "float32":
        return compare_with_plain(collected, plain, **FLOAT32_TOLERANCE)
    return compare_with_bfloat16_bound(collected, plain)
