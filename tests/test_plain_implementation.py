"""Pins of the plain implementation: what fixes each formula beside the reference's text.

Special cases that reduce to a library routine, invariants, and the vectors the
reference's own tests hold.  Each is chosen so that a plausible mistake fails it: a wrong
sign or pairing in the rotation, a norm that multiplies by w instead of 1 + w, a scale by
hidden/heads instead of head_dim, a head mapped to the wrong key/value head.
"""
import math

import pytest
import torch

from plain import gemma_plain as P
from plain import sampling_plain as S

torch.manual_seed(0)


# ---- norm ---------------------------------------------------------------------------
def test_norm_with_zero_weight_is_plain_normalisation():
    x = torch.randn(5, 48, dtype=torch.float64)
    y = P.rms_norm_one_plus_w(x, torch.zeros(48, dtype=torch.float64), 1e-6)
    assert torch.allclose(y, x / torch.sqrt(x.pow(2).mean(-1, keepdim=True) + 1e-6))
    # unit-RMS rows, eps 0: identity
    x = x / x.pow(2).mean(-1, keepdim=True).sqrt()
    assert torch.allclose(P.rms_norm_one_plus_w(x, torch.zeros(48, dtype=torch.float64), 0.0), x)


def test_eps_is_added_under_the_root():
    """Rows of mean square 1 and eps 0.5: x / sqrt(1.5) (src/wllm/models/gemma.py:47-48, rsqrt(variance + eps)).
    With eps added to the root instead the result is x / 1.5, a fifth smaller; with eps inside a mean over
    squares that forgot to divide, or left out, it is x."""
    x = torch.randn(4, 40, dtype=torch.float64)
    x = x / x.pow(2).mean(-1, keepdim=True).sqrt()
    y = P.rms_norm_one_plus_w(x, torch.zeros(40, dtype=torch.float64), 0.5)
    assert torch.allclose(y, x / math.sqrt(1.5), rtol=1e-12, atol=0)
    assert not torch.allclose(y, x / 1.5, rtol=0.1, atol=0)
    assert not torch.allclose(y, x, rtol=0.1, atol=0)


def test_norm_weight_is_an_offset_from_one():
    x = torch.randn(3, 16, dtype=torch.float64)
    w = torch.randn(16, dtype=torch.float64)
    base = P.rms_norm_one_plus_w(x, torch.zeros(16, dtype=torch.float64), 1e-6)
    assert torch.allclose(P.rms_norm_one_plus_w(x, w, 1e-6), base * (1 + w))
    assert not torch.allclose(P.rms_norm_one_plus_w(x, w, 1e-6), base * w)


def test_norm_ignores_the_scale_of_its_input():
    x = torch.randn(4, 32, dtype=torch.float64)
    w = torch.randn(32, dtype=torch.float64) * 0.1
    assert torch.allclose(P.rms_norm_one_plus_w(7.0 * x, w, 1e-12), P.rms_norm_one_plus_w(x, w, 1e-12), atol=1e-9)


# ---- embedding ---------------------------------------------------------------------------
def test_embedding_is_scaled_by_sqrt_hidden():
    table = torch.randn(10, 64, dtype=torch.float64)
    ids = torch.tensor([3, 3, 9])
    assert torch.equal(P.embed(ids, table, 64), table[ids] * 8.0)           # sqrt(64) exactly
    # the factor held in bfloat16: sqrt(2048) = 45.2548... becomes 45.25 (src/wllm/models/gemma.py:158-162)
    t = torch.ones(1, 2048, dtype=torch.float32)
    assert P.embed(torch.tensor([0]), t, 2048, torch.bfloat16)[0, 0].item() == 45.25
    assert abs(P.embed(torch.tensor([0]), t, 2048)[0, 0].item() - math.sqrt(2048)) < 1e-5


# ---- rotation ----------------------------------------------------------------------------------
def test_rotation_at_position_zero_is_identity_and_norms_are_kept():
    x = torch.randn(6, 3, 16, dtype=torch.float64)
    cos, sin = P.rope_cos_sin(torch.zeros(6, dtype=torch.long), 16, 10000.0, torch.float64)
    assert torch.allclose(P.apply_rope(x, cos, sin), x)
    cos, sin = P.rope_cos_sin(torch.arange(6), 16, 10000.0, torch.float64)
    y = P.apply_rope(x, cos, sin)
    pair = lambda t: t[..., :8].pow(2) + t[..., 8:].pow(2)     # element j with j + d/2
    assert torch.allclose(pair(y), pair(x))


def test_rotation_pairs_halves_and_turns_counterclockwise():
    # d = 4, position 1: pairs are (0, 2) and (1, 3); the first pair turns by 1 radian
    x = torch.tensor([[[1.0, 0.0, 0.0, 0.0]]], dtype=torch.float64)
    cos, sin = P.rope_cos_sin(torch.tensor([1]), 4, 10000.0, torch.float64)
    y = P.apply_rope(x, cos, sin)[0, 0]
    assert torch.allclose(y, torch.tensor([math.cos(1.0), 0.0, math.sin(1.0), 0.0], dtype=torch.float64))
    # frequency of pair j is theta^(-2j/d)
    x = torch.tensor([[[0.0, 1.0, 0.0, 0.0]]], dtype=torch.float64)
    y = P.apply_rope(x, cos, sin)[0, 0]
    a = 10000.0 ** (-2.0 / 4.0)
    assert torch.allclose(y, torch.tensor([0.0, math.cos(a), 0.0, math.sin(a)], dtype=torch.float64))


def test_rotated_dot_products_depend_on_distance_only():
    q = torch.randn(1, 1, 32, dtype=torch.float64)
    k = torch.randn(1, 1, 32, dtype=torch.float64)

    def dot(m, n):
        cq, sq = P.rope_cos_sin(torch.tensor([m]), 32, 500.0, torch.float64)
        ck, sk = P.rope_cos_sin(torch.tensor([n]), 32, 500.0, torch.float64)
        return (P.apply_rope(q, cq, sq) * P.apply_rope(k, ck, sk)).sum()

    assert torch.allclose(dot(5, 2), dot(105, 102))
    assert not torch.allclose(dot(5, 2), dot(2, 5))


def test_rotation_vanishes_for_huge_theta():
    x = torch.randn(4, 2, 8, dtype=torch.float64)
    cos, sin = P.rope_cos_sin(torch.arange(4), 8, 1e300, torch.float64)
    y = P.apply_rope(x, cos, sin)
    # only the first pair (frequency 1) still turns
    assert torch.allclose(y[..., 1:4], x[..., 1:4]) and torch.allclose(y[..., 5:], x[..., 5:])


# ---- attention -----------------------------------------------------------------------------------
def test_attention_equals_the_library_routine():
    T, nh, d = 9, 4, 16
    q, k, v = (torch.randn(T, nh, d, dtype=torch.float64) for _ in range(3))
    ref = torch.nn.functional.scaled_dot_product_attention(
        q.transpose(0, 1)[None], k.transpose(0, 1)[None], v.transpose(0, 1)[None], is_causal=True)[0].transpose(0, 1)
    assert torch.allclose(P.causal_attention(q, k, v, d), ref)


def test_attention_scale_is_head_dim_not_hidden_over_heads():
    T, nh, d = 5, 2, 16
    q, k, v = (torch.randn(T, nh, d, dtype=torch.float64) for _ in range(3))
    scores = torch.einsum("qhd,khd->hqk", q, k) / math.sqrt(d)
    probs = torch.softmax(scores.masked_fill(~torch.ones(T, T, dtype=torch.bool).tril(), float("-inf")), -1)
    assert torch.allclose(P.causal_attention(q, k, v, d), torch.einsum("hqk,khd->qhd", probs, v))


def test_attention_first_token_returns_its_value_and_equal_scores_give_the_mean():
    T, d = 6, 8
    q = torch.zeros(T, 1, d, dtype=torch.float64)
    k, v = torch.randn(T, 1, d, dtype=torch.float64), torch.randn(T, 1, d, dtype=torch.float64)
    o = P.causal_attention(q, k, v, d)
    assert torch.allclose(o[0, 0], v[0, 0])
    for t in range(T):
        assert torch.allclose(o[t, 0], v[:t + 1, 0].mean(0))


def test_grouped_heads_read_the_key_head_of_their_group():
    # query head h uses kv head h // (nh // nkv): grouped attention equals full attention
    # on key/value heads repeated in place
    T, nh, nkv, d = 7, 6, 2, 8
    q = torch.randn(T, nh, d, dtype=torch.float64)
    k, v = torch.randn(T, nkv, d, dtype=torch.float64), torch.randn(T, nkv, d, dtype=torch.float64)
    full = P.causal_attention(q, k.repeat_interleave(3, 1), v.repeat_interleave(3, 1), d)
    assert torch.allclose(P.causal_attention(q, k, v, d), full)
    wrong = P.causal_attention(q, k.repeat(1, 3, 1), v.repeat(1, 3, 1), d)      # interleaved the other way
    assert not torch.allclose(P.causal_attention(q, k, v, d), wrong)


# ---- feed-forward ----------------------------------------------------------------------------
def test_gelu_is_the_tanh_approximation():
    z = torch.linspace(-6, 6, 101, dtype=torch.float64)
    assert torch.allclose(P.gelu_tanh(z), torch.nn.functional.gelu(z, approximate="tanh"))
    assert not torch.allclose(P.gelu_tanh(z), torch.nn.functional.gelu(z), atol=1e-5)


def test_feed_forward_gates_with_the_gate_projection():
    h = torch.randn(3, 8, dtype=torch.float64)
    wg, wu, wd = (torch.randn(*s, dtype=torch.float64) for s in ((12, 8), (12, 8), (8, 12)))
    ref = (torch.nn.functional.gelu(h @ wg.T, approximate="tanh") * (h @ wu.T)) @ wd.T
    assert torch.allclose(P.geglu_mlp(h, wg, wu, wd), ref)
    assert torch.equal(P.geglu_mlp(h, torch.zeros_like(wg), wu, wd), torch.zeros(3, 8, dtype=torch.float64))


# ---- the whole model -----------------------------------------------------------------------------
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_logits_do_not_change_when_all_positions_move(model_folders, name):
    cfg = P.read_config(model_folders[name])
    w = P.read_weights(model_folders[name], torch.float64)
    ids = torch.randint(0, cfg["vocab_size"], (11,))
    a = P.forward_logits(cfg, w, ids)
    b = P.forward_logits(cfg, w, ids, positions=torch.arange(11) + 37)
    assert torch.allclose(a, b, atol=1e-9)


def test_logits_are_causal(model_folders):
    cfg = P.read_config(model_folders["A"])
    w = P.read_weights(model_folders["A"], torch.float64)
    ids = torch.randint(0, cfg["vocab_size"], (10,))
    full = P.forward_logits(cfg, w, ids)
    assert torch.allclose(P.forward_logits(cfg, w, ids[:6]), full[:6], atol=1e-10)


def _hand_norm(x, w, eps):
    return x / torch.sqrt(x.pow(2).mean(-1, keepdim=True) + eps) * (1.0 + w)


@pytest.mark.parametrize("name", ["A", "C"])
def test_layers_that_contribute_nothing_leave_one_final_norm_and_the_unscaled_head(model_folders, tmp_path, name):
    """Every o_proj and down_proj zero: each layer must hand its input on unchanged (the residual
    path, src/wllm/models/gemma.py:83-93), so logits = norm_f(E[ids] * sqrt(H)) @ head^T with exactly
    one final norm (src/wllm/models/llama.py:415) and, when tied, the table as it is stored
    (llama.py:443-446).  A head scaled like the embedding is off by sqrt(H); a second final norm, or
    one left out, changes the (1 + w) factor; a layer that normalises the stream itself changes x."""
    from helpers import degenerate_folder
    folder = degenerate_folder(model_folders[name], str(tmp_path / "none"), "no_contributions")
    cfg = P.read_config(folder)
    w = P.read_weights(folder, torch.float64)
    ids = torch.randint(0, cfg["vocab_size"], (9,))
    table = w["model.embed_tokens.weight"]
    x = table[ids] * math.sqrt(cfg["hidden_size"])
    head = table if cfg["tie_word_embeddings"] else w["lm_head.weight"]
    expected = _hand_norm(x, w["model.norm.weight"], cfg["rms_norm_eps"]) @ head.T
    got = P.forward_logits(cfg, w, ids)
    assert torch.allclose(got, expected, atol=1e-10)
    # the plausible mistakes are far away: a head scaled like the embedding, no final norm, two of them
    assert not torch.allclose(got, expected * math.sqrt(cfg["hidden_size"]), atol=1e-3)
    assert not torch.allclose(got, x @ head.T, atol=1e-3)
    twice = _hand_norm(_hand_norm(x, w["model.norm.weight"], cfg["rms_norm_eps"]), w["model.norm.weight"], cfg["rms_norm_eps"])
    assert not torch.allclose(got, twice @ head.T, atol=1e-3)


@pytest.mark.parametrize("name", ["A", "B"])
def test_one_feed_forward_is_added_to_the_stream_it_read_through_a_norm(model_folders, tmp_path, name):
    """Only layer 0's feed-forward contributes: logits = norm_f(x + mlp(norm_2(x))) @ E^T, x = E[ids] * sqrt(H)
    (src/wllm/models/gemma.py:89-93): the feed-forward reads the normalised stream and is added to the
    stream as it was, not to its normalised copy, and nothing is normalised after the sum but the
    final norm."""
    from helpers import degenerate_folder
    folder = degenerate_folder(model_folders[name], str(tmp_path / "one"), "one_feed_forward")
    cfg = P.read_config(folder)
    w = P.read_weights(folder, torch.float64)
    ids = torch.randint(0, cfg["vocab_size"], (7,))
    eps, p = cfg["rms_norm_eps"], "model.layers.0."
    x = w["model.embed_tokens.weight"][ids] * math.sqrt(cfg["hidden_size"])
    h = _hand_norm(x, w[p + "post_attention_layernorm.weight"], eps)
    gate, up = h @ w[p + "mlp.gate_proj.weight"].T, h @ w[p + "mlp.up_proj.weight"].T
    mlp = (torch.nn.functional.gelu(gate, approximate="tanh") * up) @ w[p + "mlp.down_proj.weight"].T
    assert mlp.abs().max() > 1e-3 * x.abs().max(), "the feed-forward matters in this test"
    expected = _hand_norm(x + mlp, w["model.norm.weight"], eps) @ w["model.embed_tokens.weight"].T
    got = P.forward_logits(cfg, w, ids)
    assert torch.allclose(got, expected, atol=1e-10)
    # post-norm wiring (the sum normalised, or the feed-forward added to the normalised copy) is far away
    assert not torch.allclose(got, _hand_norm(h + mlp, w["model.norm.weight"], eps) @ w["model.embed_tokens.weight"].T, atol=1e-3)
    unnormed = (torch.nn.functional.gelu(x @ w[p + "mlp.gate_proj.weight"].T, approximate="tanh")
                * (x @ w[p + "mlp.up_proj.weight"].T)) @ w[p + "mlp.down_proj.weight"].T
    assert not torch.allclose(got, _hand_norm(x + unnormed, w["model.norm.weight"], eps) @ w["model.embed_tokens.weight"].T, atol=1e-3)


def _hand_attention(h, w, p, cfg):
    """Attention of one layer written out with the library's routines: projections, the rotation as the
    complex product (x_j + i x_{j+d/2}) * exp(i * pos * theta^(-2j/d)), causal SDPA head by head."""
    nh, nkv, d = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"]
    T = h.shape[0]
    angle = torch.arange(T, dtype=torch.float64)[:, None] * cfg["rope_theta"] ** (-torch.arange(0, d, 2, dtype=torch.float64) / d)
    turn = torch.polar(torch.ones_like(angle), angle)[:, None, :]            # [T, 1, d/2]

    def rotated(x, heads):
        x = x.view(T, heads, d)
        z = torch.complex(x[..., :d // 2], x[..., d // 2:]) * turn
        return torch.cat((z.real, z.imag), -1)

    q = h @ w[p + "self_attn.q_proj.weight"].T
    k = h @ w[p + "self_attn.k_proj.weight"].T
    v = h @ w[p + "self_attn.v_proj.weight"].T
    if cfg["attention_bias"]:
        q, k, v = (t + w[p + f"self_attn.{n}_proj.bias"] for t, n in ((q, "q"), (k, "k"), (v, "v")))
    q, k, v = rotated(q, nh), rotated(k, nkv), v.view(T, nkv, d)
    out = torch.empty(T, nh, d, dtype=torch.float64)
    for head in range(nh):
        kv = head // (nh // nkv)
        out[:, head] = torch.nn.functional.scaled_dot_product_attention(q[None, :, head], k[None, :, kv], v[None, :, kv],
                                                                        is_causal=True)[0]
    return out.reshape(T, nh * d) @ w[p + "self_attn.o_proj.weight"].T


@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_one_attention_reads_the_input_norm_and_is_added_to_the_stream_as_it_was(model_folders, tmp_path, name):
    """Only layer 0's attention contributes: logits = norm_f(x + attn(norm_1(x))) @ head^T, x = E[ids] * sqrt(H)
    (src/wllm/models/gemma.py:83-87): attention reads the stream through `input_layernorm` (not through the
    layer's other norm, and not the raw stream), and its output is added to the stream as it was, which
    nothing normalises before the next norm."""
    from helpers import degenerate_folder
    folder = degenerate_folder(model_folders[name], str(tmp_path / "attn"), "one_attention")
    cfg = P.read_config(folder)
    w = P.read_weights(folder, torch.float64)
    ids = torch.randint(0, cfg["vocab_size"], (13,))
    eps, p = cfg["rms_norm_eps"], "model.layers.0."
    table = w["model.embed_tokens.weight"]
    head = table if cfg["tie_word_embeddings"] else w["lm_head.weight"]
    # the factor is a float32 number in the reference (src/wllm/models/llama.py:388-397), also under a wider model
    x = table[ids] * float(torch.tensor(cfg["hidden_size"] ** 0.5, dtype=torch.float32))
    final = lambda t: _hand_norm(t, w["model.norm.weight"], eps) @ head.T
    h = _hand_norm(x, w[p + "input_layernorm.weight"], eps)
    attn = _hand_attention(h, w, p, cfg)
    assert attn.abs().max() > 1e-3 * x.abs().max(), "the attention matters in this test"
    got = P.forward_logits(cfg, w, ids)
    assert torch.allclose(got, final(x + attn), atol=1e-10)
    # the plausible mistakes are far away: the other norm's weight, the raw stream, the sum on the
    # normalised copy, the attention's output normalised
    other = _hand_attention(_hand_norm(x, w[p + "post_attention_layernorm.weight"], eps), w, p, cfg)
    raw = _hand_attention(x, w, p, cfg)
    for wrong in (final(x + other), final(x + raw), final(h + attn), final(x + _hand_norm(attn, w[p + "input_layernorm.weight"], eps))):
        assert not torch.allclose(got, wrong, atol=1e-3)


def test_biases_are_added_before_the_rotation():
    """q_proj and k_proj weights zero, biases b_q and b_k: the query at position p is rope(b_q, p) and the
    key at s is rope(b_k, s) (src/wllm/models/llama.py:95-98,103-110: the Linear with its bias, then
    apply_rotary_pos_emb), so the scores depend on p - s.  Added after the rotation the biases would
    give every key of a head the same score and the output the running mean of v."""
    torch.manual_seed(3)
    T, nh, nkv, d, H = 9, 4, 2, 8, 12
    cfg = dict(num_attention_heads=nh, num_key_value_heads=nkv, head_dim=d, attention_bias=True)
    w = {"q_proj.weight": torch.zeros(nh * d, H, dtype=torch.float64), "k_proj.weight": torch.zeros(nkv * d, H, dtype=torch.float64),
         "v_proj.weight": torch.randn(nkv * d, H, dtype=torch.float64), "o_proj.weight": torch.eye(nh * d, dtype=torch.float64),
         "q_proj.bias": torch.randn(nh * d, dtype=torch.float64) * 2, "k_proj.bias": torch.randn(nkv * d, dtype=torch.float64) * 2,
         "v_proj.bias": torch.zeros(nkv * d, dtype=torch.float64)}
    h = torch.randn(T, H, dtype=torch.float64)
    cos, sin = P.rope_cos_sin(torch.arange(T), d, 100.0, torch.float64)
    got = P.attention_block(h, w, "", cfg, cos, sin).view(T, nh, d)
    v = (h @ w["v_proj.weight"].T).view(T, nkv, d)
    # by hand: the rotated biases as queries and keys, one head and one position at a time
    for head in range(nh):
        kv = head // (nh // nkv)
        for p in range(T):
            q = P.apply_rope(w["q_proj.bias"].view(1, nh, d), cos[p:p + 1], sin[p:p + 1])[0, head]
            keys = torch.stack([P.apply_rope(w["k_proj.bias"].view(1, nkv, d), cos[s:s + 1], sin[s:s + 1])[0, kv]
                                for s in range(p + 1)])
            probs = torch.softmax(keys @ q / math.sqrt(d), -1)
            assert torch.allclose(got[p, head], probs @ v[:p + 1, kv], atol=1e-12)
    running_mean = v.cumsum(0) / torch.arange(1, T + 1, dtype=torch.float64)[:, None, None]
    assert not torch.allclose(got[:, 0], running_mean[:, 0], atol=1e-3), "biases after the rotation would give this"


# ---- the bound of the bfloat16 comparisons ---------------------------------------------------------
def test_the_rounded_run_rounds_and_stays_near_the_exact_one(model_folders):
    """`round_to=torch.bfloat16` changes every row a little (a few roundings of 2^-9 each) and no row much."""
    from helpers import plain_exact_and_rounded
    cfg = P.read_config(model_folders["M"])
    w = P.read_weights(model_folders["M"], torch.float64)
    exact, realisations = plain_exact_and_rounded(cfg, w, torch.randint(0, cfg["vocab_size"], (40,)))
    assert len(realisations) == 4
    for rounded in realisations:
        rel = (rounded - exact).pow(2).mean(-1).sqrt() / exact.pow(2).mean(-1).sqrt()
        assert (rel > 2.0 ** -11).all() and (rel < 0.05).all(), rel
        assert torch.equal(rounded, rounded.to(torch.bfloat16).double()), "the logits themselves are rounded"
    # realisations are draws of the same noise: they differ from each other as much as from the exact run
    assert (realisations[0] - realisations[1]).abs().max() > 0.3 * (realisations[0] - exact).abs().max()
    # no rounding asked for: the same numbers as before
    assert torch.equal(P.forward_logits(cfg, w, [1, 2, 3], round_to=None), P.forward_logits(cfg, w, [1, 2, 3]))


def test_a_lost_or_foreign_key_that_carries_weight_is_far_beyond_the_bfloat16_bound(model_folders, tmp_path):
    """The bound of the bfloat16 comparisons is a multiple of the rounded run's own distance from the
    exact logits.  A fault is no rounding: in a model whose attention is sharp (queries and keys scaled
    up, as tests/test_engine_gpu.py does), a query that loses the key it weighs most, or sees a key
    of the future in its place, lands many times the bound away, rounded like everything else.  A key
    that carries no weight (one of hundreds under flat attention) hides below bfloat16's rounding from
    any bound; the float32 comparisons, fifty times as narrow as one such key's share, are there for it."""
    import os
    from helpers import bfloat16_row_errors, plain_exact_and_rounded
    from wllm_amd.weights import Checkpoint, write_safetensors
    src, folder = model_folders["M"], str(tmp_path / "sharp")
    os.makedirs(folder)
    ck = Checkpoint(src)
    tensors = {n: ck.tensor(n) for n in ck.names()}
    ck.close()
    for n in tensors:
        if n.endswith(("q_proj.weight", "k_proj.weight")):
            tensors[n] = (tensors[n].float() * 6.0).to(torch.bfloat16)
    write_safetensors(os.path.join(folder, "model.safetensors"), tensors)
    with open(os.path.join(src, "config.json")) as f, open(os.path.join(folder, "config.json"), "w") as g:
        g.write(f.read())
    cfg = P.read_config(folder)
    w = P.read_weights(folder, torch.float64)
    T = 200
    toks = torch.randint(0, cfg["vocab_size"], (T,), generator=torch.Generator().manual_seed(5))
    exact, rounded = plain_exact_and_rounded(cfg, w, toks)
    # the key each query of layer 0 weighs most, over its heads
    nh, nkv, d = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"]
    h = P.rms_norm_one_plus_w(P.embed(toks, w["model.embed_tokens.weight"], cfg["hidden_size"]),
                              w["model.layers.0.input_layernorm.weight"], cfg["rms_norm_eps"])
    cos, sin = P.rope_cos_sin(torch.arange(T), d, cfg["rope_theta"], torch.float64)
    q = P.apply_rope((h @ w["model.layers.0.self_attn.q_proj.weight"].T).view(T, nh, d), cos, sin)
    k = P.apply_rope((h @ w["model.layers.0.self_attn.k_proj.weight"].T).view(T, nkv, d), cos, sin)
    scores = torch.einsum("qhd,khd->hqk", q, k.repeat_interleave(nh // nkv, 1)) / math.sqrt(d)
    probs = torch.softmax(scores.masked_fill(~torch.ones(T, T, dtype=torch.bool).tril(), float("-inf")), -1).mean(0)
    checked = 0
    # the four late queries whose heads agree most on one key
    late = sorted(range(50, T), key=lambda i: -float(probs[i].max()))[:4]
    for p_ in late:
        top = int(probs[p_].argmax())
        assert probs[p_, top] > 0.2, "the attention is sharp"

        def lose(layer, allowed, p_=p_, top=top):
            if layer == 0:
                allowed = allowed.clone()
                allowed[p_, top] = False
            return allowed

        bad = P.forward_logits(cfg, w, toks, round_to=torch.bfloat16, tamper=lose)
        assert max(bfloat16_row_errors(bad[p_], exact[p_], [r[p_] for r in rounded])) > 4.0, (p_, top)
        # the rows before it are the rounded run's own and within the bound
        assert max(bfloat16_row_errors(bad[p_ - 1], exact[p_ - 1], [r[p_ - 1] for r in rounded])) <= 1.0
        checked += 1
    # a key of the future (a stale slot of the page): a query early enough for one key to move it
    def foreign(layer, allowed):
        if layer == 0:
            allowed = allowed.clone()
            allowed[3, 4:40] = True
        return allowed
    bad = P.forward_logits(cfg, w, toks, round_to=torch.bfloat16, tamper=foreign)
    assert max(bfloat16_row_errors(bad[3], exact[3], [r[3] for r in rounded])) > 4.0
    assert checked == 4


def test_head_dim_key_wins_over_the_derived_value(tmp_path):
    # the reference's own vector: 3072 / 16 gives 192, the key says 256
    # (tests/test_gemma_architecture.py:40-60)
    import json
    raw = dict(vocab_size=100, hidden_size=3072, intermediate_size=256, num_hidden_layers=1,
               num_attention_heads=16, num_key_value_heads=16, head_dim=256)
    (tmp_path / "config.json").write_text(json.dumps(raw))
    assert P.read_config(str(tmp_path))["head_dim"] == 256
    del raw["head_dim"]
    (tmp_path / "config.json").write_text(json.dumps(raw))
    assert P.read_config(str(tmp_path))["head_dim"] == 192


def test_greedy_generation_recomputes_everything(model_folders):
    cfg = P.read_config(model_folders["A"])
    w = P.read_weights(model_folders["A"], torch.float32)
    out = P.generate_greedy(cfg, w, [5, 9, 2], 4)
    assert len(out) == 4
    assert out[0] == int(P.forward_logits(cfg, w, [5, 9, 2])[-1].argmax())
    assert out[1] == int(P.forward_logits(cfg, w, [5, 9, 2, out[0]])[-1].argmax())


# ---- sampling --------------------------------------------------------------------------------
def test_repetition_penalty_vector_of_the_reference():
    # tests/test_sampling.py:49-55: [2, -2, 0.5], ids [0, 1], penalty 2 -> [1, -4, 0.5]
    out = S.apply_repetition_penalty(torch.tensor([2.0, -2.0, 0.5]), [0, 1, 1], 2.0)
    assert out.tolist() == [1.0, -4.0, 0.5]


def test_greedy_and_top_k_one_are_argmax_and_logprob_is_log_softmax():
    logits = torch.randn(100)
    tok, lp, _, _ = S.sample_row(logits, 0.0, 0, 1.0, 0.0, 1.0, [], 0.99)
    assert tok == int(logits.argmax())
    assert abs(lp - float(torch.log_softmax(logits.double(), -1)[tok])) < 1e-12
    for u in (0.0, 0.5, 0.999):
        assert S.sample_row(logits, 1.0, 1, 1.0, 0.0, 1.0, [], u)[0] == int(logits.argmax())


def test_top_p_keeps_the_top_token_even_if_it_alone_exceeds_p():
    # tests/test_sampling.py:90-97
    logits = torch.full((10,), -100.0)
    logits[3] = 100.0
    assert S.sample_row(logits, 1.0, 0, 0.1, 0.0, 1.0, [], 0.7)[0] == 3


def test_truncations_on_a_known_distribution():
    probs = torch.tensor([0.5, 0.25, 0.125, 0.0625, 0.0625])
    scaled = probs.log().double()
    assert S.keep_mask(scaled, 2, 1.0, 0.0).tolist() == [True, True, False, False, False]
    # cumulative 0.5, 0.75, 0.875 ...: the token that crosses p is dropped
    assert S.keep_mask(scaled, 0, 0.8, 0.0).tolist() == [True, True, False, False, False]
    assert S.keep_mask(scaled, 0, 0.4, 0.0).tolist() == [True, False, False, False, False]
    assert S.keep_mask(scaled, 0, 1.0, 0.2).tolist() == [True, True, True, False, False]


def test_draw_inverts_the_cumulative_distribution():
    logits = torch.tensor([0.5, 0.25, 0.125, 0.125]).log()
    draws = [S.sample_row(logits, 1.0, 0, 1.0, 0.0, 1.0, [], u)[0] for u in (0.0, 0.49, 0.51, 0.74, 0.76, 0.9)]
    assert draws == [0, 0, 1, 1, 2, 3]


def test_philox_known_answers():
    # Random123's known-answer vectors for philox4x32-10: all-zero and all-ones counter and key
    assert abs(S.philox_uniform(0, 0) - (((0x6627e8d5 << 32) | 0xe169c58d) >> 11) / 2 ** 53) < 1e-18
    us = [S.philox_uniform(7, c) for c in range(2000)]
    assert 0.45 < sum(us) / len(us) < 0.55 and len(set(us)) == 2000
