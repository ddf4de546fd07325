"""The sampling kernel against the plain sampler (written from the reference's `sample`)."""
import pytest
import torch

from plain import sampling_plain as S
from wllm_amd.kernels import ops
from wllm_amd.sampling import Sampler, SamplingParams

pytestmark = pytest.mark.gpu
DEV = "cuda"


def run(logits, params_rows, seeds, generated=None):
    m = logits.shape[0]
    sampler = Sampler(DEV)
    params = [SamplingParams(*p) for p in params_rows]
    toks, lps = sampler.sample(logits.clone().to(DEV), params, [s for s, _ in seeds], [c for _, c in seeds], generated)
    return toks, lps


def test_greedy_is_argmax_with_log_softmax_as_logprob():
    # tests/test_sampling.py:14-24,77-87
    torch.manual_seed(0)
    logits = torch.randn(4, 100)
    toks, lps = run(logits, [(0.0,)] * 4, [(1, 0)] * 4)
    assert toks == logits.argmax(-1).tolist()
    ref = torch.log_softmax(logits, -1).gather(-1, logits.argmax(-1, keepdim=True)).squeeze(-1)
    assert torch.allclose(torch.tensor(lps), ref, atol=1e-4)
    toks2, _ = run(logits, [(0.0,)] * 4, [(999, 5)] * 4)
    assert toks2 == toks, "the random state does not change greedy output"
    out = torch.zeros(4, dtype=torch.int32, device=DEV)
    ops.argmax_rows(logits.to(DEV), out)
    assert out.tolist() == toks


def test_top_k_one_is_argmax_and_rows_are_independent():
    # tests/test_sampling.py:27-46
    torch.manual_seed(0)
    logits = torch.randn(8, 50)
    toks, _ = run(logits, [(1.0, 1)] * 8, [(3, i) for i in range(8)])
    assert toks == logits.argmax(-1).tolist()
    mixed, _ = run(logits[:2], [(0.0,), (1.0, 1)], [(3, 0), (3, 1)])
    assert mixed == logits[:2].argmax(-1).tolist()


def test_repetition_penalty_vector_of_the_reference():
    # tests/test_sampling.py:49-55: [2, -2, 0.5] with ids [0, 1] and penalty 2 becomes [1, -4, 0.5];
    # greedy then picks token 0 with the log-softmax of the penalised row
    logits = torch.tensor([[2.0, -2.0, 0.5], [0.4, -2.0, 0.5]])
    toks, lps = run(logits, [(0.0, 0, 1.0, 0.0, 2.0)] * 2, [(0, 0)] * 2, [[0, 1, 1, 0], [0, 1]])
    assert toks == [0, 2]
    ref = torch.log_softmax(torch.tensor([[1.0, -4.0, 0.5], [0.2, -4.0, 0.5]]), -1)
    assert abs(lps[0] - ref[0, 0].item()) < 1e-5 and abs(lps[1] - ref[1, 2].item()) < 1e-5


def test_top_p_never_drops_the_top_token():
    # tests/test_sampling.py:90-97
    logits = torch.full((1, 10), -100.0)
    logits[0, 3] = 100.0
    assert run(logits, [(1.0, 0, 0.1)], [(5, 5)])[0] == [3]


CASES = [
    (0.8, 0, 1.0, 0.0, 1.0), (1.0, 5, 1.0, 0.0, 1.0), (1.3, 0, 0.7, 0.0, 1.0), (0.7, 0, 1.0, 0.05, 1.0),
    (1.0, 20, 0.9, 0.01, 1.0), (0.5, 0, 0.3, 0.0, 1.3), (2.0, 3, 0.95, 0.2, 0.8), (1e-6, 0, 1.0, 0.0, 1.0),
]


@pytest.mark.parametrize("vocab", [777, 5000])
@pytest.mark.parametrize("case", CASES)
def test_draws_fall_into_the_plain_samplers_interval(case, vocab):
    """The kernel's token for uniform number u must be the token whose interval of the cumulative
    distribution (kept tokens, index order) holds u, up to the rounding of the sums."""
    temperature, top_k, top_p, min_p, pen = case
    torch.manual_seed(vocab)
    rows = 48
    logits = torch.randn(rows, vocab) * 2.5
    generated = [torch.randint(0, vocab, (9,)).tolist() for _ in range(rows)]
    seeds = [(1234 + r, r * 7) for r in range(rows)]
    toks, lps = run(logits, [case] * rows, seeds, generated)
    for r in range(rows):
        u = S.philox_uniform(*seeds[r])
        ref_tok, ref_lp, keep, (low, high) = S.sample_row(logits[r], temperature, top_k, top_p, min_p, pen, generated[r], u)
        t = toks[r]
        assert keep[t], f"row {r}: token {t} was truncated away by the plain sampler"
        assert low[t] - 1e-5 <= u <= high[t] + 1e-5, f"row {r}: u={u} outside [{low[t]}, {high[t]}] of token {t}"
        scaled = S.apply_repetition_penalty(logits[r].double(), generated[r], pen) / max(temperature, 1e-5)
        assert abs(lps[r] - torch.log_softmax(scaled, -1)[t].item()) < 2e-4 * max(1.0, abs(lps[r]))


def test_kept_sets_match_the_plain_sampler_exactly():
    """With u swept over (0, 1) every kept token of a small distribution is drawn and no other."""
    probs = torch.tensor([0.30, 0.05, 0.20, 0.10, 0.02, 0.15, 0.08, 0.10])
    logits = probs.log()[None].repeat(400, 1)
    for case in [(1.0, 3, 1.0, 0.0, 1.0), (1.0, 0, 0.75, 0.0, 1.0), (1.0, 0, 1.0, 0.3, 1.0), (1.0, 6, 0.9, 0.1, 1.0)]:
        toks, _ = run(logits, [case] * 400, [(77, c) for c in range(400)])
        keep = S.keep_mask(probs.log().double(), case[1], case[2], case[3])
        assert set(toks) == set(torch.nonzero(keep).flatten().tolist()), f"{case}: kept {sorted(set(toks))}"


def test_frequencies_follow_the_distribution_and_draws_are_reproducible():
    probs = torch.tensor([0.5, 0.25, 0.125, 0.0625, 0.0625])
    n = 4000
    logits = probs.log()[None].repeat(n, 1)
    seeds = [(42, c) for c in range(n)]
    toks, _ = run(logits, [(1.0,)] * n, seeds)
    freq = torch.bincount(torch.tensor(toks), minlength=5).float() / n
    assert (freq - probs).abs().max() < 0.03
    again, _ = run(logits, [(1.0,)] * n, seeds)
    assert again == toks
    # a row alone draws what it draws in the batch
    assert run(logits[:1], [(1.0,)], [seeds[1234]])[0] == [toks[1234]]
    # half temperature squares the probabilities
    sharp, _ = run(logits, [(0.5,)] * n, seeds)
    f2 = torch.bincount(torch.tensor(sharp), minlength=5).float() / n
    assert (f2 - probs.pow(2) / probs.pow(2).sum()).abs().max() < 0.03


def test_large_vocabulary():
    torch.manual_seed(3)
    logits = torch.randn(3, 256000)
    logits[1, 255999] = 30.0
    toks, lps = run(logits, [(0.0,), (1.0, 0, 0.5), (1.0, 50)], [(1, 1)] * 3)
    assert toks[0] == int(logits[0].argmax()) and toks[1] == 255999
    assert toks[2] in torch.topk(logits[2], 50).indices.tolist()


@pytest.mark.parametrize("vocab", [777, 5000, 256000])
def test_a_row_spread_over_workgroups_draws_what_one_workgroup_draws(vocab):
    """A decode step's few rows are sampled by kernels that cut each row into segments; many rows by
    one workgroup a row.  All sums that decide anything are integer sums, so the two give the same
    token and the same log-probability, bit for bit."""
    torch.manual_seed(vocab + 1)
    rows = len(CASES) * 3
    logits = torch.randn(rows, vocab) * 2.5
    logits[1, vocab - 1] = logits[1].max() + 1.0           # the maximum in the last segment
    logits[2, :] = logits[2, 0]                            # all equal
    cases = [CASES[r % len(CASES)] for r in range(rows)]
    cases[3] = (0.0,)                                      # a greedy row among the others
    generated = [torch.randint(0, vocab, (9,)).tolist() for _ in range(rows)]
    seeds = [(99 + r, r * 3) for r in range(rows)]
    be = ops.backend()
    limit = be.SAMPLE_SPLIT_ROWS
    assert rows <= limit
    split = run(logits, cases, seeds, generated)
    try:
        be.SAMPLE_SPLIT_ROWS = 0
        whole = run(logits, cases, seeds, generated)
    finally:
        be.SAMPLE_SPLIT_ROWS = limit
    assert split[0] == whole[0]
    assert split[1] == whole[1]
    # rows without top-k and top-p skip the passes for their thresholds
    plain = [(0.9,), (1.2, 0, 1.0, 0.02), (0.0,)] * 2
    a = run(logits[:6], plain, seeds[:6])
    try:
        be.SAMPLE_SPLIT_ROWS = 0
        b = run(logits[:6], plain, seeds[:6])
    finally:
        be.SAMPLE_SPLIT_ROWS = limit
    assert a == b


def test_starting_a_sampling_does_not_wait_for_the_gpu():
    """`Sampler.start` only enqueues: behind a tenth of a second of queued products it returns
    while they still run (its per-row numbers travel from page-locked memory), and what it then
    gives is what a sampling of its own gives."""
    torch.manual_seed(5)
    logits = torch.randn(6, 3000, device=DEV)
    params = [SamplingParams(temperature=0.8, top_k=40, repetition_penalty=1.3 if i % 2 else 1.0, seed=i) for i in range(6)]
    generated = [[i, 2 * i + 1, 17] for i in range(6)]
    sampler = Sampler(DEV)
    expect = sampler.sample(logits.clone(), params, list(range(6)), [3] * 6, generated)
    big = torch.randn(8192, 8192, device=DEV)
    torch.cuda.synchronize()
    for _ in range(12):
        big @ big
    queued = torch.cuda.Event()
    queued.record()
    pending = sampler.start(logits.clone(), params, list(range(6)), [3] * 6, generated)
    assert not queued.query(), "start came back only after the work queued before it had run"
    assert Sampler.finish(pending) == expect
