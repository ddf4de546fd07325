"""The entry point that allocates nothing (`wllm_sample_rows_static`, csrc/wllm_no_alloc.h), called
through ctypes as a caller outside this package would call it, against the entry point it is a
variant of (`wllm_sample_rows_split`, whose scratch area the caller allocates): two calls in a row,
the second with a smaller input, give the same tokens and log-probabilities bit for bit; more rows
than its maximum are refused with an error code that has a text.  Its tokens are also held against the
plain sampler (tests/plain/sampling_plain.py), so that the check does not rest on another path of
the library alone."""
import ctypes
from ctypes import c_char_p, c_int, c_void_p

import pytest
import torch

pytestmark = pytest.mark.gpu


def _library():
    from wllm_amd.kernels.library import load
    lib = load()
    lib.wllm_sample_rows_static.argtypes = [c_void_p] * 7 + [c_int, c_int, c_int, c_void_p]
    lib.wllm_sample_rows_static.restype = c_int
    lib.wllm_sample_rows_split.argtypes = [c_void_p] * 8 + [c_int, c_int, c_int, c_void_p]
    lib.wllm_sample_rows_split.restype = c_int
    lib.wllm_sample_static_max_rows.restype = c_int
    lib.wllm_sample_static_init.restype = c_int
    lib.wllm_sample_static_error.argtypes = [c_int]
    lib.wllm_sample_static_error.restype = c_char_p
    lib.wllm_sample_split_row_words.restype = c_int
    return lib


def _inputs(rows, vocab, seed):
    g = torch.Generator().manual_seed(seed)
    logits = (torch.randn(rows, vocab, generator=g) * 3.0).cuda()
    params = torch.tensor([[0.0, 0, 1.0, 0.0, 1.0], [0.8, 0, 1.0, 0.0, 1.0], [1.0, 20, 0.9, 0.0, 1.0], [0.7, 0, 0.8, 0.05, 1.3],
                           [1.2, 5, 1.0, 0.0, 1.0]], dtype=torch.float32)[torch.arange(rows) % 5].contiguous().cuda()
    seeds = torch.stack([torch.arange(rows, dtype=torch.int64) + 1000 * seed, torch.arange(rows, dtype=torch.int64) % 7], 1).contiguous().cuda()
    # ids the repetition penalty applies to: three per row
    ids = torch.randint(0, vocab, (rows * 3,), generator=g, dtype=torch.int32).cuda()
    offsets = (torch.arange(rows + 1, dtype=torch.int32) * 3).cuda()
    return logits, params, seeds, ids, offsets


def _call(lib, static, logits, params, seeds, ids, offsets):
    rows, vocab = logits.shape
    logits = logits.clone()                       # the penalty changes logits in place
    tokens = torch.full((rows,), -7, dtype=torch.int32, device="cuda")
    logprobs = torch.full((rows,), float("nan"), dtype=torch.float32, device="cuda")
    stream = c_void_p(torch.cuda.current_stream().cuda_stream)
    head = [c_void_p(t.data_ptr()) for t in (logits, params, seeds, ids, offsets, tokens, logprobs)]
    if static:
        code = lib.wllm_sample_rows_static(*head, rows, vocab, 1, stream)
    else:
        scratch = torch.empty(rows * lib.wllm_sample_split_row_words(), dtype=torch.int64, device="cuda")
        code = lib.wllm_sample_rows_split(*head, c_void_p(scratch.data_ptr()), rows, vocab, 1, stream)
    torch.cuda.synchronize()
    return code, tokens.cpu(), logprobs.cpu()


def test_the_entry_point_without_allocation_gives_what_the_one_with_a_caller_buffer_gives():
    lib = _library()
    assert lib.wllm_sample_static_max_rows() == 64
    print("no-alloc sampler: init", flush=True)
    assert lib.wllm_sample_static_init() == 0
    # two calls in a row, the second smaller in rows and in vocabulary; then a full-size one again
    for rows, vocab, seed in ((48, 5003, 1), (5, 777, 2), (64, 2048, 3)):
        print(f"no-alloc sampler: rows {rows} vocab {vocab}", flush=True)
        inputs = _inputs(rows, vocab, seed)
        code_a, tok_a, lp_a = _call(lib, False, *inputs)
        before = torch.cuda.memory_allocated()
        code_b, tok_b, lp_b = _call(lib, True, *inputs)
        assert code_a == 0 and code_b == 0, lib.wllm_sample_static_error(code_b)
        assert torch.equal(tok_a, tok_b), (tok_a, tok_b)
        assert torch.equal(lp_a, lp_b)
        assert (tok_b >= 0).all() and (tok_b < vocab).all() and torch.isfinite(lp_b).all()
        assert len(set(tok_b.tolist())) > 1 or rows == 1
        assert torch.cuda.memory_allocated() == before
    # greedy rows are the argmax of the penalised logits whatever the array held before
    inputs = _inputs(10, 901, 4)
    _, tok, _ = _call(lib, True, *inputs)
    again = _call(lib, True, *inputs)[1]
    assert torch.equal(tok, again), "the last call's contents do not leak into the next"


def test_the_entry_point_without_allocation_follows_the_plain_sampler():
    """Every row's token is the one whose interval of the plain sampler's cumulative distribution holds
    the row's uniform number (greedy rows: the argmax of the penalised logits), and its log-probability
    is the plain sampler's."""
    from plain import sampling_plain as S
    lib = _library()
    assert lib.wllm_sample_static_init() == 0
    rows, vocab = 20, 1500
    logits, params, seeds, ids, offsets = _inputs(rows, vocab, 6)
    code, tokens, logprobs = _call(lib, True, logits, params, seeds, ids, offsets)
    assert code == 0
    for r in range(rows):
        temperature, top_k, top_p, min_p, penalty = params[r].tolist()
        generated = ids[int(offsets[r]):int(offsets[r + 1])].tolist()
        u = S.philox_uniform(int(seeds[r, 0]), int(seeds[r, 1]))
        token, logprob, keep, span = S.sample_row(logits[r].cpu(), temperature, int(top_k), top_p, min_p, penalty, generated, u)
        got = int(tokens[r])
        if temperature == 0.0:
            assert got == token, f"row {r}"
        else:
            low, high = span
            assert bool(keep[got]) and low[got] - 1e-4 <= u <= high[got] + 1e-4, f"row {r}: token {got} for u {u}"
            logprob = float(torch.log_softmax(S.apply_repetition_penalty(logits[r].cpu().double(), generated, penalty)
                                              / max(temperature, 1e-5), -1)[got])
        assert abs(float(logprobs[r]) - logprob) < 1e-3, f"row {r}"


def test_more_rows_than_the_maximum_are_refused_with_a_clear_error():
    lib = _library()
    inputs = _inputs(65, 300, 5)
    code, tokens, _ = _call(lib, True, *inputs)
    assert code == -2 and (tokens == -7).all(), "nothing was launched"
    assert b"64" in lib.wllm_sample_static_error(code) and b"rows" in lib.wllm_sample_static_error(code)
    assert lib.wllm_sample_static_error(0) == b"success"
    bad = lib.wllm_sample_rows_static(None, None, None, None, None, None, None, 1, 300, 1, None)
    assert bad == -1
