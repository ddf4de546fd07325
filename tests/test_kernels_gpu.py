"""Each kernel alone against the plain emulation of its contract, at sizes other than
the engine's tests use: widths and vocabularies that are no power of two, odd head
counts and groups (up to 40 query heads a key/value head), partial rotation, windows, pages of
1 to 40 tokens."""
import math

import numpy as np
import pytest
import torch

from kernel_emulation import EmulatedKernels
from wllm_amd.kernels import ops

pytestmark = pytest.mark.gpu
DEV = "cuda"
DTYPES = [torch.float32, torch.bfloat16]


def tol(dtype):
    # float32: accumulation order only; bfloat16: one rounding of the result (2^-8) on top
    return (1e-5, 2e-5) if dtype == torch.float32 else (1e-2, 8e-3)


def close(got, ref, dtype, what=""):
    atol, rtol = tol(dtype)
    got, ref = got.double().cpu(), ref.double().cpu()
    err = ((got - ref).abs() / (atol + rtol * ref.abs())).max().item()
    assert err <= 1.0, f"{what}: worst error {err:.2f} x tolerance, max abs diff {(got - ref).abs().max().item():.3e}"


def both(fn_name, make, dtype):
    """Runs an op on the GPU kernels and on the float64 emulation with equal operands."""
    args_gpu, kwargs = make()
    args_ref = [a.clone() if isinstance(a, torch.Tensor) else a for a in args_gpu]
    getattr(ops, fn_name)(*args_gpu, **kwargs)
    torch.cuda.synchronize()
    with ops.use_backend(EmulatedKernels(precise=True)):
        getattr(ops, fn_name)(*args_ref, **kwargs)
    return args_gpu, args_ref


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("vocab,hidden,n", [(1000, 200, 37), (777, 96, 1), (4099, 2048, 5)])
def test_embed_lookup(dtype, vocab, hidden, n):
    torch.manual_seed(0)
    table = torch.randn(vocab, hidden, device=DEV).to(dtype)
    ids = torch.randint(0, vocab, (n,), device=DEV, dtype=torch.int32)
    ids[0] = vocab - 1
    out = torch.zeros(n, hidden, device=DEV)
    ops.embed_lookup(ids, table, 3.25, out)
    assert torch.equal(out, table[ids.long()].float() * 3.25)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("hidden,n", [(200, 9), (96, 3), (2048, 4), (3072, 2), (70, 130)])
@pytest.mark.parametrize("mode", ["plain", "delta", "rows", "delta_rows"])
def test_rms_norm(dtype, hidden, n, mode):
    torch.manual_seed(1)

    def make():
        x = torch.randn(n, hidden, device=DEV) * 3
        w = torch.randn(hidden, device=DEV) * 0.2
        delta = torch.randn(n, hidden, device=DEV).to(dtype) if "delta" in mode else None
        rows = torch.tensor([n - 1, 0, n // 2], device=DEV, dtype=torch.int32) if "rows" in mode else None
        out = torch.zeros(3 if rows is not None else n, hidden, device=DEV, dtype=dtype)
        return [x, w, 1e-5, 1.0, out], dict(delta=delta, rows=rows)

    torch.manual_seed(1)
    g, r = both("rms_norm", make, dtype)
    close(g[4], r[4], dtype, "out")
    close(g[0], r[0], torch.float32, "residual stream")
    if mode == "rows":
        assert torch.equal(g[0], r[0]), "x is left alone when rows are given"


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("nh,nkv,d,rot,ps,bias", [(3, 1, 40, 24, 8, True), (8, 1, 256, 256, 16, False),
                                                 (6, 6, 24, 24, 4, False), (4, 2, 64, 32, 32, True),
                                                 # pages that are no multiple of 4 tokens (the transposed values
                                                 # of a token are then 2 bytes at an odd multiple of 2 apart)
                                                 (4, 1, 32, 32, 1, False), (3, 3, 24, 24, 3, True),
                                                 (8, 2, 64, 64, 6, False), (2, 1, 256, 256, 10, False),
                                                 (5, 1, 20, 12, 7, True)])
def test_rope_and_cache_write(dtype, nh, nkv, d, rot, ps, bias):
    n = 29
    pages = max(12, -(-n // ps) + 3)
    torch.manual_seed(2)
    width = (nh + 2 * nkv) * d

    def make():
        qkv = torch.randn(n, width, device=DEV).to(dtype)
        b = torch.randn(width, device=DEV) * 0.1 if bias else None
        positions = torch.randint(0, 5000, (n,), device=DEV, dtype=torch.int32)
        positions[0] = 0
        inv_freq = (1.0 / (10000.0 ** (torch.arange(0, rot, 2, dtype=torch.float32) / rot))).to(DEV)
        slots = torch.randperm(pages * ps, device=DEV)[:n].to(torch.int32)
        cache = torch.full((pages, 2, nkv, ps * d), 7.0, device=DEV, dtype=dtype)
        return [qkv, b, positions, inv_freq, slots, cache], dict(num_heads=nh, num_kv_heads=nkv, head_dim=d, page_size=ps)

    torch.manual_seed(2)
    g, r = both("rope_and_cache_write", make, dtype)
    close(g[0], r[0], dtype, "rotated rows")
    # the cache holds exactly what the rows hold, and nothing else moved
    k_rows = g[0].view(n, nh + 2 * nkv, d)[:, nh:nh + nkv]
    v_rows = g[0].view(n, nh + 2 * nkv, d)[:, nh + nkv:]
    slots = g[4].long()
    kview = g[5][:, 0].view(pages, nkv, ps, d)
    vview = g[5][:, 1].view(pages, nkv, d, ps)
    assert torch.equal(kview[slots // ps, :, slots % ps, :], k_rows)
    assert torch.equal(vview[slots // ps, :, :, slots % ps], v_rows)
    untouched = torch.ones(pages * ps, dtype=torch.bool, device=DEV)
    untouched[slots] = False
    assert (kview.permute(0, 2, 1, 3).reshape(pages * ps, -1)[untouched] == 7.0).all()
    assert (vview.permute(0, 3, 1, 2).reshape(pages * ps, -1)[untouched] == 7.0).all()


@pytest.mark.parametrize("dtype", DTYPES)
def test_norm_and_rotation_add_stacks_of_partial_sums(dtype):
    torch.manual_seed(7)
    n, hidden = 6, 200
    x = torch.randn(n, hidden, device=DEV)
    w = torch.randn(hidden, device=DEV) * 0.1
    stack = torch.randn(3, n, hidden, device=DEV)
    out = torch.zeros(n, hidden, device=DEV, dtype=dtype)
    x_ref, out_ref = x.clone(), out.clone()
    ops.rms_norm(x, w, 1e-6, 1.0, out, delta=stack)
    ops.rms_norm(x_ref, w, 1e-6, 1.0, out_ref, delta=((stack[0] + stack[1]) + stack[2]))
    assert torch.equal(x, x_ref) and torch.equal(out, out_ref)
    rows = torch.tensor([4, 0], device=DEV, dtype=torch.int32)
    o2, o2_ref = torch.zeros(2, hidden, device=DEV, dtype=dtype), torch.zeros(2, hidden, device=DEV, dtype=dtype)
    ops.rms_norm(x, w, 1e-6, 1.0, o2, delta=stack, rows=rows)
    ops.rms_norm(x, w, 1e-6, 1.0, o2_ref, delta=((stack[0] + stack[1]) + stack[2]), rows=rows)
    assert torch.equal(o2, o2_ref)
    # rotation: the sum of the parts replaces the row
    nh, nkv, d, ps = 3, 1, 40, 8
    width = (nh + 2 * nkv) * d
    parts = torch.randn(4, n, width, device=DEV)
    summed = (((parts[0] + parts[1]) + parts[2]) + parts[3]).to(dtype)
    positions = torch.arange(n, device=DEV, dtype=torch.int32) * 3
    inv_freq = (1.0 / (10000.0 ** (torch.arange(0, 24, 2, dtype=torch.float32) / 24))).to(DEV)
    slots = torch.arange(n, device=DEV, dtype=torch.int32)
    kw = dict(num_heads=nh, num_kv_heads=nkv, head_dim=d, page_size=ps)
    for bias in (None, torch.randn(width, device=DEV) * 0.1):
        qkv = torch.full((n, width), 9.0, device=DEV, dtype=dtype)
        cache, cache_ref = (torch.zeros(2, 2, nkv, ps * d, device=DEV, dtype=dtype) for _ in range(2))
        ops.rope_and_cache_write(qkv, bias, positions, inv_freq, slots, cache, parts=parts, **kw)
        ref = summed.clone()
        if dtype == torch.float32:
            ops.rope_and_cache_write(ref, bias, positions, inv_freq, slots, cache_ref, **kw)
            assert torch.equal(qkv, ref) and torch.equal(cache, cache_ref)
        else:
            # the parts are added in float32 and rounded once, after the rotation
            with ops.use_backend(EmulatedKernels(precise=True)):
                ops.rope_and_cache_write(ref, bias, positions, inv_freq, slots, cache_ref, parts=parts, **kw)
            close(qkv, ref, dtype)
            close(cache, cache_ref, dtype)


def test_rope_position_zero_is_identity_and_no_cache():
    nh, nkv, d = 2, 1, 16
    qkv = torch.randn(3, (nh + 2 * nkv) * d, device=DEV)
    before = qkv.clone()
    inv_freq = (1.0 / (100.0 ** (torch.arange(0, d, 2, dtype=torch.float32) / d))).to(DEV)
    ops.rope_and_cache_write(qkv, None, torch.zeros(3, device=DEV, dtype=torch.int32), inv_freq, None, None,
                             num_heads=nh, num_kv_heads=nkv, head_dim=d, page_size=4)
    assert torch.equal(qkv, before)


def _attention_case(dtype, nh, nkv, d, ps, segs, window, seed=0, spike=False):
    """segs: list of (q_len, ctx_len).  Pages are handed out in a shuffled order."""
    g = torch.Generator(device="cpu").manual_seed(seed)
    n = sum(q for q, _ in segs)
    pages_needed = sum(-(-c // ps) for _, c in segs)
    pages = pages_needed + 5
    order = torch.randperm(pages, generator=g).tolist()
    max_pages = max(-(-c // ps) for _, c in segs)
    bt = torch.zeros(len(segs), max_pages, dtype=torch.int32)
    for s, (_, c) in enumerate(segs):
        for p in range(-(-c // ps)):
            bt[s, p] = order.pop()
    cache = torch.randn(pages, 2, nkv, ps * d, generator=g).to(dtype)
    qkv = torch.randn(n, (nh + 2 * nkv) * d, generator=g).to(dtype)
    if spike:
        # one far key that must dominate: scale a query and its key so that the score stands out
        qkv[:, :d] *= 4.0
    q_len = torch.tensor([q for q, _ in segs], dtype=torch.int32)
    ctx = torch.tensor([c for _, c in segs], dtype=torch.int32)
    q_start = torch.cumsum(q_len, 0, dtype=torch.int32) - q_len
    tok_seg = torch.repeat_interleave(torch.arange(len(segs), dtype=torch.int32), q_len.long())
    out = torch.zeros(n, nh * d, dtype=dtype)
    args = [t.to(DEV) for t in (qkv, cache, bt, tok_seg, q_start.to(torch.int32), q_len, ctx, out)]
    kwargs = dict(num_heads=nh, num_kv_heads=nkv, head_dim=d, page_size=ps, scale=1.0 / math.sqrt(d), window=window,
                  max_q_len=int(q_len.max()), max_ctx_len=int(ctx.max()))
    return args, kwargs


ATTENTION_SHAPES = [
    # the reference's own kernel test: 14 query heads, 2 kv heads, head 64, pages of 16
    # (tests/test_paged_attention_kernel.py:11-15,69-91), context lengths 1, 5, 16, 17, 33, 100
    (14, 2, 64, 16, [(1, 1), (1, 5), (1, 16), (1, 17), (1, 33), (1, 100)], 0),
    (8, 1, 256, 16, [(1, 300), (7, 7), (33, 90), (1, 1)], 0),
    (6, 6, 24, 8, [(5, 5), (16, 47), (1, 64), (2, 130)], 0),
    (4, 1, 32, 4, [(23, 23), (1, 9), (3, 40)], 0),
    (16, 16, 128, 32, [(1, 77), (40, 40)], 0),
    (6, 2, 20, 16, [(9, 30), (1, 200)], 0),
    (12, 1, 48, 16, [(1, 150), (20, 64)], 0),
    (4, 2, 64, 16, [(1, 100), (30, 70), (50, 50)], 17),
    # pages that are no multiple of 4 tokens: 1, 3, 6, 10, 7
    (4, 1, 32, 1, [(1, 37), (9, 9), (3, 140)], 0),
    (6, 3, 24, 3, [(1, 131), (20, 47), (2, 260)], 0),
    (8, 2, 64, 6, [(1, 300), (33, 90), (1, 1), (5, 129)], 0),
    (2, 1, 256, 10, [(1, 257), (40, 40)], 0),
    (6, 2, 40, 7, [(1, 200), (17, 64), (1, 128)], 50),
    # more than 16 query heads a key/value head: 17, 24, 32 and 40
    (17, 1, 64, 16, [(1, 300), (1, 5), (3, 40), (20, 20)], 0),
    (24, 1, 32, 8, [(1, 129), (2, 70), (1, 1)], 0),
    (32, 1, 128, 16, [(1, 700), (1, 128), (9, 200)], 0),
    (80, 2, 32, 4, [(1, 260), (1, 33), (5, 5)], 90),
]


def _with_plan(args, kwargs):
    """Adds the work-item plan the engine would make for these segments (None where the generic kernel runs)."""
    kwargs = dict(kwargs)
    kwargs["plan"] = ops.plan_paged_attention(
        args[5].cpu().numpy(), args[6].cpu().numpy(), num_heads=kwargs["num_heads"], num_kv_heads=kwargs["num_kv_heads"],
        head_dim=kwargs["head_dim"], page_size=kwargs["page_size"], window=kwargs["window"], dtype=args[0].dtype,
        device=args[0].device)
    return kwargs


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("nh,nkv,d,ps,segs,window", ATTENTION_SHAPES)
def test_paged_attention(dtype, nh, nkv, d, ps, segs, window):
    g, r = both("paged_attention", lambda: _attention_case(dtype, nh, nkv, d, ps, segs, window), dtype)
    close(g[7], r[7], dtype, "attention output")


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_context_bound_that_is_too_low_shows(dtype):
    """The general kernel sizes its grid by the caller's bound on the context lengths, which themselves are in
    device memory.  Tokens whose keys reach beyond the bound come out as NaN, never as attention over fewer keys;
    the other tokens are what they are with the right bound."""
    args, kwargs = _attention_case(dtype, 4, 2, 40, 8, [(3, 130), (2, 300), (1, 640)], 0)
    ops.paged_attention(*args, **kwargs)
    right = args[7].clone()
    assert torch.isfinite(right.float()).all()
    args[7].zero_()
    ops.paged_attention(*args, **dict(kwargs, max_ctx_len=256))        # chunks of 128 keys: positions 256.. are cut
    got = args[7].float()
    assert torch.equal(args[7][:3], right[:3])                          # positions 127..129
    assert torch.isnan(got[3:]).all()                                   # positions 298, 299 and 639


MFMA_SHAPES = ATTENTION_SHAPES + [
    (8, 1, 256, 16, [(1, 2048), (1, 700), (1, 257), (1, 256), (1, 255)], 0),      # decoded tokens, keys split over workgroups
    (8, 1, 256, 16, [(2048, 2048)], 0),                                           # a whole prompt
    (16, 16, 256, 16, [(1, 513), (70, 300)], 0),                                   # no grouping
    (6, 2, 96, 4, [(5, 5), (1, 300), (17, 64), (2, 40)], 0),                       # pages of 4: 8-byte value loads
    (8, 2, 64, 8, [(1, 600), (3, 100), (50, 50)], 33),                             # window
    (8, 2, 64, 16, [(1, 1000), (40, 500)], 300),                                   # window over several key chunks
    (10, 5, 160, 32, [(1, 90), (33, 33)], 0),
    (3, 1, 224, 16, [(1, 400), (6, 6), (7, 20)], 0),                               # group of 3: rows straddle tokens
    (4, 2, 64, 12, [(1, 300), (2, 77), (1, 5), (1, 128), (1, 129)], 0),            # pages that do not divide 128 keys
    (8, 2, 64, 20, [(1, 500), (3, 90), (1, 260)], 70),                             # the same with a window
    (8, 2, 64, 24, [(40, 300), (1, 100)], 0),          # prompt portions with pages of a multiple of 8 that is no power of two
    (4, 1, 128, 40, [(70, 70), (33, 200)], 60),
    (8, 1, 256, 32, [(100, 1000)], 0),                 # ... and of a power of two other than 16
    (4, 4, 128, 8, [(64, 64), (20, 500)], 100),
]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("nh,nkv,d,ps,segs,window", MFMA_SHAPES)
def test_paged_attention_matrix_cores(dtype, nh, nkv, d, ps, segs, window):
    """The kernels the engine uses for these sizes, with their plan of work items: in bfloat16 tiles of 16 rows for
    decoded tokens and blocks of 64 rows for prompts, in float32 tiles of 16 rows for everything."""
    _check_matrix_cores(nh, nkv, d, ps, segs, window, dtype)


def test_float32_matrix_cores_on_whole_prompts():
    """In float32 a prompt of 2,048 tokens of 8 heads on one key head runs as blocks of 64 rows with their keys staged
    once a block (the plan of the bfloat16 kernel), one of 512 tokens, whose 64 blocks would leave most of the device
    idle, as 256 tiles of 16 rows, each with the chunks of 128 keys its rows can see."""
    plan = _check_matrix_cores(8, 1, 256, 16, [(2048, 2048)], 0, torch.float32)
    assert plan.num_items == 0 and plan.num_prefill == 504
    plan = _check_matrix_cores(8, 1, 256, 16, [(512, 512)], 0, torch.float32)
    assert plan.num_prefill == 0 and plan.num_items == 640 and plan.num_reduce == 256 - 64


@pytest.mark.parametrize("nh,nkv,d,ps,segs,window,small_pieces", [
    (8, 1, 256, 16, [(512, 2560)], 0, False),          # a late portion of a long prompt: split as the engine splits it
    (8, 1, 256, 16, [(200, 900), (1, 70)], 0, True),
    (8, 2, 64, 8, [(40, 700), (1, 300), (70, 70)], 150, True),
    (6, 2, 96, 4, [(100, 400), (9, 500)], 0, True),
    (5, 5, 32, 12, [(130, 333)], 0, True),
])
def test_prompt_portions_whose_keys_are_split_over_workgroups(nh, nkv, d, ps, segs, window, small_pieces, monkeypatch):
    """Blocks of rows whose keys are cut into pieces, each piece a workgroup, combined by the reduce kernel."""
    from wllm_amd.kernels import attention_plan
    if small_pieces:       # pieces down to 128 keys, so that small cases are cut the way large ones are
        monkeypatch.setattr(attention_plan, "PREFILL_MIN_PIECE", 4)
    plan = _check_matrix_cores(nh, nkv, d, ps, segs, window)
    assert plan.num_prefill > 0 and plan.num_reduce > 0
    assert int((plan.prefill_items[:, 5] >= 0).sum()) > 0, "no block of rows was split"


def test_a_requests_attention_has_the_same_bits_alone_and_beside_a_long_prompt(monkeypatch):
    """With many tiles to combine the reduce runs as a kernel of 16-byte loads, with few as one thread
    per element; both add a row's pieces in the same order, so a request's output does not change by
    a bit when a long prompt joins the step."""
    from wllm_amd.kernels import attention_plan
    monkeypatch.setattr(attention_plan, "PREFILL_MIN_PIECE", 4)
    nh, nkv, d, ps = 8, 2, 64, 8
    dtype = torch.bfloat16
    args, kwargs = _attention_case(dtype, nh, nkv, d, ps, [(40, 700), (1, 600), (300, 900)], 0, seed=23)
    both_kw = _with_plan(args, kwargs)
    assert both_kw["plan"].num_reduce >= 64
    ops.paged_attention(*args, **both_kw)
    beside = args[7][:41].clone()
    # the first two requests alone: the same rows of qkv, the same pages
    alone = [args[0][:41].contiguous(), args[1], args[2][:2].contiguous(), args[3][:41].contiguous(),
             args[4][:2].contiguous(), args[5][:2].contiguous(), args[6][:2].contiguous(), torch.zeros_like(args[7][:41])]
    alone_kw = _with_plan(alone, dict(kwargs, max_q_len=40, max_ctx_len=700))
    assert 0 < alone_kw["plan"].num_reduce < 64
    ops.paged_attention(*alone, **alone_kw)
    assert torch.equal(alone[7], beside)


def _check_matrix_cores(nh, nkv, d, ps, segs, window, dtype=torch.bfloat16):
    args, kwargs = _attention_case(dtype, nh, nkv, d, ps, segs, window, seed=11)
    ref_args = [a.clone() for a in args]
    kw = _with_plan(args, kwargs)
    expect_plan = d % 32 == 0 and ps % 4 == 0
    assert (kw["plan"] is not None) == expect_plan
    # stale slots beyond a request's length hold NaN: they must not leak into the result
    cache, bt, ctx = args[1], args[2], args[6]
    kview = cache[:, 0].view(cache.shape[0], nkv, ps, d)
    vview = cache[:, 1].view(cache.shape[0], nkv, d, ps)
    for s_, (_, c) in enumerate(segs):
        if c % ps:
            last = int(bt[s_, (c - 1) // ps])
            kview[last, :, c % ps:, :] = float("nan")
            vview[last, :, :, c % ps:] = float("nan")
    ref_args[1] = cache.clone()
    ops.paged_attention(*args, **kw)
    torch.cuda.synchronize()
    with ops.use_backend(EmulatedKernels(precise=True)):
        ops.paged_attention(*ref_args, **kwargs)
    assert torch.isfinite(args[7].float()).all()
    close(args[7], ref_args[7], dtype, "attention output")
    return kw["plan"]


@pytest.mark.parametrize("dtype", DTYPES)
def test_paged_attention_finds_one_far_key(dtype):
    """One key among hundreds carries the whole weight: its value must come out."""
    nh, nkv, d, ps = 8, 1, 64, 16
    args, kwargs = _attention_case(dtype, nh, nkv, d, ps, [(1, 700)], 0, seed=3)
    qkv, cache, bt = args[0], args[1], args[2]
    far = 123
    page, off = int(bt[0, far // ps]), far % ps
    kview = cache[:, 0].view(cache.shape[0], nkv, ps, d)
    vview = cache[:, 1].view(cache.shape[0], nkv, d, ps)
    q = qkv[0, :d].float()
    kview[page, 0, off] = (q / q.norm() * 40.0).to(dtype)          # score far above the rest
    ops.paged_attention(*args, **kwargs)
    got = args[7][0, :d].float()
    assert torch.allclose(got, vview[page, 0, :, off].float(), atol=2e-2), "the far key's value is the output"


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("m,n,k", [(1, 100, 64), (7, 777, 250), (65, 130, 96), (128, 64, 2048), (3, 2560, 2048),
                                   (8, 2048, 16384), (17, 777, 96), (33, 1000, 128), (64, 4099, 2048), (49, 32768, 256),
                                   (200, 777, 64), (2, 16, 32), (16, 20, 1056), (16, 2048, 8192), (12, 100, 4128),
                                   (9, 3072, 24576), (11, 16500, 320),
                                   # more than 64 rows of an unsplit product (logits of many rows): groups of 64 rows in one launch
                                   (65, 24600, 64), (130, 25001, 96), (256, 26000, 128), (200, 50000, 32),
                                   # some hundred rows and a long K axis: the tiled product, its K axis in pieces
                                   (65, 2048, 16384), (300, 96, 8192), (513, 200, 8192), (1024, 48, 16384), (130, 3072, 24576)])
def test_linear(dtype, m, n, k):
    torch.manual_seed(4)
    for out_dtype in {dtype, torch.float32}:
        for tiled in (False, True):         # from the weight row by row, and from its tile-major copy
            def make():
                x = torch.randn(m, k, device=DEV).to(dtype)
                w = (torch.randn(n, k, device=DEV) / math.sqrt(k)).to(dtype)
                return [x, w, torch.zeros(m, n, device=DEV, dtype=out_dtype)], {"tiles": ops.tile_weight(w) if tiled else None}
            torch.manual_seed(4)
            g, r = both("linear", make, dtype)
            close(g[2], r[2], out_dtype, f"product to {out_dtype}, tiled {tiled}")


def test_float32_logits_of_a_large_vocabulary_at_few_rows():
    """7 to 64 rows, two segments of the K axis and 120,000 columns: more partial sums than the buffer
    of split sums holds at once, so the rows run in groups; every group's rows have the bits they have
    in a product of many rows (more than 64: the tiled kernel)."""
    torch.manual_seed(15)
    n, k = 120000, 3072
    x = torch.randn(100, k, device=DEV)
    w = torch.randn(n, k, device=DEV) / math.sqrt(k)
    many = torch.zeros(100, n, device=DEV)
    ops.linear(x, w, many)
    close(many, x.double() @ w.double().T, torch.float32, "product of many rows")
    for rows in (6, 7, 12, 16, 40):
        few = torch.full((rows, n), 9.0, device=DEV)
        ops.linear(x[3:3 + rows].contiguous(), w, few)
        assert torch.equal(few, many[3:3 + rows]), f"{rows} rows"


@pytest.mark.parametrize("n,k", [(777, 250), (2048, 2048), (100, 4128), (33, 64), (2560, 16384)])
def test_float32_product_of_few_rows_has_the_bits_of_the_product_of_many(n, k):
    """In float32 an element is the sum over k in ascending order whatever the number of rows, so a
    token's projection in a decode step equals, bit for bit, its projection inside a long prompt."""
    torch.manual_seed(14)
    x = torch.randn(100, k, device=DEV)
    w = torch.randn(n, k, device=DEV) / math.sqrt(k)
    many = torch.zeros(100, n, device=DEV)          # more than 64 rows: the tiled kernel
    ops.linear(x, w, many)
    close(many, x.double() @ w.double().T, torch.float32, "product of many rows")
    for rows in (1, 7, 16, 17, 32, 47, 64):         # the kernel that streams the weights, one to four tiles of rows
        for tiles in (None, ops.tile_weight(w)):
            few = torch.full((rows, n), 9.0, device=DEV)
            ops.linear(x[11:11 + rows].contiguous(), w, few, tiles=tiles)
            assert torch.equal(few, many[11:11 + rows]), f"{rows} rows, tile-major copy {tiles is not None}"


@pytest.mark.parametrize("m,n,k", [(8, 2048, 16384), (5, 2560, 2048), (16, 1000, 8192), (1, 777, 516), (3, 40000, 2048),
                                   (40, 2048, 4096), (64, 1000, 2048)])
def test_float32_linear_leaves_partial_sums_to_the_caller(m, n, k):
    """A float32 product of few rows and not many columns gives every segment of its K axis wavefronts
    of their own; the stack of their sums, added in order, has the bits of the product made whole."""
    torch.manual_seed(18)
    x = torch.randn(m, k, device=DEV)
    w = torch.randn(n, k, device=DEV) / math.sqrt(k)
    s = ops.linear_splits(m, n, k, torch.float32)
    whole = torch.zeros(m, n, device=DEV)
    ops.linear(x, w, whole)
    close(whole, x.double() @ w.double().T, torch.float32, "product")
    if n >= 16384:
        assert s == 1, "many columns are wavefronts enough"
        return
    assert s == -(-k // 512)
    stack = torch.full((s, m, n), 7.0, device=DEV)
    ops.linear(x, w, stack)
    total = stack[0].clone()
    for p in range(1, s):
        total += stack[p]
    assert torch.equal(total, whole)


def test_tile_weight_is_the_documented_permutation():
    torch.manual_seed(12)
    for n, k, halves in ((40, 96, 1), (16, 32, 1), (2 * 23, 64, 2), (777, 2048, 1)):
        w = torch.randn(n, k, device=DEV).to(torch.bfloat16)
        got = ops.tile_weight(w, halves)
        with ops.use_backend(EmulatedKernels(precise=True)):
            ref = ops.tile_weight(w, halves)
        assert torch.equal(got, ref)
    assert ops.tile_weight(torch.randn(8, 40, device=DEV).to(torch.bfloat16)) is None      # 40 keys: no tiles
    # float32: bands of 16 rows and chunks of 16 keys, both padded with zeros
    for n, k in ((40, 96), (16, 16), (23, 20), (777, 2048), (5, 4)):
        w = torch.randn(n, k, device=DEV)
        got = ops.tile_weight(w)
        with ops.use_backend(EmulatedKernels(precise=True)):
            ref = ops.tile_weight(w)
        assert got.shape == ref.shape == (ops.tiled_size(n, k, torch.float32),) and torch.equal(got, ref)
    assert ops.tile_weight(torch.randn(8, 42, device=DEV)) is None                         # 42 keys: no tiles


@pytest.mark.parametrize("m,n,k", [(8, 2048, 16384), (5, 2560, 2048), (64, 1000, 1024), (1, 777, 512), (16, 1000, 8192),
                                   (3, 3072, 24576), (40, 2048, 16384), (100, 2048, 16384), (512, 96, 8192), (1025, 96, 8192),
                                   (700, 2048, 16384), (1000, 3072, 24576)])
def test_linear_leaves_partial_sums_to_the_caller(m, n, k):
    torch.manual_seed(8)
    x = torch.randn(m, k, device=DEV).to(torch.bfloat16)
    w = (torch.randn(n, k, device=DEV) / math.sqrt(k)).to(torch.bfloat16)
    s = ops.linear_splits(m, n, k, torch.bfloat16)
    for tiles in (None, ops.tile_weight(w)):
        whole = torch.zeros(m, n, device=DEV)
        ops.linear(x, w, whole, tiles)
        if s == 1:
            with pytest.raises(ops.KernelShapeError):
                ops.linear(x, w, torch.zeros(2, m, n, device=DEV), tiles)
            continue
        stack = torch.full((s, m, n), 7.0, device=DEV)
        ops.linear(x, w, stack, tiles)
        total = stack[0].clone()
        for p in range(1, s):
            total += stack[p]
        assert torch.equal(total, whole), "the partial sums add up, in order, to what the kernel gives unsplit"
        close(whole, x.double() @ w.double().T, torch.float32, "product")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("act", ["gelu_tanh", "silu"])
@pytest.mark.parametrize("m,inter,k", [(8, 16384, 2048), (3, 250, 96), (64, 777, 128), (100, 384, 96), (17, 112, 80),
                                       (16, 1000, 4128), (1, 250, 96), (13, 2000, 3072), (16, 20, 32),
                                       # some hundred rows: the tiled product with the activation in its registers
                                       (65, 4000, 2048), (130, 250, 128), (256, 777, 320), (200, 64, 64)])
def test_gated_linear(dtype, act, m, inter, k):
    torch.manual_seed(9)

    for tiled in (False, True):
        def make():
            x = torch.randn(m, k, device=DEV).to(dtype)
            w = (torch.randn(2 * inter, k, device=DEV) / math.sqrt(k)).to(dtype)
            return ([x, w, torch.zeros(m, inter, device=DEV, dtype=dtype), act, torch.zeros(m, 2 * inter, device=DEV, dtype=dtype)],
                    {"tiles": ops.tile_weight(w, 2) if tiled else None})

        torch.manual_seed(9)
        g, r = both("gated_linear", make, dtype)
        close(g[2], r[2], dtype, f"tiled {tiled}")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("act", ["gelu_tanh", "silu"])
def test_gated_activation(dtype, act):
    torch.manual_seed(5)

    for inter in (250, 256, 1032):
        def make():
            gu = (torch.randn(13, 2 * inter, device=DEV) * 3).to(dtype)
            return [gu, torch.zeros(13, inter, device=DEV, dtype=dtype), act], {}

        torch.manual_seed(5)
        g, r = both("gated_activation", make, dtype)
        close(g[1], r[1], dtype)
        if act == "gelu_tanh":
            ref = torch.nn.functional.gelu(g[0][:, :inter].float(), approximate="tanh") * g[0][:, inter:].float()
            close(g[1], ref, dtype, "against the library's gelu")


def test_argmax_rows_lowest_index_among_equals():
    torch.manual_seed(6)
    logits = torch.randn(9, 777, device=DEV)
    logits[2, 500] = logits[2, 30] = 50.0
    logits[3] = 0.0
    logits[4, 776] = 60.0
    out = torch.zeros(9, device=DEV, dtype=torch.int32)
    ops.argmax_rows(logits, out)
    assert out.tolist() == logits.argmax(-1).tolist()
    assert out[2] == 30 and out[3] == 0 and out[4] == 776


def test_shape_errors_are_raised_on_the_host():
    x = torch.zeros(4, 64, device=DEV)
    with pytest.raises(ops.KernelShapeError):
        ops.rms_norm(x, torch.zeros(63, device=DEV), 1e-6, 1.0, torch.zeros(4, 64, device=DEV))
    with pytest.raises(ops.KernelShapeError):
        ops.linear(x, torch.zeros(10, 32, device=DEV), torch.zeros(4, 10, device=DEV))
    with pytest.raises(ops.KernelShapeError):
        ops.linear(x.to(torch.bfloat16), torch.zeros(10, 64, device=DEV), torch.zeros(4, 10, device=DEV))


def test_feed_tokens_writes_only_the_named_places():
    ids = torch.arange(10, dtype=torch.int32, device=DEV)
    dst = torch.tensor([3, -1, 7, 99, 5], dtype=torch.int32, device=DEV)
    src = torch.tensor([0, 1, 2, 0, 44], dtype=torch.int32, device=DEV)       # 99 and 44 are out of range: skipped
    source = torch.tensor([100, 200, 300], dtype=torch.int32, device=DEV)
    ops.feed_tokens(ids, dst, src, source)
    assert ids.tolist() == [0, 1, 2, 100, 4, 5, 6, 300, 8, 9]


@pytest.mark.parametrize("tiled", [False, True])
@pytest.mark.parametrize("m,k,nh,nkv,d,ps,with_bias,with_cache", [
    (8, 2048, 8, 1, 256, 16, False, True), (16, 96, 3, 1, 32, 4, True, True), (1, 320, 4, 2, 64, 8, False, True),
    (5, 4128, 2, 2, 96, 12, True, True), (3, 64, 5, 5, 128, 16, False, False),
    # 17 to 32 tokens: two tiles of 16
    (17, 2048, 8, 1, 256, 16, False, True), (29, 320, 4, 2, 64, 8, True, True), (32, 3072, 2, 2, 256, 16, False, True),
    (20, 96, 3, 1, 32, 4, True, False)])
def test_qkv_projection_rotation_and_cache_write_in_one_kernel(tiled, m, k, nh, nkv, d, ps, with_bias, with_cache):
    dtype = torch.bfloat16
    assert ops.qkv_rope_takes(m, dtype, k, d, d)
    assert not ops.qkv_rope_takes(33, dtype, k, d, d) and not ops.qkv_rope_takes(m, torch.float32, k, d, d)
    assert not ops.qkv_rope_takes(m, dtype, k, d, d // 2), "heads rotated in part take the two kernels"
    width = (nh + 2 * nkv) * d

    def make():
        g = torch.Generator(device="cpu").manual_seed(21)
        x = torch.randn(m, k, generator=g).to(dtype).to(DEV)
        w = (torch.randn(width, k, generator=g) / math.sqrt(k)).to(dtype).to(DEV)
        bias = (torch.randn(width, generator=g) * 0.3).to(DEV) if with_bias else None
        positions = torch.randint(0, 3000, (m,), generator=g, dtype=torch.int32).to(DEV)
        inv_freq = (1.0 / (10000.0 ** (torch.arange(0, d, 2, dtype=torch.float32) / d))).to(DEV)
        pages = m + 3
        slots = (torch.randperm(pages * ps, generator=g)[:m]).to(torch.int32).to(DEV) if with_cache else None
        cache = torch.zeros(pages, 2, nkv, ps * d, dtype=dtype, device=DEV) if with_cache else None
        qkv = torch.zeros(m, width, dtype=dtype, device=DEV)
        return [x, w, qkv, bias, positions, inv_freq, slots, cache], dict(
            num_heads=nh, num_kv_heads=nkv, head_dim=d, page_size=ps, tiles=ops.tile_weight(w) if tiled else None)

    g_, r_ = both("qkv_rope", make, dtype)
    close(g_[2], r_[2], dtype, "rotated queries, keys and values")
    if with_cache:
        close(g_[7], r_[7], dtype, "pages")
        assert (g_[7] != 0).sum() == (r_[7] != 0).sum(), "only the tokens' slots are written"


@pytest.mark.parametrize("tiled", [False, True])
@pytest.mark.parametrize("m,n,k", [(8, 2048, 2048), (8, 3072, 4096), (16, 96, 64), (1, 48, 4064), (5, 3072, 1056), (13, 16, 32)])
def test_product_into_the_residual_stream_with_sums_of_squares(tiled, m, n, k):
    dtype = torch.bfloat16
    assert ops.linear_residual_takes(m, dtype, n, k)
    assert not ops.linear_residual_takes(m, dtype, n, 16384), "a long K axis is left to the split product"
    assert not ops.linear_residual_takes(17, dtype, n, k) and not ops.linear_residual_takes(m, dtype, n + 8, k)

    def make():
        g = torch.Generator(device="cpu").manual_seed(31)
        x = torch.randn(m, k, generator=g).to(dtype).to(DEV)
        w = (torch.randn(n, k, generator=g) / math.sqrt(k)).to(dtype).to(DEV)
        residual = torch.randn(m, n, generator=g).to(DEV)
        sumsq = torch.full((m, n // 16), -1.0, device=DEV)
        return [x, w, residual, sumsq], {"tiles": ops.tile_weight(w) if tiled else None}

    g_, r_ = both("linear_residual", make, dtype)
    close(g_[2], r_[2], torch.float32, "residual")
    assert torch.allclose(g_[3].double(), (g_[2].double() ** 2).view(m, -1, 16).sum(-1), rtol=1e-5), "sums of squares of what was written"


@pytest.mark.parametrize("tiled", [False, True])
@pytest.mark.parametrize("act", ["gelu_tanh", "silu"])
@pytest.mark.parametrize("m,inter,k,offset", [(8, 16384, 2048, 1.0), (16, 250, 512, 0.0), (1, 777, 1024, 1.0), (11, 64, 3072, 1.0)])
def test_gated_product_with_the_norm_on_load(tiled, act, m, inter, k, offset):
    """The gated product reading the float32 residual stream and normalising it on the way, against
    rms_norm followed by the gated product."""
    dtype = torch.bfloat16
    assert ops.gated_linear_norm_takes(m, dtype, k)
    assert not ops.gated_linear_norm_takes(17, dtype, k) and not ops.gated_linear_norm_takes(m, dtype, k + 64)
    g = torch.Generator(device="cpu").manual_seed(41)
    residual = (torch.randn(m, k, generator=g) * 3).to(DEV)
    norm_w = (torch.randn(k, generator=g) * 0.2).to(DEV)
    w = (torch.randn(2 * inter, k, generator=g) / math.sqrt(k)).to(dtype).to(DEV)
    # the producer's sums: here per band of 16 columns, as `linear_residual` leaves them
    sumsq = (residual.double() ** 2).view(m, -1, 16).sum(-1).float()
    x = ops.NormOnLoad(residual, sumsq, norm_w, 1e-6, offset, dtype)
    tiles = ops.tile_weight(w, 2) if tiled else None
    out = torch.zeros(m, inter, dtype=dtype, device=DEV)
    ops.gated_linear(x, w, out, act, None, tiles)
    torch.cuda.synchronize()
    # the two kernels it replaces
    h = torch.zeros(m, k, dtype=dtype, device=DEV)
    ops.rms_norm(residual.clone(), norm_w, 1e-6, offset, h)
    two = torch.zeros(m, inter, dtype=dtype, device=DEV)
    ops.gated_linear(h, w, two, act, torch.zeros(m, 2 * inter, dtype=dtype, device=DEV), tiles)
    close(out, two, dtype, "against norm then product on the GPU")
    ref = torch.zeros(m, inter, dtype=dtype, device=DEV)
    with ops.use_backend(EmulatedKernels(precise=True)):
        ops.gated_linear(x, w, ref, act, None, tiles)
    close(out, ref, dtype, "against the emulation")


def test_a_key_has_one_rounding_more_in_a_step_of_many_rows():
    """Where queries and keys are rounded to bfloat16: once, after the rotation, in the fused projection of
    a decode step; twice in a step of many rows (the library's product rounds the projection, the rotation
    rounds again).  The same token's key and query, written by a step of 8 rows and by a step of 100, differ
    by that one rounding and no more: every element within one step of the bfloat16 grid at the row's size
    (2^-7 of the largest element), most of them equal."""
    torch.manual_seed(21)
    nh, nkv, d, ps, hidden = 4, 2, 64, 16, 256
    width = (nh + 2 * nkv) * d
    w = (torch.randn(width, hidden, device=DEV) / math.sqrt(hidden)).to(torch.bfloat16)
    x = torch.randn(100, hidden, device=DEV).to(torch.bfloat16)
    inv_freq = (1.0 / (10000.0 ** (torch.arange(0, d, 2, dtype=torch.float32) / d))).to(DEV)
    kw = dict(num_heads=nh, num_kv_heads=nkv, head_dim=d, page_size=ps)

    def run(rows):
        positions = torch.arange(rows, device=DEV, dtype=torch.int32) + 37
        slots = torch.arange(rows, device=DEV, dtype=torch.int32)
        qkv = torch.zeros(rows, width, device=DEV, dtype=torch.bfloat16)
        cache = torch.zeros(8, 2, nkv, ps * d, device=DEV, dtype=torch.bfloat16)
        if ops.qkv_rope_takes(rows, torch.bfloat16, hidden, d, d):
            ops.qkv_rope(x[:rows].contiguous(), w, qkv, None, positions, inv_freq, slots, cache, **kw)
            path = "fused"
        else:
            ops.linear(x[:rows].contiguous(), w, qkv)
            ops.rope_and_cache_write(qkv, None, positions, inv_freq, slots, cache, **kw)
            path = "two kernels"
        return qkv, cache, path

    few, cache_few, path_few = run(8)
    many, cache_many, path_many = run(100)
    assert (path_few, path_many) == ("fused", "two kernels")
    # what the cache holds is what the rows hold, in both
    for qkv, cache, rows in ((few, cache_few, 8), (many, cache_many, 100)):
        keys = cache[:, 0].view(8, nkv, ps, d).permute(0, 2, 1, 3).reshape(8 * ps, nkv * d)[:rows]
        assert torch.equal(keys, qkv[:, nh * d:(nh + nkv) * d])
    a, b = few.float(), many[:8].float()
    grid = a.abs().amax(-1, keepdim=True) * 2.0 ** -7
    assert ((a - b).abs() <= grid).all(), "more than one rounding apart"
    assert (a == b).float().mean() > 0.5
