"""Each part alone against the plain implementation's function for it: norm, attention with its
rotation (whole sequences and cut into portions), feed-forward, block, embedding and head."""
import math
from types import SimpleNamespace

import pytest
import torch

from plain import gemma_plain as P
from wllm_amd.cache import CacheManager
from wllm_amd.engine import ModelRunner, StepEntry
from wllm_amd.parts import build_block, build_feed_forward, build_mixer, build_norm
from wllm_amd.parts.blocks import ResidualStream
from wllm_amd.parts.specs import AttentionSpec, BlockSpec, GatedMLPSpec, NormSpec, PositionSpec, ScheduleEntry

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda")


class DictFetcher:
    """Hands a part its tensors from a dict, as the checkpoint fetcher would."""

    def __init__(self, tensors, dtype):
        self.tensors, self.dtype, self.device = tensors, dtype, DEV

    def has(self, name):
        return name in self.tensors

    def matrix(self, name):
        return self.tensors[name].to(self.dtype)

    def vector(self, name):
        return self.tensors[name].to(torch.float32)

    def to_device(self, t):
        return t.contiguous().to(DEV)


def context_for(part_needs, dtype, segments, page_size=4, hidden=1, vocab=10):
    """A step context for one schedule entry: `segments` = [(request, first position, tokens)]."""
    model = SimpleNamespace(dtype=dtype, device=DEV,
                            plan=SimpleNamespace(schedule=(ScheduleEntry(0),), max_positions=4096,
                                                 embedding=SimpleNamespace(vocab_size=vocab)))
    return model


def settle(y, ctx=None):
    """A part's contribution may be a product still to be made, or a stack of partial sums that the
    next norm would add."""
    if hasattr(y, "make"):
        y = y.make(ctx)
    if y.dim() == 3:
        total = y[0].clone()
        for p in range(1, y.shape[0]):
            total += y[p]
        return total
    return y


def rand(*shape, scale=1.0, dtype=torch.float32):
    return (torch.randn(*shape) * scale).to(torch.bfloat16).to(dtype)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("hidden,eps,offset", [(96, 1e-5, 1.0), (200, 1e-6, 0.0)])
def test_norm_part(dtype, hidden, eps, offset):
    torch.manual_seed(0)
    w = rand(hidden, scale=0.2)
    norm = build_norm(NormSpec(size=hidden, eps=eps, weight="w", weight_offset=offset))
    assert list(norm.expected_tensors()) == ["w"]
    norm.load(DictFetcher({"w": w}, dtype))
    x = torch.randn(7, hidden)
    out = torch.empty(7, hidden, dtype=dtype, device=DEV)
    norm.forward(x.to(DEV), out)
    ref = P.rms_norm_one_plus_w(x.double(), w.double() - (1.0 - offset), eps)
    tol = 1e-5 if dtype == torch.float32 else 1e-2
    assert torch.allclose(out.double().cpu(), ref, atol=tol, rtol=tol)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("nh,nkv,d,hidden,theta,ps", [(4, 1, 32, 64, 10000.0, 4), (6, 6, 24, 96, 500.0, 8), (8, 2, 64, 48, 1e6, 16)])
def test_attention_part_whole_and_in_portions(dtype, nh, nkv, d, hidden, theta, ps):
    """The mixer alone, with pages of its own: a sequence fed whole, and the same sequence fed in
    portions beside another request, against the plain attention block."""
    torch.manual_seed(1)
    names = {k: k for k in ("q", "k", "v", "o")}
    spec = AttentionSpec(hidden_size=hidden, num_heads=nh, num_kv_heads=nkv, head_dim=d, scale=1 / math.sqrt(d),
                         position=PositionSpec(kind="rope", rotary_dim=d, theta=theta),
                         q_weight="q", k_weight="k", v_weight="v", o_weight="o")
    mixer = build_mixer(spec)
    s = 1 / math.sqrt(hidden)
    W = {"q": rand(nh * d, hidden, scale=s), "k": rand(nkv * d, hidden, scale=s), "v": rand(nkv * d, hidden, scale=s),
         "o": rand(hidden, nh * d, scale=1 / math.sqrt(nh * d))}
    mixer.load(DictFetcher(W, dtype))
    T = 37
    h = {"a": rand(T, hidden), "b": rand(20, hidden)}
    cfg = dict(num_attention_heads=nh, num_key_value_heads=nkv, head_dim=d, attention_bias=False)
    plain_w = {f"x.{k}_proj.weight": v.double() for k, v in W.items()}
    ref = {}
    for rid, x in h.items():
        cos, sin = P.rope_cos_sin(torch.arange(x.shape[0]), d, theta, torch.float64)
        ref[rid] = P.attention_block(x.double(), plain_w, "x.", cfg, cos, sin)

    model = SimpleNamespace(dtype=dtype, device=DEV, plan=SimpleNamespace(
        schedule=(ScheduleEntry(0),), max_positions=4096, embedding=SimpleNamespace(vocab_size=10)))
    tol = 2e-5 if dtype == torch.float32 else 2e-2

    def run(steps):
        cache = CacheManager({0: mixer.cache_need()}, ps, 24, 4, dtype, DEV, poison_freed_pages=True)
        runner = ModelRunner(model, cache)
        got = {rid: [] for rid in h}
        for step in steps:
            entries = []
            for rid, a, b in step:
                if not cache.is_open(rid):
                    cache.open(rid)
                entries.append(StepEntry(rid, [0] * (b - a), []))
            ctx = runner.prepare(entries)
            x = torch.cat([h[rid][a:b] for rid, a, b in step]).to(dtype).to(DEV)
            y = settle(mixer.forward(ctx, 0, x), ctx)
            runner.commit(entries)
            o = 0
            for rid, a, b in step:
                got[rid].append(y[o:o + b - a].double().cpu())
                o += b - a
        return {rid: torch.cat(v) for rid, v in got.items()}

    whole = run([[("a", 0, T)], [("b", 0, 20)]])
    cut = run([[("a", 0, 5)], [("a", 5, 7), ("b", 0, 9)], [("b", 9, 10), ("a", 7, 30)], [("a", 30, 31), ("b", 10, 20)],
               [("a", 31, T)]])
    for got in (whole, cut):
        for rid in h:
            assert torch.allclose(got[rid], ref[rid], atol=tol, rtol=tol), f"request {rid}"


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_feed_forward_part(dtype):
    torch.manual_seed(2)
    hidden, inter = 80, 112
    ffn = build_feed_forward(GatedMLPSpec(hidden_size=hidden, intermediate_size=inter, activation="gelu_tanh",
                                          gate_weight="g", up_weight="u", down_weight="d"))
    # weights of the usual size, 1/sqrt(fan-in), so that outputs are O(1) and an absolute bound means something
    W = {"g": rand(inter, hidden, scale=hidden ** -0.5), "u": rand(inter, hidden, scale=hidden ** -0.5),
         "d": rand(hidden, inter, scale=inter ** -0.5)}
    ffn.load(DictFetcher(W, dtype))
    h = rand(9, hidden)
    model = SimpleNamespace(dtype=dtype, device=DEV, plan=SimpleNamespace(
        schedule=(), max_positions=64, embedding=SimpleNamespace(vocab_size=10)))
    runner = ModelRunner(model, CacheManager({}, 4, 4, 2, dtype, DEV))
    runner.cache.open("r")
    ctx = runner.prepare([StepEntry("r", [0] * 9, [])])
    y = settle(ffn.forward(ctx, h.to(dtype).to(DEV)), ctx)
    ref = P.geglu_mlp(h.double(), W["g"].double(), W["u"].double(), W["d"].double())
    tol = 1e-5 if dtype == torch.float32 else 2e-2
    assert torch.allclose(y.double().cpu(), ref, atol=tol, rtol=tol)


@pytest.mark.parametrize("T", [19, 7])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_block_and_whole_model_parts(model_folders, dtype, T):
    """One pre-norm block of configuration B against the plain decoder layer (19 tokens: the
    general way through the norm kernels; 7 tokens in bfloat16: the attention output is added to
    the stream by its product kernel and the feed-forward applies its norm while it reads);
    embedding and head of the loaded model against the plain functions."""
    from wllm_amd.kernels import ops
    from wllm_amd.parts import load_model
    folder = model_folders["B"]
    cfg = P.read_config(folder)
    W = P.read_weights(folder, torch.float64)
    model = load_model(folder, dtype, "cuda")
    x = rand(T, cfg["hidden_size"])
    runner = ModelRunner.create(model, num_pages=8, page_size=8, max_requests=2)
    runner.open("r")
    entries = [StepEntry("r", [0] * T, [])]
    ctx = runner.prepare(entries)
    stream = ResidualStream(x.to(DEV).clone())
    model.blocks[1].forward(ctx, 1, stream)
    out = stream.x.double().cpu()
    if stream.pending is not None:          # else both contributions went straight into the stream
        out = out + settle(stream.pending).double().cpu()
    cos, sin = P.rope_cos_sin(torch.arange(T), cfg["head_dim"], cfg["rope_theta"], torch.float64)
    ref = P.decoder_layer(x.double(), W, 1, cfg, cos, sin)
    tol = 2e-5 if dtype == torch.float32 else 3e-2
    assert torch.allclose(out, ref, atol=tol, rtol=tol)
    # embedding: the factor is sqrt(hidden) held in the model's dtype
    ids = torch.tensor([0, 5, 776], dtype=torch.int32, device=DEV)
    e = torch.empty(3, cfg["hidden_size"], device=DEV)
    ops.embed_lookup(ids, model.embed_table, model.embed_scale, e)
    ref_e = P.embed(ids.cpu().long(), W["model.embed_tokens.weight"], cfg["hidden_size"],
                    torch.bfloat16 if dtype == torch.bfloat16 else None)
    assert torch.allclose(e.double().cpu(), ref_e, atol=1e-6, rtol=1e-6)
    assert model.head_weight is model.embed_table, "tied: the head is the table itself, unscaled"
