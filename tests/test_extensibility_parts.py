"""That every kind of part can be replaced without a change to the framework's files.

A second toy architecture, defined here: a feed-forward that routes each token to one of several
experts (router logits in float32), a position encoding with frequencies of its own (a table the
framework's attention rotates by), and a norm without a mean (so it offers no recipe for a kernel to
apply while reading: the stream falls back to running it).  They are registered next to the
framework's parts, mixed layer by layer with the framework's own, loaded from a folder written by
the random-weights mode, stepped in portions and mixed batches, and compared with a plain
whole-sequence computation written here.  The toy is no model of anyone's.
"""
import os
from dataclasses import dataclass

import pytest
import torch

from helpers import compare_with_plain, max_live_tokens, random_ids, replay_and_collect, trace_mixed, trace_portions, trace_whole
from kernel_emulation import EmulatedKernels
from plain import gemma_plain as P
from wllm_amd.config import register_architecture
from wllm_amd.engine import ModelRunner
from wllm_amd.engine.replay import TraceReplayer, pages_for_max_tokens
from wllm_amd.kernels import ops
from wllm_amd.parts import load_model, register_feed_forward, register_norm, register_position
from wllm_amd.parts.specs import (AttentionSpec, BlockSpec, EmbeddingSpec, FeedForwardSpec, GatedMLPSpec, HeadSpec, ModelPlan,
                                  NormSpec, PositionSpec, ScheduleEntry)
from wllm_amd.weights import ExpectedTensor
from wllm_amd.weights.random_init import write_random_model

H, E, I, HEADS, KV, D = 48, 3, 40, 3, 1, 32


# ---- a feed-forward with routing: each token goes to the expert whose router logit is largest ----
@dataclass(frozen=True)
class RoutedSpec(FeedForwardSpec):
    kind: str = "toy_routed"
    hidden_size: int = 0
    inner_size: int = 0
    num_experts: int = 0
    prefix: str = ""


@register_feed_forward("toy_routed", replace=True)
class RoutedFeedForward:
    def __init__(self, spec):
        self.spec = spec

    def expected_tensors(self):
        s, out = self.spec, {}
        out[s.prefix + "router"] = ExpectedTensor((s.num_experts, s.hidden_size))
        for e in range(s.num_experts):
            out[f"{s.prefix}e{e}.in"] = ExpectedTensor((s.inner_size, s.hidden_size))
            out[f"{s.prefix}e{e}.out"] = ExpectedTensor((s.hidden_size, s.inner_size))
        return out

    def load(self, fetch):
        s = self.spec
        self.router = fetch.to_device(fetch.matrix(s.prefix + "router")).float()       # logits in float32
        self.w_in = [fetch.to_device(fetch.matrix(f"{s.prefix}e{e}.in")) for e in range(s.num_experts)]
        self.w_out = [fetch.to_device(fetch.matrix(f"{s.prefix}e{e}.out")) for e in range(s.num_experts)]

    def forward(self, ctx, h):
        s = self.spec
        choice = (h.float() @ self.router.T).argmax(-1)
        y = torch.zeros_like(h)
        for e in range(s.num_experts):
            rows = (choice == e).nonzero()[:, 0]
            if rows.numel() == 0:
                continue
            mid = torch.empty(rows.numel(), s.inner_size, dtype=h.dtype, device=h.device)
            ops.linear(h[rows].contiguous(), self.w_in[e], mid)
            mid = torch.relu(mid.float()).to(h.dtype)
            out = torch.empty(rows.numel(), s.hidden_size, dtype=h.dtype, device=h.device)
            ops.linear(mid, self.w_out[e], out)
            y[rows] = out
        return y


# ---- a position encoding: the framework's rotation with another table of frequencies ----------
@register_position("toy_linear", replace=True)
class LinearFrequencies:
    """inv_freq[j] = 1 / (theta * (j + 1)): the attention part rotates by whatever table it is given."""

    def __init__(self, spec):
        self.spec = spec
        self.inv_freq = None

    def prepare(self, device):
        j = torch.arange(self.spec.rotary_dim // 2, dtype=torch.float32)
        self.inv_freq = (1.0 / (self.spec.theta * (j + 1.0))).to(device)


# ---- a norm: y = x * w / (max |x| + eps); no `on_load`, so no kernel can fold it into its read ----
@register_norm("toy_max", replace=True)
class MaxNorm:
    def __init__(self, spec):
        self.spec = spec

    def expected_tensors(self):
        return {self.spec.weight: ExpectedTensor((self.spec.size,), role="vector", init="norm")}

    def load(self, fetch):
        self.weight = fetch.to_device(fetch.vector(self.spec.weight))

    def forward(self, x, out, delta=None, rows=None):
        v = x
        if delta is not None:
            d = delta.float() if delta.dim() == 2 else delta.sum(0)
            v = x + d
            if rows is None:
                x.copy_(v)
        if rows is not None:
            v = v[rows.long()]
        out.copy_((v / (v.abs().amax(-1, keepdim=True) + self.spec.eps) * self.weight).to(out.dtype))
        return out


@dataclass(frozen=True)
class Toy2Config:
    vocab_size: int

    @classmethod
    def from_dict(cls, raw):
        return cls(raw["vocab_size"])


def toy2_plan(cfg):
    rms = lambda name: NormSpec(size=H, eps=1e-5, weight=name, weight_offset=1.0)
    mx = lambda name: NormSpec(size=H, eps=1e-3, weight=name, kind="toy_max")
    attn = lambda p, pos: AttentionSpec(hidden_size=H, num_heads=HEADS, num_kv_heads=KV, head_dim=D, scale=D ** -0.5, position=pos,
                                        q_weight=p + "q", k_weight=p + "k", v_weight=p + "v", o_weight=p + "o")
    layers = (
        BlockSpec(mixer=attn("a.", PositionSpec(kind="toy_linear", rotary_dim=D, theta=3.0)),
                  feed_forward=RoutedSpec(hidden_size=H, inner_size=I, num_experts=E, prefix="a.ffn."),
                  mixer_norm=mx("a.n1"), feed_forward_norm=rms("a.n2")),
        BlockSpec(mixer=attn("b.", PositionSpec(kind="rope", rotary_dim=D, theta=50.0)),
                  feed_forward=GatedMLPSpec(hidden_size=H, intermediate_size=64, activation="gelu_tanh", gate_weight="b.gate",
                                            up_weight="b.up", down_weight="b.down"),
                  mixer_norm=rms("b.n1"), feed_forward_norm=mx("b.n2")),
    )
    return ModelPlan(embedding=EmbeddingSpec(cfg.vocab_size, H, "emb"), layers=layers,
                     schedule=(ScheduleEntry(0), ScheduleEntry(1), ScheduleEntry(0)),
                     final_norm=rms("final"), head=HeadSpec(cfg.vocab_size, H, "head"), max_positions=200)


register_architecture("ToyRoutedForCausalLM", Toy2Config.from_dict, toy2_plan, replace=True)
RAW = {"architectures": ["ToyRoutedForCausalLM"], "vocab_size": 83}


# ---- the plain computation ------------------------------------------------------------------
def plain_toy2(W, ids):
    T = len(ids)
    x = W["emb"][torch.as_tensor(ids)]
    rms = lambda v, w: v * torch.rsqrt(v.pow(2).mean(-1, keepdim=True) + 1e-5) * (1.0 + w)
    mx = lambda v, w: v / (v.abs().amax(-1, keepdim=True) + 1e-3) * w

    def attention(h, p, inv_freq):
        q = (h @ W[p + "q"].T).view(T, HEADS, D)
        k = (h @ W[p + "k"].T).view(T, KV, D)
        v = (h @ W[p + "v"].T).view(T, KV, D)
        ang = torch.arange(T, dtype=torch.float32)[:, None] * inv_freq[None, :]
        cos, sin = torch.cat([ang.cos(), ang.cos()], -1).to(h.dtype), torch.cat([ang.sin(), ang.sin()], -1).to(h.dtype)
        q, k = P.apply_rope(q, cos, sin), P.apply_rope(k, cos, sin)
        k, v = k.repeat_interleave(HEADS // KV, 1), v.repeat_interleave(HEADS // KV, 1)
        scores = torch.einsum("qhd,khd->hqk", q, k) * D ** -0.5
        i = torch.arange(T)
        probs = torch.softmax(scores.masked_fill(~(i[None, :] <= i[:, None])[None], float("-inf")), -1)
        return torch.einsum("hqk,khd->qhd", probs, v).reshape(T, HEADS * D) @ W[p + "o"].T

    j = torch.arange(D // 2, dtype=torch.float32)
    linear_freq = 1.0 / (3.0 * (j + 1.0))
    rope_freq = 1.0 / (50.0 ** (torch.arange(0, D, 2, dtype=torch.float32) / D))

    def layer_a(x):
        x = x + attention(mx(x, W["a.n1"]), "a.", linear_freq)
        h = rms(x, W["a.n2"])
        choice = (h.float() @ W["a.ffn.router"].float().T).argmax(-1)
        y = torch.stack([torch.relu(h[t] @ W[f"a.ffn.e{int(choice[t])}.in"].T) @ W[f"a.ffn.e{int(choice[t])}.out"].T
                         for t in range(T)])
        return x + y

    def layer_b(x):
        x = x + attention(rms(x, W["b.n1"]), "b.", rope_freq)
        h = mx(x, W["b.n2"])
        return x + P.geglu_mlp(h, W["b.gate"], W["b.up"], W["b.down"])

    x = layer_a(layer_b(layer_a(x)))
    return rms(x, W["final"]) @ W["head"].T


@pytest.fixture(scope="module")
def toy2_folder(tmp_path_factory):
    from wllm_amd.parts import build_model
    folder = str(tmp_path_factory.mktemp("toy2"))
    write_random_model(folder, RAW, build_model(RAW).expected_tensors(), seed=9, std=0.2, norm_std=0.3)
    # the max-norm's weights multiply directly: move them away from zero
    from wllm_amd.weights import Checkpoint, write_safetensors
    ck = Checkpoint(folder)
    tensors = {n: ck.tensor(n) for n in ck.names()}
    ck.close()
    for n in ("a.n1", "b.n2"):
        tensors[n] = (tensors[n].float() + 1.5).to(torch.bfloat16)
    write_safetensors(os.path.join(folder, "model.safetensors"), tensors)
    return folder


def check_toy2(folder, device):
    model = load_model(folder, "float32", device)
    W = P.read_weights(folder, torch.float32)
    requests = {f"r{i}": random_ids(50 + i, n, 83) for i, n in enumerate([33, 47, 25, 58])}
    plain = {rid: plain_toy2(W, t) for rid, t in requests.items()}
    # every expert is used somewhere, or the routing is not tested
    h_all = torch.cat([W["emb"][torch.as_tensor(t)] for t in requests.values()])
    assert len(set((h_all @ W["a.ffn.router"].T).argmax(-1).tolist())) == E
    for family in (trace_whole, trace_portions, trace_mixed):
        trace = family(requests)
        runner = ModelRunner.create(model, num_pages=pages_for_max_tokens(max_live_tokens(trace), 4), page_size=4,
                                    max_requests=4, poison_freed_pages=True)
        got = replay_and_collect(TraceReplayer(runner), trace)
        compare_with_plain(got, plain, atol=5e-5, rtol=2e-4)
        runner.cache.check()


def test_routed_feed_forward_other_positions_and_norm_on_the_cpu(toy2_folder):
    with ops.use_backend(EmulatedKernels()):
        check_toy2(toy2_folder, "cpu")


@pytest.mark.gpu
def test_routed_feed_forward_other_positions_and_norm_on_the_gpu(toy2_folder):
    check_toy2(toy2_folder, "cuda")


@pytest.mark.gpu
def test_the_toy_parts_run_in_bfloat16_decode_steps_beside_the_fused_kernels(toy2_folder):
    """bfloat16, few rows: the framework's parts take their short ways (fused projection, product
    into the residual stream), the toy norm has no recipe to hand on, and the step still runs; the
    greedy continuation agrees with the float32 run up to near ties."""
    outs = {}
    for dtype in ("float32", "bfloat16"):
        model = load_model(toy2_folder, dtype, "cuda")
        runner = ModelRunner.create(model, num_pages=64, page_size=4, max_requests=2)
        from wllm_amd.engine import Request, Scheduler
        s = Scheduler(runner)
        r = Request("r", random_ids(3, 21, 83), 12)
        s.add_request(r)
        s.run_to_completion()
        runner.cache.check()
        outs[dtype] = r.output_token_ids
    same = sum(a == b for a, b in zip(outs["float32"], outs["bfloat16"]))
    assert same >= 6, f"bfloat16 continuation {outs['bfloat16']} strays early from float32 {outs['float32']}"
