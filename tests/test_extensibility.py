"""That another architecture can be added without a change to the framework's files.

A toy architecture is defined here, in the test: a mixer with a state of its own (a decaying
sum of its inputs, one vector per request), registered next to the framework's attention; a
schedule that runs a layer twice and lets a run read another run's cache.  It is registered,
built from a config.json, loaded from a folder written by the random-weights mode, and stepped
in portions and mixed batches; the results are compared with a plain whole-sequence computation
written here.  The toy is no model of anyone's.
"""
import json
import math
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
from wllm_amd.parts import load_model, register_mixer
from wllm_amd.parts.specs import (AttentionSpec, BlockSpec, EmbeddingSpec, GatedMLPSpec, HeadSpec, MixerSpec, ModelPlan,
                                  NormSpec, PositionSpec, ScheduleEntry)
from wllm_amd.weights import ExpectedTensor
from wllm_amd.weights.random_init import write_random_model


# ---- the toy mixer: s_t = decay * s_{t-1} + h_t ; y_t = s_t @ W^T -------------------------------
@dataclass(frozen=True)
class DecaySpec(MixerSpec):
    kind: str = "toy_decay"
    hidden_size: int = 0
    decay: float = 0.5
    weight: str = ""


@register_mixer("toy_decay", replace=True)
class DecayMixer:
    def __init__(self, spec):
        self.spec = spec
        self.w = None

    def expected_tensors(self):
        return {self.spec.weight: ExpectedTensor((self.spec.hidden_size, self.spec.hidden_size))}

    def load(self, fetch):
        self.w = fetch.to_device(fetch.matrix(self.spec.weight))

    def cache_need(self):
        return None                       # no pages

    def state_shape(self):
        return (self.spec.hidden_size,)   # one vector per request, in a state slot

    def forward(self, ctx, entry, h):
        state = ctx.state(entry)
        mixed = torch.empty(h.shape, dtype=torch.float32, device=h.device)
        for s in range(ctx.num_segments):
            slot = int(ctx.host_state_slots[s])
            q0, ql = int(ctx.host_q_start[s]), int(ctx.host_q_len[s])
            cur = state[slot]
            for i in range(q0, q0 + ql):
                cur = self.spec.decay * cur + h[i].float()
                mixed[i] = cur
            state[slot] = cur
        y = ctx.buffer("toy_out", tuple(h.shape), h.dtype)
        ops.linear(mixed.to(h.dtype), self.w, y)
        return y


@dataclass(frozen=True)
class ToyConfig:
    vocab_size: int
    hidden_size: int
    decay: float
    window: int

    @classmethod
    def from_dict(cls, raw):
        return cls(raw["vocab_size"], raw["hidden_size"], raw["decay"], raw["window"])


def toy_plan(cfg: ToyConfig) -> ModelPlan:
    h = cfg.hidden_size
    norm = lambda name: NormSpec(size=h, eps=1e-5, weight=name, weight_offset=0.0)
    ffn = lambda p: GatedMLPSpec(hidden_size=h, intermediate_size=2 * h, activation="silu", gate_weight=p + "gate",
                                 up_weight=p + "up", down_weight=p + "down")
    attn = lambda p, window: AttentionSpec(
        hidden_size=h, num_heads=4, num_kv_heads=2, head_dim=8, scale=0.25, window=window,
        position=PositionSpec(kind="rope", rotary_dim=4, theta=100.0),      # partial rotation
        q_weight=p + "q", k_weight=p + "k", v_weight=p + "v", o_weight=p + "o")
    layers = (
        BlockSpec(mixer=attn("l0.", None), feed_forward=ffn("l0."), mixer_norm=norm("l0.n1"), feed_forward_norm=norm("l0.n2")),
        BlockSpec(mixer=DecaySpec(hidden_size=h, decay=cfg.decay, weight="l1.decay_w"), feed_forward=ffn("l1."),
                  mixer_norm=norm("l1.n1"), feed_forward_norm=norm("l1.n2")),
        BlockSpec(mixer=attn("l2.", cfg.window), feed_forward=ffn("l2."), mixer_norm=norm("l2.n1"), feed_forward_norm=norm("l2.n2")),
    )
    # layer 0 twice (each run with a cache of its own), the toy mixer twice (each run with a state
    # of its own), a windowed layer, and a last run of layer 0 that reads the first run's cache
    schedule = (ScheduleEntry(0), ScheduleEntry(1), ScheduleEntry(2), ScheduleEntry(0), ScheduleEntry(1),
                ScheduleEntry(0, reads_cache_of=0))
    return ModelPlan(embedding=EmbeddingSpec(cfg.vocab_size, h, "emb", scale=1.0), layers=layers, schedule=schedule,
                     final_norm=norm("final"), head=HeadSpec(cfg.vocab_size, h, "head"), max_positions=256)


register_architecture("ToyDecayForCausalLM", ToyConfig.from_dict, toy_plan, replace=True)
RAW = {"architectures": ["ToyDecayForCausalLM"], "vocab_size": 97, "hidden_size": 32, "decay": 0.7, "window": 11}


# ---- its plain computation: whole sequence, no cache --------------------------------------------
def plain_norm(x, w):
    return x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + 1e-5) * w


def plain_attention(h, W, p, window, kv_from=None):
    T = h.shape[0]
    q = (h @ W[p + "q"].T).view(T, 4, 8)
    k = (h @ W[p + "k"].T).view(T, 2, 8)
    v = (h @ W[p + "v"].T).view(T, 2, 8)
    cos, sin = P.rope_cos_sin(torch.arange(T), 4, 100.0, h.dtype)

    def rot(x):     # only the first 4 elements of a head turn
        return torch.cat([P.apply_rope(x[..., :4], cos, sin), x[..., 4:]], -1)

    q, k = rot(q), rot(k)
    mine = (k, v)
    if kv_from is not None:
        k, v = kv_from
    k, v = k.repeat_interleave(2, 1), v.repeat_interleave(2, 1)
    scores = torch.einsum("qhd,khd->hqk", q, k) * 0.25
    i = torch.arange(T)
    ok = i[None, :] <= i[:, None]
    if window:
        ok &= i[None, :] > i[:, None] - window
    probs = torch.softmax(scores.masked_fill(~ok[None], float("-inf")), -1)
    return torch.einsum("hqk,khd->qhd", probs, v).reshape(T, 32) @ W[p + "o"].T, mine


def plain_toy(W, ids, cfg=RAW):
    x = W["emb"][torch.as_tensor(ids)]
    silu_mlp = lambda h, p: (torch.nn.functional.silu(h @ W[p + "gate"].T) * (h @ W[p + "up"].T)) @ W[p + "down"].T
    first_kv = None
    for entry, (layer, reads) in enumerate([(0, None), (1, None), (2, None), (0, None), (1, None), (0, 0)]):
        p = f"l{layer}."
        h = plain_norm(x, W[p + "n1"])
        if layer == 1:
            s, rows = torch.zeros(32, dtype=x.dtype), []
            for t in range(h.shape[0]):
                s = cfg["decay"] * s + h[t]
                rows.append(s)
            y = torch.stack(rows) @ W["l1.decay_w"].T
        else:
            y, kv = plain_attention(h, W, p, cfg["window"] if layer == 2 else None, kv_from=first_kv if reads == 0 else None)
            if entry == 0:
                first_kv = kv
        x = x + y
        x = x + silu_mlp(plain_norm(x, W[p + "n2"]), p)
    return plain_norm(x, W["final"]) @ W["head"].T


@pytest.fixture(scope="module")
def toy_folder(tmp_path_factory):
    from wllm_amd.parts import build_model
    folder = str(tmp_path_factory.mktemp("toy"))
    model = build_model(RAW)
    write_random_model(folder, RAW, model.expected_tensors(), seed=5, std=0.15, norm_std=0.3)
    # norm weights of this toy multiply directly: move them near one
    from wllm_amd.weights import Checkpoint, write_safetensors
    ck = Checkpoint(folder)
    tensors = {n: ck.tensor(n) for n in ck.names()}
    ck.close()
    for n in tensors:
        if n.endswith(("n1", "n2", "final")):
            tensors[n] = (tensors[n].float() + 1.0).to(torch.bfloat16)
    write_safetensors(os.path.join(folder, "model.safetensors"), tensors)
    return folder


def check_toy(toy_folder, device):
    model = load_model(toy_folder, "float32", device)
    needs = model.cache_needs()
    assert sorted(needs) == [0, 2, 3], "runs 1 and 4 keep no pages, run 5 reads run 0's"
    assert sorted(model.state_shapes()) == [1, 4], "each run of the toy mixer has a state of its own"
    W = P.read_weights(toy_folder, torch.float32)
    requests = {f"r{i}": random_ids(i, n, 97) for i, n in enumerate([30, 45, 26, 61, 38])}
    plain = {rid: plain_toy(W, t) for rid, t in requests.items()}
    for family in (trace_whole, trace_portions, trace_mixed):
        trace = family(requests)
        runner = ModelRunner.create(model, num_pages=pages_for_max_tokens(max_live_tokens(trace), 4), page_size=4,
                                    max_requests=4, poison_freed_pages=True)
        assert len(runner.cache.groups) == 2, "all keys and a window of them: two groups of pages"
        got = replay_and_collect(TraceReplayer(runner), trace)
        compare_with_plain(got, plain, atol=5e-5, rtol=2e-4)
        runner.cache.check()
        assert all(g.pool.num_free == g.pool.num_pages for g in runner.cache.groups)


def test_toy_architecture_on_the_cpu_with_emulated_kernels(toy_folder):
    with ops.use_backend(EmulatedKernels()):
        check_toy(toy_folder, "cpu")


@pytest.mark.gpu
def test_toy_architecture_on_the_gpu(toy_folder):
    check_toy(toy_folder, "cuda")
