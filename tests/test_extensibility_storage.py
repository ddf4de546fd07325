"""That what a mixer keeps, and how positions enter, can be something the framework has no case of.

A third toy architecture, defined here: a mixer that pages a compressed vector per token instead of
keys and values (its pages come from the cache manager like any others, in a group of their own)
and counts its tokens in an int32 state row; a position encoding that is no rotation (a learned
table added to queries and keys by a step of its own, with its tensor in the checkpoint); and a
model folder for it written by the command line's `random-model`, which knows the architecture only
through the registry.  Nothing under `wllm_amd/` is edited for any of it.  The toy is no model of
anyone's.
"""
import json
from dataclasses import dataclass

import pytest
import torch

from helpers import compare_with_plain, max_live_tokens, random_ids, replay_and_collect, trace_mixed, trace_portions, trace_whole
from kernel_emulation import EmulatedKernels
from plain import gemma_plain as P
from wllm_amd import cli
from wllm_amd.cache import PagedNeed, StateNeed
from wllm_amd.config import register_architecture
from wllm_amd.engine import ModelRunner
from wllm_amd.engine.replay import TraceReplayer, pages_for_max_tokens
from wllm_amd.kernels import ops
from wllm_amd.parts import load_model, register_mixer, register_position
from wllm_amd.parts.specs import (AttentionSpec, BlockSpec, EmbeddingSpec, GatedMLPSpec, HeadSpec, MixerSpec, ModelPlan,
                                  NormSpec, PositionSpec, ScheduleEntry)
from wllm_amd.weights import ExpectedTensor

H, R, HEADS, KV, D, MAXPOS = 40, 6, 2, 1, 16, 160


# ---- a mixer that pages a compressed vector: c_t = h_t Wc^T is kept; y_t = mean(c_0..c_t) Wu^T ----
@dataclass(frozen=True)
class LatentSpec(MixerSpec):
    kind: str = "toy_latent"
    hidden_size: int = 0
    rank: int = 0
    prefix: str = ""


@register_mixer("toy_latent", replace=True)
class LatentMixer:
    def __init__(self, spec):
        self.spec = spec

    def expected_tensors(self):
        s = self.spec
        return {s.prefix + "compress": ExpectedTensor((s.rank, s.hidden_size)),
                s.prefix + "expand": ExpectedTensor((s.hidden_size, s.rank))}

    def load(self, fetch):
        self.wc = fetch.to_device(fetch.matrix(self.spec.prefix + "compress"))
        self.wu = fetch.to_device(fetch.matrix(self.spec.prefix + "expand"))

    def cache_need(self):
        return PagedNeed((self.spec.rank,), dtype=torch.float32)      # pages of [page_size, rank], float32 in every mode

    def state_shape(self):
        return StateNeed((1,), torch.int32)                            # how many tokens the request has fed

    def forward(self, ctx, entry, h):
        pages, counts = ctx.pages(entry), ctx.state(entry)
        assert counts.dtype == torch.int32
        latent = torch.empty(h.shape[0], self.spec.rank, dtype=h.dtype, device=h.device)
        ops.linear(h, self.wc, latent)
        flat = pages.storage.view(-1, self.spec.rank)                  # [pages * page_size, rank]
        flat[pages.slots.long()] = latent.float()
        mixed = torch.empty(h.shape[0], self.spec.rank, dtype=torch.float32, device=h.device)
        tables = pages.block_tables.cpu()
        for s in range(ctx.num_segments):
            q0, ql, total = int(ctx.host_q_start[s]), int(ctx.host_q_len[s]), int(ctx.host_ctx_len[s])
            slot = int(ctx.host_state_slots[s])
            assert int(counts[slot, 0]) == total - ql, "the state row has counted the tokens fed before"
            counts[slot, 0] += ql
            pos = torch.arange(total)
            where = (tables[s][pos // pages.page_size].long() * pages.page_size + pos % pages.page_size).to(h.device)
            sums = flat[where].cumsum(0)[total - ql:]
            mixed[q0:q0 + ql] = sums / torch.arange(total - ql + 1, total + 1, device=h.device)[:, None]
        y = ctx.buffer("latent_out", tuple(h.shape), h.dtype)
        ops.linear(mixed.to(h.dtype), self.wu, y)
        return y


# ---- a position encoding that is no rotation: a learned row per position added to queries and keys ----
@register_position("toy_additive", replace=True)
class AdditivePositions:
    inv_freq = None                          # nothing for the rotation kernels to turn by

    def __init__(self, spec):
        self.spec = spec

    def expected_tensors(self):
        return {"positions.table": ExpectedTensor((MAXPOS, self.spec.rotary_dim))}

    def load(self, fetch):
        self.table = fetch.to_device(fetch.matrix("positions.table"))

    def prepare(self, device):
        pass

    def apply(self, ctx, qkv, *, num_heads, num_kv_heads, head_dim):
        rows = self.table[ctx.positions.long()]                           # [tokens, head_dim]
        qk = qkv[:, :(num_heads + num_kv_heads) * head_dim].view(qkv.shape[0], num_heads + num_kv_heads, head_dim)
        qk += rows[:, None, :].to(qkv.dtype)


@dataclass(frozen=True)
class Toy3Config:
    vocab_size: int
    rank: int

    @classmethod
    def from_dict(cls, raw):
        if raw["rank"] <= 0:
            raise ValueError("rank must be positive")
        return cls(raw["vocab_size"], raw["rank"])


def toy3_plan(cfg):
    norm = lambda name: NormSpec(size=H, eps=1e-5, weight=name, weight_offset=1.0)
    ffn = lambda p: GatedMLPSpec(hidden_size=H, intermediate_size=56, activation="gelu_tanh", gate_weight=p + "gate",
                                 up_weight=p + "up", down_weight=p + "down")
    layers = (
        BlockSpec(mixer=LatentSpec(hidden_size=H, rank=cfg.rank, prefix="a."), feed_forward=ffn("a."),
                  mixer_norm=norm("a.n1"), feed_forward_norm=norm("a.n2")),
        BlockSpec(mixer=AttentionSpec(hidden_size=H, num_heads=HEADS, num_kv_heads=KV, head_dim=D, scale=D ** -0.5,
                                      position=PositionSpec(kind="toy_additive", rotary_dim=D),
                                      q_weight="b.q", k_weight="b.k", v_weight="b.v", o_weight="b.o"),
                  feed_forward=ffn("b."), mixer_norm=norm("b.n1"), feed_forward_norm=norm("b.n2")),
    )
    return ModelPlan(embedding=EmbeddingSpec(cfg.vocab_size, H, "emb"), layers=layers,
                     schedule=(ScheduleEntry(0), ScheduleEntry(1), ScheduleEntry(0)),
                     final_norm=norm("final"), head=HeadSpec(cfg.vocab_size, H, "head"), max_positions=MAXPOS)


register_architecture("ToyLatentForCausalLM", Toy3Config.from_dict, toy3_plan, replace=True)
RAW = {"architectures": ["ToyLatentForCausalLM"], "vocab_size": 71, "rank": R, "a_key_of_its_own": "kept"}


def plain_toy3(W, ids):
    T = len(ids)
    x = W["emb"][torch.as_tensor(ids)]
    rms = lambda v, w: v * torch.rsqrt(v.pow(2).mean(-1, keepdim=True) + 1e-5) * (1.0 + w)

    def latent(h):
        c = h @ W["a.compress"].T
        return (c.cumsum(0) / torch.arange(1, T + 1)[:, None]) @ W["a.expand"].T

    def attention(h):
        q = (h @ W["b.q"].T).view(T, HEADS, D) + W["positions.table"][:T, None, :]
        k = (h @ W["b.k"].T).view(T, KV, D) + W["positions.table"][:T, None, :]
        v = (h @ W["b.v"].T).view(T, KV, D)
        k, v = k.repeat_interleave(HEADS // KV, 1), v.repeat_interleave(HEADS // KV, 1)
        scores = torch.einsum("qhd,khd->hqk", q, k) * D ** -0.5
        i = torch.arange(T)
        probs = torch.softmax(scores.masked_fill(~(i[None, :] <= i[:, None])[None], float("-inf")), -1)
        return torch.einsum("hqk,khd->qhd", probs, v).reshape(T, HEADS * D) @ W["b.o"].T

    for p, mixer in (("a.", latent), ("b.", attention), ("a.", latent)):
        x = x + mixer(rms(x, W[p + "n1"]))
        x = x + P.geglu_mlp(rms(x, W[p + "n2"]), W[p + "gate"], W[p + "up"], W[p + "down"])
    return rms(x, W["final"]) @ W["head"].T


@pytest.fixture(scope="module")
def toy3_folder(tmp_path_factory):
    """Written by the command line: `random-model --config FILE`, the file naming the toy architecture."""
    root = tmp_path_factory.mktemp("toy3")
    (root / "toy.json").write_text(json.dumps(RAW))
    folder = str(root / "model")
    assert cli.main(["random-model", "--out", folder, "--config", str(root / "toy.json"), "--seed", "4", "--std", "0.2",
                     "--norm-std", "0.2"]) == 0
    with open(f"{folder}/config.json") as f:
        assert json.load(f) == RAW, "config.json is what was given, keys the framework does not know included"
    return folder


def test_random_model_refuses_what_the_architecture_refuses(tmp_path):
    (tmp_path / "bad.json").write_text(json.dumps(dict(RAW, rank=0)))
    with pytest.raises(ValueError, match="rank"):
        cli.main(["random-model", "--out", str(tmp_path / "m"), "--config", str(tmp_path / "bad.json")])


def check_toy3(folder, device, dtype="float32"):
    model = load_model(folder, dtype, device)
    needs = model.cache_needs()
    assert sorted(needs) == [0, 1, 2] and isinstance(needs[0], PagedNeed)
    W = P.read_weights(folder, torch.float32)
    requests = {f"r{i}": random_ids(70 + i, n, 71) for i, n in enumerate([29, 44, 18, 53])}
    plain = {rid: plain_toy3(W, t) for rid, t in requests.items()}
    for family in (trace_whole, trace_portions, trace_mixed):
        trace = family(requests)
        runner = ModelRunner.create(model, num_pages=pages_for_max_tokens(max_live_tokens(trace), 4), page_size=4,
                                    max_requests=4, poison_freed_pages=True)
        cache = runner.cache
        assert len(cache.groups) == 2, "compressed vectors and keys/values: two groups of pages"
        latent_group = cache.groups[cache.group_of_entry[0]]
        assert tuple(latent_group.storage.shape[2:]) == (4, R) and latent_group.storage.dtype == torch.float32
        assert cache.state[0].dtype == torch.int32 and tuple(cache.state[0].shape) == (4 + 1, 1)      # max_requests rows and the padding row
        got = replay_and_collect(TraceReplayer(runner), trace)
        tol = dict(atol=5e-5, rtol=2e-4) if dtype == "float32" else dict(atol=8e-2, rtol=3e-2)      # logits up to 3 from weights of std 0.2
        compare_with_plain(got, plain, **tol)
        cache.check()
        assert all(g.pool.num_free == g.pool.num_pages for g in cache.groups)


def test_paged_latents_int_state_and_additive_positions_on_the_cpu(toy3_folder):
    with ops.use_backend(EmulatedKernels()):
        check_toy3(toy3_folder, "cpu")


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_paged_latents_int_state_and_additive_positions_on_the_gpu(toy3_folder, dtype):
    check_toy3(toy3_folder, "cuda", dtype)
