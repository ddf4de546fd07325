"""That a part can bring a kernel of its own without a change to the framework's files.

The toy mixer here keeps a state per request (a decaying sum of its inputs) and updates it on the GPU,
in a kernel that lies beside this test (`tests/toy_kernels/decay_state.hip`): compiled by the
framework's builder into a library of its own, registered as an operation with its signature, its host
check and its plain emulation, and called through `ops.call`.  Because the update reads the step's
device arrays alone, the mixer's steps can be captured in a graph.  Rows of a captured graph that
stand for no request have a state row of their own: the test decodes from a graph wider than its
live requests while a request holds state slot 0, and compares with the plain computation.
The toy is no model of anyone's.
"""
import os
from ctypes import c_float, c_int, c_void_p
from dataclasses import dataclass

import pytest
import torch

from helpers import compare_with_plain, max_live_tokens, random_ids, replay_and_collect, trace_mixed, trace_portions, trace_whole
from kernel_emulation import EmulatedKernels
from plain import gemma_plain as P
from wllm_amd.config import register_architecture
from wllm_amd.engine import ModelRunner
from wllm_amd.engine.replay import TraceReplayer, pages_for_max_tokens
from wllm_amd.kernels import library, ops
from wllm_amd.parts import load_model, register_mixer
from wllm_amd.parts.specs import (AttentionSpec, BlockSpec, EmbeddingSpec, GatedMLPSpec, HeadSpec, MixerSpec, ModelPlan,
                                  NormSpec, PositionSpec, ScheduleEntry)
from wllm_amd.weights import ExpectedTensor
from wllm_amd.weights.random_init import write_random_model

TOY_KERNELS = os.path.join(os.path.dirname(os.path.abspath(__file__)), "toy_kernels")
HIDDEN, DECAY, VOCAB = 48, 0.8, 131


# ---- the operation: signature, host check, launch, emulation ------------------------------------
def _check(h, state, slots, seg_q_start, seg_q_len, mixed, decay):
    if h.dim() != 2 or h.dtype not in (torch.float32, torch.bfloat16) or not h.is_contiguous():
        raise ops.KernelShapeError("h: expected a contiguous [tokens, hidden] of float32 or bfloat16")
    n, hidden = h.shape
    if state.dtype != torch.float32 or state.dim() != 2 or state.shape[1] != hidden or not state.is_contiguous():
        raise ops.KernelShapeError(f"state: expected float32 [slots, {hidden}]")
    for name, t in (("slots", slots), ("seg_q_start", seg_q_start), ("seg_q_len", seg_q_len)):
        if t.dtype != torch.int32 or t.dim() != 1 or t.shape != slots.shape:
            raise ops.KernelShapeError(f"{name}: expected int32 [segments]")
    if mixed.dtype != torch.float32 or tuple(mixed.shape) != (n, hidden) or not mixed.is_contiguous():
        raise ops.KernelShapeError(f"mixed: expected float32 [{n}, {hidden}]")


def _emulate(h, state, slots, seg_q_start, seg_q_len, mixed, decay):
    for s in range(slots.shape[0]):
        cur = state[int(slots[s])]
        for t in range(int(seg_q_start[s]), int(seg_q_start[s]) + int(seg_q_len[s])):
            cur = decay * cur + h[t].float()
            mixed[t] = cur
        state[int(slots[s])] = cur


ops.register_op(
    "toy_decay_state", entry_point="toy_decay_state",
    argtypes=[c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_float, c_void_p],
    library=lambda: library.load(source_dir=TOY_KERNELS, library_name="libtoy_kernels.so"),
    check=_check, emulate=_emulate, replace=True,
    launch=lambda fn, stream, h, state, slots, seg_q_start, seg_q_len, mixed, decay: fn(
        ops.pointer(h), int(h.dtype == torch.bfloat16), ops.pointer(state), ops.pointer(slots), ops.pointer(seg_q_start),
        ops.pointer(seg_q_len), ops.pointer(mixed), slots.shape[0], h.shape[1], decay, stream))


# ---- the mixer ---------------------------------------------------------------------------------
@dataclass(frozen=True)
class DecayKernelSpec(MixerSpec):
    kind: str = "toy_decay_kernel"
    hidden_size: int = 0
    decay: float = 0.5
    weight: str = ""


@register_mixer("toy_decay_kernel", replace=True)
class DecayKernelMixer:
    graph_capturable = True       # nothing of the step is read on the host

    def __init__(self, spec):
        self.spec = spec
        self.w = None

    def expected_tensors(self):
        return {self.spec.weight: ExpectedTensor((self.spec.hidden_size, self.spec.hidden_size))}

    def load(self, fetch):
        self.w = fetch.to_device(fetch.matrix(self.spec.weight))

    def cache_need(self):
        return None

    def state_shape(self):
        return (self.spec.hidden_size,)

    def forward(self, ctx, entry, h):
        mixed = ctx.buffer("toy_mixed", tuple(h.shape), torch.float32)
        ops.call("toy_decay_state", h, ctx.state(entry), ctx.state_slots, ctx.seg_q_start, ctx.seg_q_len, mixed,
                 self.spec.decay)
        narrow = ctx.buffer("toy_mixed_narrow", tuple(h.shape), h.dtype)
        narrow.copy_(mixed)
        y = ctx.buffer("toy_out", tuple(h.shape), h.dtype)
        ops.linear(narrow, self.w, y)
        return y


@dataclass(frozen=True)
class ToyConfig:
    vocab_size: int
    hidden_size: int
    decay: float

    @classmethod
    def from_dict(cls, raw):
        return cls(raw["vocab_size"], raw["hidden_size"], raw["decay"])


def toy_plan(cfg: ToyConfig) -> ModelPlan:
    h = cfg.hidden_size
    norm = lambda name: NormSpec(size=h, eps=1e-5, weight=name, weight_offset=0.0)
    ffn = lambda p: GatedMLPSpec(hidden_size=h, intermediate_size=2 * h, activation="silu", gate_weight=p + "gate",
                                 up_weight=p + "up", down_weight=p + "down")
    attn = AttentionSpec(hidden_size=h, num_heads=4, num_kv_heads=2, head_dim=16, scale=0.25, window=None,
                         position=PositionSpec(kind="rope", rotary_dim=16, theta=100.0),
                         q_weight="l0.q", k_weight="l0.k", v_weight="l0.v", o_weight="l0.o")
    layers = (
        BlockSpec(mixer=attn, feed_forward=ffn("l0."), mixer_norm=norm("l0.n1"), feed_forward_norm=norm("l0.n2")),
        BlockSpec(mixer=DecayKernelSpec(hidden_size=h, decay=cfg.decay, weight="l1.decay_w"), feed_forward=ffn("l1."),
                  mixer_norm=norm("l1.n1"), feed_forward_norm=norm("l1.n2")),
    )
    return ModelPlan(embedding=EmbeddingSpec(cfg.vocab_size, h, "emb", scale=1.0), layers=layers,
                     schedule=(ScheduleEntry(0), ScheduleEntry(1)), final_norm=norm("final"),
                     head=HeadSpec(cfg.vocab_size, h, "head"), max_positions=256)


register_architecture("ToyDecayKernelForCausalLM", ToyConfig.from_dict, toy_plan, replace=True)
RAW = {"architectures": ["ToyDecayKernelForCausalLM"], "vocab_size": VOCAB, "hidden_size": HIDDEN, "decay": DECAY}


# ---- its plain computation: whole sequence, no cache --------------------------------------------
def plain_toy(W, ids):
    norm = lambda x, w: x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + 1e-5) * w
    mlp = lambda h, p: (torch.nn.functional.silu(h @ W[p + "gate"].T) * (h @ W[p + "up"].T)) @ W[p + "down"].T
    x = W["emb"][torch.as_tensor(ids)]
    T = x.shape[0]
    h = norm(x, W["l0.n1"])
    cos, sin = P.rope_cos_sin(torch.arange(T), 16, 100.0, h.dtype)
    q = P.apply_rope((h @ W["l0.q"].T).view(T, 4, 16), cos, sin)
    k = P.apply_rope((h @ W["l0.k"].T).view(T, 2, 16), cos, sin)
    v = (h @ W["l0.v"].T).view(T, 2, 16)
    scores = torch.einsum("qhd,khd->hqk", q, k.repeat_interleave(2, 1)) * 0.25
    probs = torch.softmax(scores.masked_fill(~torch.ones(T, T, dtype=torch.bool).tril(), float("-inf")), -1)
    x = x + torch.einsum("hqk,khd->qhd", probs, v.repeat_interleave(2, 1)).reshape(T, 64) @ W["l0.o"].T
    x = x + mlp(norm(x, W["l0.n2"]), "l0.")
    h = norm(x, W["l1.n1"])
    s, rows = torch.zeros(HIDDEN, dtype=x.dtype), []
    for t in range(T):
        s = DECAY * s + h[t]
        rows.append(s)
    x = x + torch.stack(rows) @ W["l1.decay_w"].T
    x = x + mlp(norm(x, W["l1.n2"]), "l1.")
    return norm(x, W["final"]) @ W["head"].T


@pytest.fixture(scope="module")
def toy_folder(tmp_path_factory):
    from wllm_amd.parts import build_model
    from wllm_amd.weights import Checkpoint, write_safetensors
    folder = str(tmp_path_factory.mktemp("toy_kernel"))
    write_random_model(folder, RAW, build_model(RAW).expected_tensors(), seed=9, std=0.15, norm_std=0.3)
    ck = Checkpoint(folder)
    tensors = {n: ck.tensor(n) for n in ck.names()}
    ck.close()
    for n in tensors:       # the norm weights of this toy multiply directly: move them near one
        if n.endswith(("n1", "n2", "final")):
            tensors[n] = (tensors[n].float() + 1.0).to(torch.bfloat16)
    write_safetensors(os.path.join(folder, "model.safetensors"), tensors)
    return folder


REQUESTS = {f"r{i}": random_ids(50 + i, n, VOCAB) for i, n in enumerate([30, 45, 26, 61, 38])}


def check_replay(toy_folder, device):
    model = load_model(toy_folder, "float32", device)
    assert sorted(model.state_shapes()) == [1] and model.graph_capturable()
    W = P.read_weights(toy_folder, torch.float32)
    plain = {rid: plain_toy(W, t) for rid, t in REQUESTS.items()}
    for family in (trace_whole, trace_portions, trace_mixed):
        trace = family(REQUESTS)
        runner = ModelRunner.create(model, num_pages=pages_for_max_tokens(max_live_tokens(trace), 8), page_size=8,
                                    max_requests=4, poison_freed_pages=True)
        compare_with_plain(replay_and_collect(TraceReplayer(runner), trace), plain, atol=5e-5, rtol=2e-4)
        runner.cache.check()


def test_a_registered_operation_runs_on_the_cpu_through_its_emulation(toy_folder):
    emu = EmulatedKernels()
    with ops.use_backend(emu):
        check_replay(toy_folder, "cpu")
    assert emu.calls["toy_decay_state"] > 10


def test_the_host_check_of_a_registered_operation_runs_before_the_launch():
    with ops.use_backend(EmulatedKernels()):
        h = torch.zeros(3, 8)
        args = (torch.zeros(2, 8), torch.zeros(1, dtype=torch.int32), torch.zeros(1, dtype=torch.int32),
                torch.ones(1, dtype=torch.int32))
        with pytest.raises(ops.KernelShapeError):
            ops.call("toy_decay_state", h, *args, torch.zeros(3, 9), 0.5)
    with pytest.raises(KeyError):
        ops.call("no_such_operation")
    with pytest.raises(ValueError):
        ops.register_op("toy_decay_state", entry_point="x", argtypes=[], launch=None)


@pytest.mark.gpu
def test_a_registered_kernel_follows_the_plain_computation_on_the_gpu(toy_folder):
    check_replay(toy_folder, "cuda")


@pytest.mark.gpu
def test_padding_rows_of_a_captured_graph_have_a_state_row_of_their_own(toy_folder):
    """Three requests decode from a graph of four rows; the fourth row is padding and runs the toy's
    state update like any other.  The first request holds state slot 0 all the while.  Replays are
    checked against the plain computation one by one, with eager steps (prompts) between them."""
    model = load_model(toy_folder, "float32", "cuda")
    W = P.read_weights(toy_folder, torch.float32)
    requests = {rid: REQUESTS[rid] for rid in ("r0", "r1", "r2")}
    plain = {rid: plain_toy(W, t) for rid, t in requests.items()}
    runner = ModelRunner.create(model, num_pages=40, page_size=8, max_requests=4)
    runner.enable_graphs(buckets=(4,))
    replayer = TraceReplayer(runner)
    prompt = 12
    trace = [{"step": i, "entries": [{"id": rid, "tokens": t[:prompt], "want": list(range(prompt))}], "end": []}
             for i, (rid, t) in enumerate(requests.items())]
    assert runner.cache.open("probe") == 0, "the first request to come takes state slot 0"
    runner.cache.close("probe")
    longest = max(len(t) for t in requests.values())
    for p in range(prompt, longest):
        live = [rid for rid, t in requests.items() if p < len(t)]
        trace.append({"step": len(trace), "entries": [{"id": rid, "tokens": [requests[rid][p]], "want": [0]} for rid in live],
                      "end": [rid for rid in live if p == len(requests[rid]) - 1]})
    got = replay_and_collect(replayer, trace)
    assert runner.graph_steps == longest - prompt, "every decode step was a replay"
    assert len(got) == sum(len(t) for t in requests.values())
    compare_with_plain(got, plain, atol=5e-5, rtol=2e-4)
    # the padding row's state moved (it ran the update), and it is no request's
    state = runner.cache.state[1]
    assert state[runner.cache.padding_slot].abs().sum() > 0
    runner.cache.check()
