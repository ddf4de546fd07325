"""Generation on the GPU through the entry point and the scheduler, the replay program as a
subprocess, long decoding and the first tokens of a sequence."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

from helpers import (TINY, VARIED, assert_varied, bfloat16_row_errors, compare_replay, plain_exact_and_rounded, plain_for, random_ids,
                     replay_and_collect, trace_tail, trace_whole)
from plain import gemma_plain
from wllm_amd.engine import LLM, ModelRunner, Request, Scheduler
from wllm_amd.engine.replay import TraceReplayer
from wllm_amd.parts import load_model
from wllm_amd.sampling import SamplingParams

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def plain_model(folder):
    return gemma_plain.read_config(folder), gemma_plain.read_weights(folder, torch.float32)


@pytest.mark.parametrize("name,lengths,new", [("C", [9, 20], 6), ("AV", [7, 16, 23], 12), ("MV", [33, 70, 12], 12)])
def test_greedy_generation_through_the_entry_point_float32(model_folders, varied_folders, name, lengths, new):
    """Greedy decoding of models whose continuation varies (so that a wrong key, page or position
    changes the tokens): the plain implementation's full recomputation, token for token."""
    folder = model_folders[name] if name in model_folders else varied_folders[name]
    cfg, w = plain_model(folder)
    prompts = [random_ids(i + 1, n, cfg["vocab_size"]) for i, n in enumerate(lengths)]
    llm = LLM(folder, dtype="float32", num_blocks=64, block_size=(TINY.get(name) or VARIED[name])["page_size"])
    outs = llm.generate(prompts, max_new_tokens=new)
    for p, o in zip(prompts, outs):
        assert_varied(o.token_ids)
        assert o.token_ids == gemma_plain.generate_greedy(cfg, w, p, new)
        assert o.finish_reason == "length" and len(o.logprobs) == new
        full = gemma_plain.forward_logits(cfg, w, p + o.token_ids[:-1])
        ref_lp = torch.log_softmax(full[len(p) - 1:].double(), -1).gather(-1, torch.tensor(o.token_ids)[:, None])[:, 0]
        assert torch.allclose(torch.tensor(o.logprobs, dtype=torch.float64), ref_lp, atol=1e-4)
    llm.runner.cache.check()


@pytest.mark.parametrize("name,lengths,new,temperature", [("A", [7, 16, 23], 8, 0.3), ("B", [5, 31, 64], 6, 0.5),
                                                          ("M", [33, 70], 6, 0.8)])
def test_seeded_sampling_through_the_entry_point_float32(model_folders, name, lengths, new, temperature):
    """The first case is a tiny workload of its own: prompts of 7/16/23 ids, 8 tokens each, pages of 4.
    Greedy decoding of these three models repeats the last prompt token whatever the context adds (the
    tied head's logit of a token for itself wins), so they sample, at a temperature at which the
    context decides among a handful of tokens: every token must be the one that the plain
    implementation's distribution gives the request's uniform number."""
    from plain import sampling_plain
    folder = model_folders[name]
    cfg, w = plain_model(folder)
    prompts = [random_ids(i + 1, n, cfg["vocab_size"]) for i, n in enumerate(lengths)]
    params = [SamplingParams(temperature=temperature, seed=900 + i) for i in range(len(prompts))]
    llm = LLM(folder, dtype="float32", num_blocks=64, block_size=TINY[name]["page_size"])
    outs = llm.generate(prompts, params, max_new_tokens=new)
    assert len({t for o in outs for t in o.token_ids}) >= 6, "the sampled tokens vary"
    for i, (p, o) in enumerate(zip(prompts, outs)):
        tokens = list(p)
        for k, t in enumerate(o.token_ids):
            logits = gemma_plain.forward_logits(cfg, w, tokens)[-1]
            u = sampling_plain.philox_uniform(900 + i, k)
            _, _, _, (low, high) = sampling_plain.sample_row(logits, temperature, 0, 1.0, 0.0, 1.0, [], u)
            assert low[t] - 1e-4 <= u <= high[t] + 1e-4, f"request {i} token {k}"
            ref_lp = float(torch.log_softmax(logits.double() / temperature, -1)[t])
            assert abs(o.logprobs[k] - ref_lp) < 1e-4
            tokens.append(t)
        assert o.finish_reason == "length"
    llm.runner.cache.check()


@pytest.mark.parametrize("name", ["A", "M"])
def test_greedy_generation_bfloat16_follows_the_plain_implementation_up_to_near_ties(model_folders, name):
    cfg, w = plain_model(model_folders[name])
    prompts = [random_ids(i + 50, n, cfg["vocab_size"]) for i, n in enumerate([12, 40])]
    llm = LLM(model_folders[name], dtype="bfloat16", num_blocks=64, block_size=16)
    for p, o in zip(prompts, llm.generate(prompts, max_new_tokens=8)):
        tokens = list(p)
        for t in o.token_ids:
            logits = gemma_plain.forward_logits(cfg, w, tokens, scale_rounding=torch.bfloat16)[-1]
            best = int(logits.argmax())
            if t != best:
                # a different token is acceptable only where the plain logits nearly tie
                assert (logits[best] - logits[t]).item() < 2e-2, f"token {t} instead of {best}, gap {(logits[best] - logits[t]).item()}"
                break
            tokens.append(t)


def test_chunked_prefill_beside_decodes_with_seeded_temperature(model_folders):
    """A second tiny workload: four prompts of 5/31/64/97 ids, portions of 16 beside
    decoding requests, temperature 0.8 from a seeded generator, pages of 8.  Each request's tokens
    equal those it gets alone, and each token is one the plain implementation's distribution gives
    the request's uniform number."""
    from plain import sampling_plain
    folder = model_folders["B"]
    cfg, w = plain_model(folder)
    model = load_model(folder, "float32", "cuda")
    prompts = [random_ids(7 * i + 3, n, cfg["vocab_size"]) for i, n in enumerate([5, 31, 64, 97])]
    params = [SamplingParams(temperature=0.8, seed=500 + i) for i in range(4)]

    def run(which, budget):
        runner = ModelRunner.create(model, num_pages=40, page_size=8, max_requests=4)
        s = Scheduler(runner, max_prefill_tokens_per_step=budget)
        reqs = [Request(i, prompts[i], 10, sampling_params=params[i]) for i in which]
        for r in reqs:
            s.add_request(r)
        s.run_to_completion()
        runner.cache.check()
        return reqs

    together = run(range(4), 16)
    for i, r in enumerate(together):
        assert run([i], None)[0].output_token_ids == r.output_token_ids
        tokens = list(prompts[i])
        for k, t in enumerate(r.output_token_ids):
            logits = gemma_plain.forward_logits(cfg, w, tokens)[-1]
            u = sampling_plain.philox_uniform(r.seed, k)
            _, _, _, (low, high) = sampling_plain.sample_row(logits, 0.8, 0, 1.0, 0.0, 1.0, [], u)
            assert low[t] - 1e-4 <= u <= high[t] + 1e-4
            tokens.append(t)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding(model_folders, dtype):
    """300 tokens decoded one by one after a short prompt, over many page boundaries."""
    folder = model_folders["M"]
    cfg, _ = plain_model(folder)
    toks = random_ids(9, 340, cfg["vocab_size"])
    plain = plain_for(cfg, folder, {"r": toks}, dtype)
    runner = ModelRunner.create(load_model(folder, dtype, "cuda"), num_pages=22, page_size=16, max_requests=2)
    got = replay_and_collect(TraceReplayer(runner), trace_tail({"r": toks}, tail=300))
    compare_replay(got, plain, dtype)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B"])
def test_first_tokens_of_a_sequence(model_folders, name, dtype):
    """Prompts of one, two and three tokens, whole and token by token."""
    folder = model_folders[name]
    cfg, _ = plain_model(folder)
    requests = {f"r{n}": random_ids(n, n, cfg["vocab_size"]) for n in (1, 2, 3)}
    plain = plain_for(cfg, folder, requests, dtype)
    model = load_model(folder, dtype, "cuda")
    for trace in (trace_whole(requests), trace_tail(requests, tail=3)):
        runner = ModelRunner.create(model, num_pages=8, page_size=TINY[name]["page_size"], max_requests=2)
        compare_replay(replay_and_collect(TraceReplayer(runner), trace), plain, dtype)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_run_program(model_folders, tmp_path, dtype):
    """bin/trace_run as a user calls it: steps on standard input, `done <step>` lines, logits files."""
    folder = model_folders["A"]
    cfg, w = plain_model(folder)
    a, b = random_ids(1, 30, 512), random_ids(2, 21, 512)
    steps = [
        {"step": 0, "entries": [{"id": "a", "tokens": a[:17], "want": [0, 16]}], "end": []},
        {"step": 1, "entries": [{"id": "a", "tokens": a[17:19], "want": []}, {"id": "b", "tokens": b[:20], "want": [19]}], "end": []},
        {"step": 2, "entries": [{"id": "b", "tokens": b[20:], "want": [0]}, {"id": "a", "tokens": a[19:], "want": [10]}], "end": ["a", "b"]},
        {"step": 7, "entries": [{"id": "a", "tokens": b[:2], "want": [1]}], "end": ["a"]},
    ]
    out = tmp_path / "out"
    proc = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", folder, "--dtype", dtype,
                           "--out", str(out), "--max-tokens", "128"],
                          input="\n".join(json.dumps(s) for s in steps) + "\n", capture_output=True, text=True, timeout=300)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert proc.stdout.split() == ["done", "0", "done", "1", "done", "2", "done", "7"]
    expect = {0: [("a", 0), ("a", 16)], 1: [("b", 19)], 2: [("b", 20), ("a", 29)], 7: [("b", 1)]}
    if dtype == "float32":
        plain = {"a": gemma_plain.forward_logits(cfg, w, a), "b": gemma_plain.forward_logits(cfg, w, b)}
    else:
        w64 = gemma_plain.read_weights(folder, torch.float64)
        plain = {"a": plain_exact_and_rounded(cfg, w64, a), "b": plain_exact_and_rounded(cfg, w64, b)}
    for step, rows in expect.items():
        got = torch.from_numpy(np.fromfile(out / f"{step}.f32", dtype="<f4").reshape(len(rows), 512))
        for row, (rid, pos) in zip(got, rows):
            if dtype == "float32":
                ref = plain[rid][pos].double()
                assert ((row.double() - ref).abs() <= 2e-5 + 1e-4 * ref.abs()).all(), f"step {step}"
            else:
                assert max(bfloat16_row_errors(row, plain[rid][0][pos], [r[pos] for r in plain[rid][1]])) <= 1.0, f"step {step}"


def test_trace_run_says_when_a_trace_holds_more_than_max_tokens(model_folders, tmp_path):
    """Two live requests of 100 tokens against --max-tokens 128: one line that names the step and
    the limit, a non-zero exit, and the steps before it done."""
    folder = model_folders["A"]
    a, b = random_ids(3, 100, 512), random_ids(4, 100, 512)
    steps = [
        {"step": 0, "entries": [{"id": "a", "tokens": a, "want": [99]}], "end": []},
        {"step": 1, "entries": [{"id": "b", "tokens": b, "want": [99]}], "end": ["a", "b"]},
    ]
    out = tmp_path / "out"
    proc = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", folder, "--dtype", "float32",
                           "--out", str(out), "--max-tokens", "128"],
                          input="\n".join(json.dumps(s) for s in steps) + "\n", capture_output=True, text=True, timeout=300)
    assert proc.returncode != 0
    assert proc.stdout.split() == ["done", "0"]
    assert "step 1" in proc.stderr and "--max-tokens 128" in proc.stderr
    assert "Traceback" not in proc.stderr
    assert (out / "0.f32").exists() and not (out / "1.f32").exists()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["MV", "WV"])
def test_captured_graphs_give_what_eager_steps_give(varied_folders, name, dtype):
    """Decode steps replayed from captured graphs against the same steps run kernel by kernel:
    several replays with eager work (prompt portions of newly admitted requests) between them,
    batches that grow and shrink through the buckets, every replay checked.  "WV" has 32 query heads
    on one key/value head: a decoded token's rows fill two tiles of the decode kernel, and the
    contexts grow past one chunk of keys, so its graphs hold partial results of both tiles."""
    folder = varied_folders[name]
    model = load_model(folder, dtype, "cuda")
    vocab = VARIED[name]["config"].vocab_size
    prompts = [random_ids(40 + i, n, vocab) for i, n in enumerate([9, 33, 17, 120, 5, 41])]
    news = [30, 12, 25, 28, 40, 18]

    def run(graphs):
        runner = ModelRunner.create(model, num_pages=40, page_size=16, max_requests=4)
        if graphs:
            runner.enable_graphs(buckets=(1, 2, 4))
        s = Scheduler(runner, max_prefill_tokens_per_step=16)
        reqs = [Request(i, p, n) for i, (p, n) in enumerate(zip(prompts, news))]
        for r in reqs:
            s.add_request(r)
        s.run_to_completion()
        runner.cache.check()
        return reqs, runner

    eager, _ = run(False)
    graphed, runner = run(True)
    assert runner.graph_steps > 20 and len(runner.graphs) >= 2
    for a, b in zip(eager, graphed):
        assert a.output_token_ids == b.output_token_ids
        assert_varied(a.output_token_ids)
        assert torch.allclose(torch.tensor(a.logprobs), torch.tensor(b.logprobs), atol=1e-5 if dtype == "float32" else 2e-2)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_graphs_for_classes_of_context_lengths(varied_folders, dtype):
    """A bucket has a graph for each class of context lengths; requests that grow from 20 to 150
    tokens pass through the graphs for at most 48, 96 and 200 tokens, beside a shorter request
    that comes later, and generate what steps run kernel by kernel generate."""
    model = load_model(varied_folders["MV"], dtype, "cuda")
    prompts = [random_ids(70, 20, 1000), random_ids(71, 30, 1000), random_ids(72, 6, 1000)]
    news = [130, 90, 25]

    def run(graphs):
        runner = ModelRunner.create(model, num_pages=40, page_size=16, max_requests=2)
        if graphs:
            runner.enable_graphs(buckets=(1, 2), max_context=200, contexts=(48, 96))
            assert runner.graph_contexts == (48, 96, 200)
        s = Scheduler(runner, max_prefill_tokens_per_step=32, lookahead=True)
        reqs = [Request(i, p, n) for i, (p, n) in enumerate(zip(prompts, news))]
        for r in reqs:
            s.add_request(r)
        s.run_to_completion()
        runner.cache.check()
        return reqs, runner

    eager, _ = run(False)
    graphed, runner = run(True)
    assert sorted(runner.graphs[2]) == [48, 96, 200] and runner.graph_steps > 100, {b: sorted(g) for b, g in runner.graphs.items()}
    widths = {c: g.table_width for c, g in runner.graphs[2].items()}
    assert widths == {48: 3, 96: 6, 200: 13}
    for a, b in zip(eager, graphed):
        assert a.output_token_ids == b.output_token_ids
        assert_varied(a.output_token_ids)


def test_a_full_batch_of_any_size_has_its_graph(varied_folders):
    """The largest number of requests the cache admits is a bucket of its own: a full batch of 3
    (or 17) does not fall back to steps run kernel by kernel."""
    model = load_model(varied_folders["MV"], "bfloat16", "cuda")
    runner = ModelRunner.create(model, num_pages=40, page_size=16, max_requests=3)
    runner.enable_graphs()
    assert runner.graph_buckets == (1, 2, 3)
    s = Scheduler(runner, max_prefill_tokens_per_step=64)
    reqs = [Request(i, random_ids(90 + i, 11 + i, 1000), 12) for i in range(3)]
    for r in reqs:
        s.add_request(r)
    s.run_to_completion()
    assert 3 in runner.graphs and runner.graph_steps >= 8
    plain = ModelRunner.create(model, num_pages=40, page_size=16, max_requests=3)
    s2 = Scheduler(plain, max_prefill_tokens_per_step=64)
    again = [Request(i, random_ids(90 + i, 11 + i, 1000), 12) for i in range(3)]
    for r in again:
        s2.add_request(r)
    s2.run_to_completion()
    assert [r.output_token_ids for r in reqs] == [r.output_token_ids for r in again]
    assert_varied(reqs[0].output_token_ids)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("graphs", [False, True])
def test_looking_ahead_gives_the_same_tokens_on_the_gpu(varied_folders, dtype, graphs):
    """Steps started before the step before them was read (token ids taken from the device, in
    eager steps and in replayed graphs) against the same requests run step by step: mixed greedy
    and seeded sampling, prompt portions beside decoded tokens, requests that stop on a token: in the
    middle of what they generate, at the last output but one (the step run ahead has filled the
    request's length by then) and at the last."""
    folder = varied_folders["MV"]
    model = load_model(folder, dtype, "cuda")
    prompts = [random_ids(90 + i, n, 1000) for i, n in enumerate([9, 33, 17, 70, 5, 41, 12])]
    news = [30, 12, 25, 8, 40, 18, 22]
    params = [SamplingParams(temperature=0.7, top_p=0.9, seed=40 + i) if i % 2 else SamplingParams() for i in range(7)]

    # Looking ahead changes which requests share a step (a request that stops is in one step more).
    # In bfloat16 the kernels for at most 16 rows and for more round differently, so the portions
    # are kept small enough that every step of both runs has at most 16 rows and takes the same
    # kernels; float32 has no such boundary.
    budget = 16 if dtype == "float32" else 8

    def run(lookahead, stops):
        runner = ModelRunner.create(model, num_pages=40, page_size=16, max_requests=4)
        if graphs:
            runner.enable_graphs(buckets=(1, 2, 4))
        s = Scheduler(runner, max_prefill_tokens_per_step=budget, lookahead=lookahead)
        reqs = [Request(i, p, n, sampling_params=sp, **stops.get(i, {}))
                for i, (p, n, sp) in enumerate(zip(prompts, news, params))]
        for r in reqs:
            s.add_request(r)
        s.run_to_completion()
        runner.cache.check()
        assert not runner.cache.requests
        return reqs, runner

    free, _ = run(False, {})
    for r in free:
        assert_varied(r.output_token_ids)

    def stop_at(i, index):
        """A token of request i that first occurs at `index` of what it generates freely, or near it."""
        out = free[i].output_token_ids
        index = next(k for k in [index] + list(range(len(out) - 1, -1, -1)) if out.index(out[k]) == k)
        return out[index], index

    # three stop in the middle, one at its last output but one, one at its last
    wanted = {0: 11, 3: 2, 4: 20, 1: news[1] - 2, 5: news[5] - 1}
    stops, places = {}, {}
    for i, index in wanted.items():
        token, places[i] = stop_at(i, index)
        stops[i] = dict(eos_token_id=token) if i % 2 == 0 else dict(stop_token_ids=frozenset([token]))
    assert places[1] == news[1] - 2 or places[5] == news[5] - 1, "a stop at the end of a request's length is among them"
    stepwise, _ = run(False, stops)
    ahead, runner = run(True, stops)
    if graphs:
        assert runner.graph_steps > 20
    assert sum(r.finish_reason == "stop" for r in ahead) == 5
    for i, index in places.items():
        assert ahead[i].output_token_ids == free[i].output_token_ids[:index + 1]
    for a, b in zip(stepwise, ahead):
        assert a.output_token_ids == b.output_token_ids and a.finish_reason == b.finish_reason
        assert torch.allclose(torch.tensor(a.logprobs), torch.tensor(b.logprobs), atol=1e-5 if dtype == "float32" else 2e-2)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_requests_preempted_between_replayed_graphs_and_steps_run_ahead(varied_folders, dtype):
    """Pages run out in the middle of decoding (`admission="prompt_only"` admits on the prompts alone)
    while decode steps replay captured graphs and every step is started before the one before it was
    read: the request admitted last gives its pages back, keeps what it generated, comes back through
    a prompt of its own and goes on.  In float32 every request generates what it generates with pages
    to spare, step by step and kernel by kernel; in bfloat16 (where a token recomputed inside a prompt
    is rounded differently from the token that was decoded) every request still completes, the cache's
    books are right after every step, and the requests that were never preempted generate the same."""
    model = load_model(varied_folders["MV"], dtype, "cuda")
    prompts = [random_ids(300 + i, n, 1000) for i, n in enumerate([20, 37, 12, 30, 25])]
    news = [40, 30, 45, 28, 35]

    def run(pages, admission, graphs, lookahead):
        runner = ModelRunner.create(model, num_pages=pages, page_size=16, max_requests=4)
        if graphs:
            runner.enable_graphs(buckets=(1, 2, 4))
        s = Scheduler(runner, max_prefill_tokens_per_step=32, admission=admission, lookahead=lookahead)
        reqs = [Request(i, p, n) for i, (p, n) in enumerate(zip(prompts, news))]
        for r in reqs:
            s.add_request(r)
        steps = 0
        while s.has_unfinished_requests():
            s.step()
            runner.cache.check()
            steps += 1
            assert steps < 2000
        assert not runner.cache.requests
        return reqs, s, runner

    roomy, s0, _ = run(40, "pledged", False, False)
    assert s0.stats["preemptions"] == 0
    tight, s1, runner = run(9 + 1, "prompt_only", True, True)       # nine pages for requests, one for the graphs' padding rows
    assert s1.stats["preemptions"] >= 2 and runner.graph_steps > 20
    assert sum(r.num_preemptions > 0 for r in tight) >= 2
    for a, b in zip(roomy, tight):
        assert b.finish_reason == "length" and len(b.output_token_ids) == len(a.output_token_ids)
        assert_varied(b.output_token_ids)
        if dtype == "float32" or b.num_preemptions == 0:
            assert a.output_token_ids == b.output_token_ids, f"request {a.request_id} (preempted {b.num_preemptions} times)"


def test_command_line_takes_stop_tokens(varied_folders):
    """`--stop-token-ids`: the request ends with the first of them that it generates, which is kept
    (the reference's finishing rule, src/wllm/engine/sequence.py:53-59)."""
    folder = varied_folders["AV"]
    cfg, w = plain_model(folder)
    prompt = random_ids(5, 9, 512)
    free = gemma_plain.generate_greedy(cfg, w, prompt, 8)
    stop = free[3]
    first = free.index(stop)
    args = [sys.executable, "-m", "wllm_amd.cli", "generate", "--model", folder, "--dtype", "float32", "--num-blocks", "32",
            "--block-size", "4", "--max-new-tokens", "8", "--prompt-ids", ",".join(str(t) for t in prompt),
            "--stop-token-ids", f"{stop},511"]
    proc = subprocess.run(args, capture_output=True, text=True, timeout=300, cwd=ROOT)
    assert proc.returncode == 0, proc.stderr[-2000:]
    line = [json.loads(l) for l in proc.stdout.splitlines() if l.startswith("{")][0]
    assert line["token_ids"] == free[:first + 1] and line["finish_reason"] == "stop"


def test_command_line_generates_what_the_entry_point_generates(varied_folders, tmp_path):
    folder = varied_folders["AV"]
    cfg, w = plain_model(folder)
    prompts = [random_ids(5, 9, 512), random_ids(6, 14, 512)]
    args = [sys.executable, "-m", "wllm_amd.cli", "generate", "--model", folder, "--dtype", "float32", "--num-blocks", "32",
            "--block-size", "4", "--max-new-tokens", "6", "--chunked-prefill-tokens", "8"]
    for p in prompts:
        args += ["--prompt-ids", ",".join(str(t) for t in p)]
    proc = subprocess.run(args, capture_output=True, text=True, timeout=300, cwd=ROOT)
    assert proc.returncode == 0, proc.stderr[-2000:]
    lines = [json.loads(l) for l in proc.stdout.splitlines() if l.startswith("{")]
    assert [l["token_ids"] for l in lines] == [gemma_plain.generate_greedy(cfg, w, p, 6) for p in prompts]
    assert all(l["finish_reason"] == "length" for l in lines)
    assert_varied(lines[0]["token_ids"])
