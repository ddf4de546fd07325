"""Decode and prefill throughput of the engine at the Gemma-2B layer sizes (or `--shape`), on one MI355X.

    python bench.py --gpus 1 --steps K --warmup W

A step is one decode step of the engine: the scheduler's step over a batch of running
requests (model step from the paged cache, sampling, bookkeeping), measured as the
reference measures decode (scripts/benchmark_decode.py:59-75): warm-up steps, then K timed
steps between device synchronisations, tokens/s = K * batch / elapsed.  Weights are random
(seeded normal, std 0.02), prompts are seeded uniform token ids; no dataset and no checkpoint
is used.  One JSON line is printed.  For more than one GPU the program says that it runs
on one and exits with 2.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

# MI355X's published peaks: HBM3E bandwidth and dense matrix rates per dtype
PEAK_HBM_GBS = 8000.0
PEAK_FLOPS = {"bf16": 2.5e15, "fp16": 2.5e15, "fp8": 5.0e15, "fp32": 157.3e12}


def build_model(shape: dict, dtype: str, seed: int):
    import torch

    from wllm_amd.parts import build_model as build
    from wllm_amd.weights.random_init import RandomFetcher
    model = build(shape)
    tdt = {"bf16": torch.bfloat16, "fp32": torch.float32}[dtype]
    model.load_from(RandomFetcher(model.expected_tensors(), seed, tdt, "cuda:0", std=0.02, norm_std=0.1,
                                  tiled_copies=True))
    return model


def step_flops(model, tokens: int, context_before: int, logit_rows: int) -> float:
    """Floating-point operations of one step over `tokens` new tokens of one request, as the parts count them."""
    keys = tokens * context_before + tokens * (tokens + 1) / 2.0       # what the queries see (causal)
    flops = 0.0
    for e in model.plan.schedule:
        block = model.blocks[e.layer]
        flops += block.mixer.flops(tokens, keys) + block.feed_forward.flops(tokens)
    flops += 2.0 * logit_rows * model.plan.head.hidden_size * model.plan.head.vocab_size
    return flops


def kv_bytes_per_token(model) -> int:
    """Bytes of cache a token holds over all layers: what a decode step reads of a live request, per token."""
    import math
    total = 0
    for need in model.cache_needs().values():
        dtype = getattr(need, "dtype", None) or model.dtype
        total += math.prod(need.page_shape(1)) * dtype.itemsize
    return total


def measure_prefill(model, tokens: int, block_size: int, repeats: int = 6, warm: int = 3):
    """Returns (mean seconds, best seconds) of `repeats` steps that run a prompt of `tokens` tokens whole."""
    import torch

    from wllm_amd.engine import ModelRunner, StepEntry
    pages = -(-tokens // block_size) + 1
    runner = ModelRunner.create(model, num_pages=pages, page_size=block_size, max_requests=2)
    g = torch.Generator().manual_seed(1)
    ids = torch.randint(0, model.plan.embedding.vocab_size, (tokens,), generator=g).tolist()
    times = []
    for i in range(repeats + warm):     # the first runs find the clocks low and the library's products unchosen
        runner.open("p")
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        runner.step([StepEntry("p", ids, [tokens - 1])])
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        runner.close("p")
        if i >= warm:
            times.append(dt)
    del runner
    torch.cuda.empty_cache()
    return sum(times) / len(times), min(times)


def measure_mixed_step(model, block_size: int, prompt_rows: int = 512, decoding: int = 64, context: int = 2048,
                       repeats: int = 5):
    """One step of `prompt_rows` rows of a prompt beside `decoding` decoded tokens of requests that hold
    `context` tokens each: (mean seconds, share of the time that is the library's products)."""
    import torch

    from wllm_amd.engine import ModelRunner, StepEntry
    from wllm_amd.kernels import ops
    pages = decoding * (-(-(context + repeats + 4) // block_size)) + (-(-(prompt_rows * (repeats + 3)) // block_size)) + 2
    runner = ModelRunner.create(model, num_pages=pages, page_size=block_size, max_requests=decoding + 1)
    g = torch.Generator().manual_seed(3)
    vocab = model.plan.embedding.vocab_size
    for i in range(decoding):
        runner.open(i)
        for p in range(0, context, 2048):
            runner.step([StepEntry(i, torch.randint(0, vocab, (min(2048, context - p),), generator=g).tolist(), [])])
    runner.open("p")
    backend = ops.backend()
    times, library = [], []
    for i in range(repeats + 2):
        entries = [StepEntry(r, [int(torch.randint(0, vocab, (1,), generator=g))], [0]) for r in range(decoding)]
        entries.append(StepEntry("p", torch.randint(0, vocab, (prompt_rows,), generator=g).tolist(), []))
        backend.library_events = [] if i >= 2 else None
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        runner.step(entries)
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        if i >= 2:
            times.append(dt)
            library.append(sum(a.elapsed_time(b) for a, b in backend.library_events) / 1000.0)
        backend.library_events = None
    del runner
    torch.cuda.empty_cache()
    mean = sum(times) / len(times)
    return mean, (sum(library) / len(library)) / mean


def measure_decode(model, batch: int, context: int, steps: int, warmup: int, block_size: int, hip_graphs: bool,
                   chunk: int = 2048):
    """Returns (seconds for `steps` steps, mean context length during them)."""
    import torch

    from wllm_amd.engine import ModelRunner, Request, Scheduler
    # requests admitted first decode while the later ones are still prefilled, one portion of a prompt a step
    total_new = batch * (-(-context // chunk)) + warmup + steps + 2
    pages = batch * (-(-(context + total_new) // block_size)) + 2
    runner = ModelRunner.create(model, num_pages=pages, page_size=block_size, max_requests=batch)
    if hip_graphs and hasattr(runner, "enable_graphs"):
        runner.enable_graphs()
    sched = Scheduler(runner, max_prefill_tokens_per_step=chunk, compute_logprobs=False, lookahead=True)
    g = torch.Generator().manual_seed(2)
    vocab = model.plan.embedding.vocab_size
    for i in range(batch):
        sched.add_request(Request(i, torch.randint(0, vocab, (context,), generator=g).tolist(), total_new))
    while sched.waiting or any(r.status.value != "running" for r in sched.running):
        sched.step()
    for _ in range(warmup):
        sched.step()
    assert len(sched.running) == batch and all(r.status.value == "running" for r in sched.running)
    len_before = sum(r.num_computed for r in sched.running) / batch
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        sched.step()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    assert len(sched.running) == batch, "a request finished inside the timed steps"
    mean_ctx = (len_before + sum(r.num_computed for r in sched.running) / batch) / 2.0
    del sched, runner
    torch.cuda.empty_cache()
    return dt, mean_ctx


class _StressDefaults:
    """The stress workload's options as the default line runs it."""
    seed, stress_requests, block_size, stress_pool_fraction, no_graphs, row_multiple = 0, 64, 16, 0.5, False, 256
    dtype, shape = "bf16", "gemma-2b"


def run_stress(model, args) -> dict:
    """Continuous batching under pressure: 64 requests at once, prompt lengths uniform in
    [128, 4096], output lengths uniform in [16, 512] (seeded), prompt portions of at most 512
    tokens a step beside the decoding requests, temperature 0.7 with per-request seeds, and a page
    pool too small for all requests together, so that some wait for admission."""
    import numpy as np
    import torch

    from wllm_amd.engine import ModelRunner, Request, Scheduler
    from wllm_amd.sampling import SamplingParams
    rng = np.random.default_rng(args.seed)
    n = args.stress_requests
    prompts = rng.integers(128, 4097, size=n)
    outputs = rng.integers(16, 513, size=n)
    vocab = model.plan.embedding.vocab_size
    need = int(sum(-(-(int(p) + int(o)) // args.block_size) for p, o in zip(prompts, outputs)))
    pages = max(int(need * args.stress_pool_fraction), -(-4608 // args.block_size) + 1)
    runner = ModelRunner.create(model, num_pages=pages, page_size=args.block_size, max_requests=n)
    if not args.no_graphs:
        runner.enable_graphs()
    sched = Scheduler(runner, max_prefill_tokens_per_step=512, seed=args.seed, lookahead=True,
                      row_multiple=args.row_multiple or None)
    for i in range(n):
        ids = rng.integers(0, vocab, size=int(prompts[i])).tolist()
        sched.add_request(Request(i, ids, int(outputs[i]), sampling_params=SamplingParams(temperature=0.7, seed=1000 + i)))
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    finished = sched.run_to_completion()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    runner.cache.check()
    generated = sum(len(r.output_token_ids) for r in finished)
    assert len(finished) == n and generated == int(outputs.sum())
    sizes = {"gemma-2b": "Gemma-2B", "gemma-7b": "Gemma-7B"}.get(args.shape, os.path.basename(args.shape))
    return {"metric": f"continuous-batching stress, {sizes} layer sizes", "value": round(generated / dt, 1),
            "unit": "generated tokens/s", "seconds": round(dt, 3), "requests": n, "steps": sched.stats["steps"],
            "prompt_tokens": int(prompts.sum()), "generated_tokens": generated,
            "total_tokens_per_s": round((generated + int(prompts.sum())) / dt, 1),
            "pool_pages": pages, "pages_all_requests_need": need, "peak_pages": sched.stats["peak_pages"],
            "admission_waits": sched.stats["admission_waits"], "preemptions": sched.stats["preemptions"],
            "graph_steps": runner.graph_steps, "dtype": args.dtype}


def main() -> int:
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=64)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--context", type=int, default=2048, help="prompt length of every request")
    ap.add_argument("--prefill-tokens", type=int, default=2048)
    ap.add_argument("--dtype", default="bf16", choices=["bf16", "fp32"])
    ap.add_argument("--shape", default="gemma-2b", help="a named layer shape or a config.json")
    ap.add_argument("--layers", type=int, default=None, help="run fewer layers than the shape has")
    ap.add_argument("--block-size", type=int, default=16)
    ap.add_argument("--no-graphs", action="store_true", help="do not replay captured graphs for decode")
    ap.add_argument("--no-points", action="store_true", help="skip every point beside the line's own batch")
    ap.add_argument("--points", default="all", choices=["basic", "all"],
                    help="basic: batch 1 and 64 and the long context; all (default): also batch 128 and 256, batch 64 at "
                         "longer contexts, the stress workload, float32 decoding and the Gemma-7B layer sizes")
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--workload", default="decode", choices=["decode", "stress"],
                    help="decode: the contract's line; stress: continuous batching of 64 mixed requests")
    ap.add_argument("--stress-requests", type=int, default=64)
    ap.add_argument("--row-multiple", type=int, default=256,
                    help="stress: a step's rows are trimmed to a multiple of this where the budget cuts a portion (0: off)")
    ap.add_argument("--stress-pool-fraction", type=float, default=0.5,
                    help="page pool as a fraction of what all requests together would need")
    args = ap.parse_args()
    world = int(os.environ.get("WORLD_SIZE", "1"))
    if args.gpus != 1 or world != 1:
        if int(os.environ.get("RANK", "0")) == 0:
            print(f"bench.py: this engine runs on one GPU; --gpus {args.gpus} (world size {world}) is not supported")
        return 2

    import torch

    import wllm_amd  # noqa: F401
    from wllm_amd.cli import read_shape
    from wllm_amd.kernels import ops

    ops.backend()
    shape = read_shape(args.shape)
    full_layers = shape["num_hidden_layers"]
    if args.layers is not None:
        shape["num_hidden_layers"] = args.layers
    with torch.inference_mode():
        model = build_model(shape, args.dtype, args.seed)
        if args.workload == "stress":
            print(json.dumps(run_stress(model, args)))
            return 0
        graphs = not args.no_graphs
        points = {}

        def decode_point(name, m, b, context, k, warm, dtype):
            """A decode point: tokens a second, milliseconds a step, and the share of HBM's peak that the
            bytes the step has to read (every weight once, the live requests' cache) make of its time."""
            d, ctx_len = measure_decode(m, b, context, k, warm, args.block_size, graphs)
            gbs = (m.weight_bytes() + b * ctx_len * kv_bytes_per_token(m)) / (d / k) / 1e9
            if name is not None:
                points[name] = round(k * b / d, 1)
                points[name + "_ms"] = round(1000.0 * d / k, 4)
                points[name + "_frac"] = round(gbs / PEAK_HBM_GBS, 4)
            return d, gbs

        def prefill_point(name, m, tokens, dtype, repeats=4):
            mean, best = measure_prefill(m, tokens, args.block_size, repeats=repeats)
            points[name] = round(tokens / mean, 1)
            points[name + "_ms"] = round(1000.0 * mean, 3)
            points[name + "_frac"] = round(step_flops(m, tokens, 0, 1) / mean / PEAK_FLOPS[dtype], 4)

        t_prefill, t_prefill_best = measure_prefill(model, args.prefill_tokens, args.block_size)
        prefill_flops = step_flops(model, args.prefill_tokens, 0, 1)

        dt, achieved = decode_point(None, model, args.batch, args.context, args.steps, args.warmup, args.dtype)
        ms_per_step = 1000.0 * dt / args.steps
        value = args.steps * args.batch / dt

        limit = model.plan.max_positions
        if not args.no_points:
            few = min(args.warmup, 4)
            half = max(8, args.steps // 2)
            decode_point("decode_b1", model, 1, args.context, args.steps, few, args.dtype)
            decode_point("decode_b64", model, 64, args.context, half, few, args.dtype)
            # the same batch near the longest context the configuration allows
            new_tokens = args.batch * (-(-limit // 2048)) + args.warmup + args.steps + 2      # as `measure_decode` counts them
            long_context = min(limit - 1024, (limit - new_tokens) // 256 * 256)
            if long_context > args.context:
                decode_point(f"decode_b{args.batch}_context_{long_context}", model, args.batch, long_context, args.steps, few,
                             args.dtype)
            if args.points == "all":
                # further batch sizes, context lengths and prompt lengths of the same configuration
                decode_point("decode_b128", model, 128, args.context, half, few, args.dtype)
                decode_point("decode_b256", model, 256, args.context, half, few, args.dtype)
                for context in (4096, long_context):
                    if args.context < context <= limit - 1024:
                        decode_point(f"decode_b64_context_{context}", model, 64, context, half, few, args.dtype)
                for tokens in (512, 4096, 8192):
                    if tokens <= limit and tokens != args.prefill_tokens:
                        prefill_point(f"prefill_{tokens}", model, tokens, args.dtype)
                # a step of a prompt's portion beside decoded tokens, and the library's share of it
                mixed, share = measure_mixed_step(model, args.block_size)
                points["mixed_512_rows_beside_64_decoded_ms"] = round(1000.0 * mixed, 3)
                points["mixed_step_library_products_share"] = round(share, 3)
                if args.dtype == "bf16" and args.shape == "gemma-2b" and args.layers is None:
                    # the continuous-batching stress workload on the same model: generated tokens a second
                    stress = run_stress(model, _StressDefaults)
                    points["stress_generated_tokens_per_s"] = stress["value"]
                    points["stress_seconds"] = stress["seconds"]
        plan = model.plan
        layers_run = len(plan.schedule)
        weight_bytes = model.weight_bytes()
        if not args.no_points and args.points == "all" and args.dtype == "bf16" and args.shape == "gemma-2b" and args.layers is None:
            # the other measured configurations, each with all its layers: the true 32-bit path of the same
            # sizes, and the Gemma-7B layer sizes
            del model
            torch.cuda.empty_cache()
            other = build_model(shape, "fp32", args.seed)
            decode_point(f"fp32_decode_b{args.batch}", other, args.batch, args.context, half, 2, "fp32")
            prefill_point(f"fp32_prefill_{args.prefill_tokens}", other, args.prefill_tokens, "fp32", repeats=2)
            del other
            torch.cuda.empty_cache()
            other = build_model(read_shape("gemma-7b"), "bf16", args.seed)
            for b, k in ((1, half), (8, half), (64, max(8, half // 2))):
                decode_point(f"gemma7b_decode_b{b}", other, b, args.context, k, 2, "bf16")
            prefill_point(f"gemma7b_prefill_{args.prefill_tokens}", other, args.prefill_tokens, "bf16", repeats=3)
            del other
            torch.cuda.empty_cache()

    c = shape
    sizes = {"gemma-2b": "Gemma-2B", "gemma-7b": "Gemma-7B"}.get(args.shape, os.path.basename(args.shape))
    line = {
        "metric": f"decode tokens/s, {sizes} layer sizes, after {args.context:,}-token prompts",
        "value": round(value, 1),
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": args.dtype,
        "data": "synthetic: seeded random weights (normal, std 0.02) and seeded uniform token ids",
        "config": {
            "model": f"{sizes} layer sizes ({c['architectures'][0]}), random weights",
            "global_batch": args.batch, "seq_len": args.context, "parallelism": "single GPU",
            "layers": layers_run, "layers_of_full_model": full_layers, "hidden_size": plan.embedding.hidden_size,
            "intermediate_size": c.get("intermediate_size"), "num_attention_heads": c.get("num_attention_heads"),
            "num_key_value_heads": c.get("num_key_value_heads", c.get("num_attention_heads")), "head_dim": c.get("head_dim"),
            "vocab_size": plan.embedding.vocab_size, "tied_embeddings": plan.head.weight is None,
            "rope_theta": c.get("rope_theta", 10000.0), "rms_norm_eps": c.get("rms_norm_eps", 1e-6),
            "max_position_embeddings": limit, "kv_block_size": args.block_size,
            "sampling": "greedy", "hip_graphs": graphs, "lookahead": True,
        },
        "prefill": {"value": round(args.prefill_tokens / t_prefill, 1), "tokens": args.prefill_tokens,
                    "ms": round(1000.0 * t_prefill, 3), "ms_mean": round(1000.0 * t_prefill, 3),
                    "ms_best": round(1000.0 * t_prefill_best, 3),
                    "frac": round(prefill_flops / t_prefill / PEAK_FLOPS[args.dtype], 4)},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                     "frac": round(achieved / PEAK_HBM_GBS, 4),
                     "bytes_per_step": int(achieved * 1e9 * dt / args.steps), "weight_bytes": weight_bytes},
        "points": points,
    }
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())
