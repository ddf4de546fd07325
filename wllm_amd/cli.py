"""Command line.  Options carry the reference's names and meanings where it has them
(src/wllm/cli.py:21-56): --model, --device, --dtype, --num-blocks, --block-size,
--chunked-prefill-tokens, --cuda-graphs (also spelled --hip-graphs here).  The reference's command
starts a server; this engine is token ids in, token ids out, so the commands are

    python -m wllm_amd.cli generate --model DIR --prompt-ids 5,17,3 [--prompt-ids ...]
    python -m wllm_amd.cli random-model --out DIR --config NAME|FILE --seed N
    python -m wllm_amd.cli bench-decode --model DIR 1,8,64      (the reference's table,
                                                                 scripts/benchmark_decode.py:78-93)
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

SHAPES_DIR = os.path.join(os.path.dirname(os.path.abspath(__file__)), "config", "shapes")


def named_shapes() -> list:
    """Layer shapes one can ask for by name in `random-model`: config.json files kept as data."""
    return sorted(f[:-5] for f in os.listdir(SHAPES_DIR) if f.endswith(".json"))


def read_shape(name_or_file: str) -> dict:
    path = os.path.join(SHAPES_DIR, name_or_file + ".json") if name_or_file in named_shapes() else name_or_file
    with open(path, "r", encoding="utf-8") as f:
        return json.load(f)


def _engine_options(ap: argparse.ArgumentParser) -> None:
    ap.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    ap.add_argument("--device", default="cuda", choices=["cuda"], help="the engine runs on the GPU only")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--num-blocks", type=int, default=256, help="KV cache blocks (block_size tokens each)")
    ap.add_argument("--block-size", type=int, default=16)
    # the reference's name for the option (src/wllm/cli.py:21-56) and this engine's
    ap.add_argument("--cuda-graphs", "--hip-graphs", dest="hip_graphs", action="store_true",
                    help="replay captured HIP graphs for decode steps")
    ap.add_argument("--chunked-prefill-tokens", type=int, default=None,
                    help="max prompt tokens processed per scheduler step (enables chunked prefill)")


def _llm(args):
    from wllm_amd.engine.llm import LLM
    return LLM(args.model, dtype=args.dtype, device=args.device, num_blocks=args.num_blocks,
               block_size=args.block_size, max_prefill_tokens_per_step=args.chunked_prefill_tokens,
               hip_graphs=args.hip_graphs, seed=getattr(args, "seed", 0) or 0)


def cmd_generate(args) -> int:
    from wllm_amd.sampling import SamplingParams
    prompts = [[int(t) for t in p.split(",") if t.strip()] for p in (args.prompt_ids or [])]
    if args.prompt_file:
        with open(args.prompt_file, "r", encoding="utf-8") as f:
            for line in f:
                line = line.strip()
                if line:
                    prompts.append([int(t) for t in json.loads(line)] if line.startswith("[")
                                   else [int(t) for t in line.replace(",", " ").split()])
    if not prompts:
        print("generate: give --prompt-ids or --prompt-file", file=sys.stderr)
        return 2
    sp = SamplingParams(temperature=args.temperature, top_k=args.top_k, top_p=args.top_p, min_p=args.min_p,
                        repetition_penalty=args.repetition_penalty, seed=args.seed)
    llm = _llm(args)
    stops = [int(t) for t in (args.stop_token_ids or "").split(",") if t.strip()]
    outs = llm.generate(prompts, sp, max_new_tokens=args.max_new_tokens, eos_token_id=args.eos_token_id,
                        stop_token_ids=stops)
    for o in outs:
        print(json.dumps({"prompt_token_ids": o.prompt_token_ids, "token_ids": o.token_ids,
                          "finish_reason": o.finish_reason}))
    return 0


def cmd_random_model(args) -> int:
    import torch

    from wllm_amd.parts import write_random_model_from_config_json
    raw = read_shape(args.config)
    if args.num_hidden_layers is not None:
        raw["num_hidden_layers"] = args.num_hidden_layers
    store = {"bfloat16": torch.bfloat16, "float32": torch.float32}[args.store_dtype]
    # the architecture named in the file parses and checks its own keys
    write_random_model_from_config_json(args.out, raw, args.seed, std=args.std, norm_std=args.norm_std,
                                        store_dtype=store)
    print(f"wrote {args.out}")
    return 0


def cmd_bench_decode(args) -> int:
    """Decode throughput by batch size, measured as the reference measures it
    (scripts/benchmark_decode.py:52-75): identical prompts, warm-up steps, then timed steps
    between device synchronisations, tokens/sec = steps * batch / elapsed."""
    import torch

    from wllm_amd.engine.request import Request
    llm = None
    sizes = [int(b) for b in args.batch_sizes.split(",")]
    print(f"{'batch_size':>10} | {'tokens/sec':>12} | {'ms/token (per-seq)':>20}")
    print("-" * 48)
    for b in sizes:
        args.num_blocks = b * (-(-(args.prompt_len + args.steps + args.warmup + 1) // args.block_size) + 1)
        llm = _llm(args)
        vocab = llm.model.plan.embedding.vocab_size
        g = torch.Generator().manual_seed(0)
        prompt = torch.randint(0, vocab, (args.prompt_len,), generator=g).tolist()
        for i in range(b):
            llm.scheduler.add_request(Request(i, prompt, args.steps + args.warmup + 1))
        while any(r.status.value != "running" for r in llm.scheduler.running) or llm.scheduler.waiting:
            llm.scheduler.step()
        for _ in range(args.warmup):
            llm.scheduler.step()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps - 1):
            llm.scheduler.step()
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        tps = (args.steps - 1) * b / dt
        print(f"{b:>10} | {tps:>12.1f} | {1000.0 * b / tps:>20.2f}")
        del llm
        torch.cuda.empty_cache()
    return 0


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog="wllm_amd", description="Gemma inference engine for one MI355X")
    sub = ap.add_subparsers(dest="command", required=True)

    g = sub.add_parser("generate", help="generate token ids for prompts given as token ids")
    _engine_options(g)
    g.add_argument("--prompt-ids", action="append", help="comma-separated token ids; may be repeated")
    g.add_argument("--prompt-file", help="one prompt per line: a JSON list or ids separated by spaces or commas")
    g.add_argument("--max-new-tokens", type=int, default=16)
    g.add_argument("--temperature", type=float, default=0.0, help="0 is greedy")
    g.add_argument("--top-k", type=int, default=0)
    g.add_argument("--top-p", type=float, default=1.0)
    g.add_argument("--min-p", type=float, default=0.0)
    g.add_argument("--repetition-penalty", type=float, default=1.0)
    g.add_argument("--seed", type=int, default=None)
    g.add_argument("--eos-token-id", type=int, default=None)
    # the reference's finishing rule takes a set of stop tokens beside the end token (src/wllm/engine/sequence.py:53-59)
    g.add_argument("--stop-token-ids", default=None, help="comma-separated token ids that end a request (the token is kept)")
    g.set_defaults(func=cmd_generate)

    r = sub.add_parser("random-model", help="write a model folder with seeded random weights")
    r.add_argument("--out", required=True)
    r.add_argument("--config", required=True, help=f"one of {named_shapes()} or a config.json")
    r.add_argument("--seed", type=int, default=0)
    r.add_argument("--std", type=float, default=0.02)
    r.add_argument("--norm-std", type=float, default=0.1)
    r.add_argument("--num-hidden-layers", type=int, default=None, help="override the number of layers")
    r.add_argument("--store-dtype", default="bfloat16", choices=["bfloat16", "float32"])
    r.set_defaults(func=cmd_random_model)

    b = sub.add_parser("bench-decode", help="decode tokens/sec by batch size")
    _engine_options(b)
    b.add_argument("batch_sizes", nargs="?", default="1,2,4,8,16,32", help="comma-separated batch sizes")
    b.add_argument("--prompt-len", type=int, default=64)
    b.add_argument("--steps", type=int, default=64)
    b.add_argument("--warmup", type=int, default=8)
    b.set_defaults(func=cmd_bench_decode)

    args = ap.parse_args(argv)
    return args.func(args)


if __name__ == "__main__":
    sys.exit(main())
