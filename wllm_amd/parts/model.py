"""The generic causal language model, assembled from a ModelPlan.

It owns the embedding, the layers (built once each, even when the schedule names
one several times), the final norm and the head, and runs them over a step's
flat batch in the order the plan's schedule gives.  It knows no architecture:
`load_model` reads config.json, asks the registry for the architecture's
configuration parser and plan builder, and hands the plan to `CausalLM`.
That is the reference's `load_native` dispatch (src/wllm/models/llama.py:619-653)
with the model class replaced by a plan.
"""
from __future__ import annotations

import math
from typing import Optional

import torch

from wllm_amd.config.registry import read_config_json, resolve_architecture
from wllm_amd.kernels import ops
from wllm_amd.parts.blocks import ResidualStream
from wllm_amd.parts.registry import build_block, build_norm
from wllm_amd.parts.specs import ModelPlan
from wllm_amd.weights.checkpoint import Checkpoint, ExpectedTensor, TensorFetcher, WeightError

DTYPES = {"bfloat16": torch.bfloat16, "float32": torch.float32}


def resolve_dtype(dtype) -> torch.dtype:
    if isinstance(dtype, torch.dtype):
        if dtype not in DTYPES.values():
            raise ValueError(f"dtype {dtype} is not supported; use bfloat16 or float32")
        return dtype
    if dtype not in DTYPES:
        raise ValueError(f"dtype {dtype!r} is not supported; use one of {sorted(DTYPES)}")
    return DTYPES[dtype]


class CausalLM:
    def __init__(self, plan: ModelPlan, config=None):
        self.plan = plan
        self.config = config
        self.blocks = [build_block(spec) for spec in plan.layers]
        self.final_norm = build_norm(plan.final_norm)
        self.embed_table: Optional[torch.Tensor] = None
        self.head_weight: Optional[torch.Tensor] = None
        self.embed_scale: float = plan.embedding.scale
        self.dtype: Optional[torch.dtype] = None
        self.device = None

    # ---- what the model needs from the cache manager ---------------------------
    def cache_needs(self) -> dict:
        """{schedule entry: CacheNeed} for the entries that own a cache."""
        needs = {}
        for i, e in enumerate(self.plan.schedule):
            if e.reads_cache_of is not None:
                continue
            need = self.blocks[e.layer].mixer.cache_need()
            if need is not None:
                needs[i] = need
        for i, e in enumerate(self.plan.schedule):
            if e.reads_cache_of is not None:
                mine = self.blocks[e.layer].mixer.cache_need()
                theirs = needs.get(e.reads_cache_of)
                if mine is None or theirs is None or type(mine) is not type(theirs) \
                        or mine.page_shape(1) != theirs.page_shape(1):
                    raise ValueError(f"schedule entry {i} cannot read the cache of entry {e.reads_cache_of}: shapes differ")
        return needs

    def state_shapes(self) -> dict:
        shapes = {}
        for i, e in enumerate(self.plan.schedule):
            shape = self.blocks[e.layer].mixer.state_shape()      # a shape (float32) or a StateNeed
            if shape is not None:
                shapes[i] = shape
        return shapes

    def graph_capturable(self) -> bool:
        """True if every part runs from the step's device arrays alone, so that a step can be
        captured once and replayed with other contents.  A mixer says so with an attribute."""
        return all(getattr(b.mixer, "graph_capturable", False) for b in self.blocks)

    # ---- weights ---------------------------------------------------------------
    def expected_tensors(self) -> dict:
        emb, head = self.plan.embedding, self.plan.head
        out = {emb.weight: ExpectedTensor((emb.vocab_size, emb.hidden_size))}
        for block in self.blocks:
            for part in block.parts():
                out.update(part.expected_tensors())
        out.update(self.final_norm.expected_tensors())
        if head.weight is not None:
            out[head.weight] = ExpectedTensor((head.vocab_size, head.hidden_size))
        return out

    def load(self, checkpoint: Checkpoint, dtype: torch.dtype, device, tiled_copies: bool = False) -> None:
        """`tiled_copies`: keep, beside each bfloat16 matrix, a copy in the order the few-row product
        kernels read fastest (decode steps run about a third faster; the matrices take twice the memory)."""
        emb, head = self.plan.embedding, self.plan.head
        # a tied checkpoint may still carry the head; it is accepted if it is the table
        extra = ()
        tied_head_name = head.tied_checkpoint_name
        if head.weight is None and tied_head_name is not None and tied_head_name in checkpoint:
            extra = (tied_head_name,)
        checkpoint.check(self.expected_tensors(), self.plan.ignored_tensor_suffixes, allowed_extra=extra)
        fetch = TensorFetcher(checkpoint, dtype, device, tiled_copies=tiled_copies)
        if extra:
            table = fetch.matrix(emb.weight)
            if checkpoint.shape(tied_head_name) != tuple(table.shape) or not torch.equal(
                    fetch.matrix(tied_head_name), table):
                raise WeightError(f"{tied_head_name} is stored although the embeddings are tied, and differs from "
                                  f"{emb.weight}", unexpected=[tied_head_name])
        self.load_from(fetch)

    def load_from(self, fetch) -> None:
        """Loads every part through a fetcher: an object with `matrix(name)`, `vector(name)`,
        `table(name)`, `to_device(tensor)`, `has(name)` and the attributes `dtype`, `device`."""
        emb, head = self.plan.embedding, self.plan.head
        dtype, device = fetch.dtype, fetch.device
        self.embed_table = fetch.to_device(fetch.matrix(emb.weight))
        for block in self.blocks:
            for part in block.parts():
                part.load(fetch)
        self.final_norm.load(fetch)
        self.head_weight = self.embed_table if head.weight is None else fetch.to_device(fetch.matrix(head.weight))
        self.head_tiles = ops.tile_weight(self.head_weight) if getattr(fetch, "tiled_copies", False) else None
        scale = emb.scale
        if emb.scale_in_model_dtype:
            scale = float(torch.tensor(scale, dtype=torch.float32).to(dtype).to(torch.float32))
        self.embed_scale = scale
        self.dtype, self.device = dtype, device

    def weight_bytes(self) -> int:
        """Bytes of every weight a step reads once (the tied table counts once)."""
        seen, total = set(), 0
        tensors = [self.embed_table if self.head_weight is not self.embed_table else None, self.head_weight,
                   self.final_norm.weight]
        for block in self.blocks:
            for part in block.parts():
                # a tile-major copy (t_*) holds the same numbers as its matrix; a step reads one of the two
                tensors.extend(v for k, v in vars(part).items() if isinstance(v, torch.Tensor) and not k.startswith("t_"))
        for t in tensors:
            if t is not None and t.data_ptr() not in seen:
                seen.add(t.data_ptr())
                total += t.numel() * t.element_size()
        return total

    # ---- one step ----------------------------------------------------------------
    def forward(self, ctx) -> torch.Tensor:
        """Runs the batch of `ctx` through the schedule and returns float32 logits
        [len(ctx.logit_rows), vocab] at the wanted rows (an empty tensor if none)."""
        n, hidden = ctx.n, self.plan.embedding.hidden_size
        x = ctx.buffer("residual", (n, hidden), torch.float32)
        ops.embed_lookup(ctx.token_ids, self.embed_table, self.embed_scale, x)
        stream = ResidualStream(x)
        for entry, e in enumerate(self.plan.schedule):
            self.blocks[e.layer].forward(ctx, entry, stream)
        m = ctx.num_logit_rows
        vocab = self.plan.head.vocab_size
        if m == 0:
            # the pending contribution of the last block is never needed
            return torch.empty((0, vocab), dtype=torch.float32, device=x.device)
        last = stream.normed(self.final_norm, ctx.buffer("final_normed", (m, hidden), self.dtype), rows=ctx.logit_rows)
        logits = ctx.buffer("logits", (m, vocab), torch.float32)
        ops.linear(last, self.head_weight, logits, self.head_tiles)
        return logits


def build_model(raw_config: dict) -> CausalLM:
    entry = resolve_architecture(raw_config.get("architectures"))
    config = entry.parse_config(raw_config)
    return CausalLM(entry.build_plan(config), config)


def load_model(folder: str, dtype="bfloat16", device="cuda", tiled_copies: Optional[bool] = None) -> CausalLM:
    """A model folder (config.json, model.safetensors) to a loaded model.  `tiled_copies` (default:
    yes on a GPU) keeps a second copy of each matrix in the order the few-row product kernels
    of decode steps read fastest, at twice the matrices' memory."""
    dtype = resolve_dtype(dtype)
    model = build_model(read_config_json(folder))
    checkpoint = Checkpoint(folder)
    if tiled_copies is None:
        tiled_copies = torch.device(device).type == "cuda"
    try:
        model.load(checkpoint, dtype, torch.device(device), tiled_copies=tiled_copies)
    finally:
        checkpoint.close()
    return model


def write_random_model_from_config_json(folder: str, raw_config: dict, seed: int, *, std: float = 0.02,
                                        norm_std: float = 0.1, store_dtype: torch.dtype = torch.bfloat16) -> str:
    """The random-weights mode: the contents of a config.json (of any registered architecture) and a
    seed to a model folder.  The configuration is parsed and checked by its architecture; what is
    written as config.json is `raw_config` itself."""
    from wllm_amd.weights.random_init import write_random_model
    model = build_model(raw_config)
    return write_random_model(folder, raw_config, model.expected_tensors(), seed, std=std, norm_std=norm_std,
                              store_dtype=store_dtype)


def write_random_model_folder(folder: str, config, seed: int, *, std: float = 0.02, norm_std: float = 0.1,
                              store_dtype: torch.dtype = torch.bfloat16) -> str:
    """The same from a typed configuration that can write itself as config.json (`to_dict()`)."""
    return write_random_model_from_config_json(folder, config.to_dict(), seed, std=std, norm_std=norm_std,
                                               store_dtype=store_dtype)
