"""A plain, slow Gemma-1 forward pass: whole sequences, no cache, no batching.

Written from the formulas of the reference (Sehastrajit-S/wLLM); every function
cites the file and lines it follows.  It is the oracle of the test-suite and
shares no code with the engine: it reads config.json and model.safetensors with
the `json` module and the `safetensors` package, and computes with ordinary
torch tensor arithmetic in one floating-point type (float32, or float64 to
calibrate tolerances).

The reference is read, not run.
"""
from __future__ import annotations

import json
import math
import os

import torch
from safetensors import safe_open


# --------------------------------------------------------------------------
# model folder
# --------------------------------------------------------------------------

def read_config(folder: str) -> dict:
    """The keys and defaults of `ModelConfig.from_json`
    (src/wllm/models/config.py:38-71), except that `tie_word_embeddings`
    absent means tied, which is what a Gemma-1 checkpoint is.
    """
    with open(os.path.join(folder, "config.json"), "r", encoding="utf-8") as f:
        raw = json.load(f)
    rope_theta = raw.get("rope_theta")
    if rope_theta is None:
        rope_theta = raw.get("rope_parameters", {}).get("rope_theta", 10000.0)  # config.py:43-45
    heads = raw["num_attention_heads"]
    head_dim = raw.get("head_dim")
    if head_dim is None:
        head_dim = raw["hidden_size"] // heads  # config.py:32-36
    bias = raw.get("attention_bias")
    if bias is None:
        bias = raw.get("model_type") == "qwen2"  # config.py:54-56
    return {
        "vocab_size": raw["vocab_size"],
        "hidden_size": raw["hidden_size"],
        "intermediate_size": raw["intermediate_size"],
        "num_hidden_layers": raw["num_hidden_layers"],
        "num_attention_heads": heads,
        "num_key_value_heads": raw.get("num_key_value_heads", heads),  # config.py:64
        "head_dim": head_dim,
        "rms_norm_eps": raw.get("rms_norm_eps", 1e-6),  # config.py:65
        "rope_theta": float(rope_theta),
        "tie_word_embeddings": raw.get("tie_word_embeddings", True),
        "attention_bias": bool(bias),
    }


def read_weights(folder: str, dtype: torch.dtype = torch.float32) -> dict:
    """Every tensor of model.safetensors by its name, converted to `dtype`
    (src/wllm/models/llama.py:640-642 merges the files into one dict of names).
    """
    out = {}
    with safe_open(os.path.join(folder, "model.safetensors"), framework="pt", device="cpu") as f:
        for name in f.keys():
            out[name] = f.get_tensor(name).to(dtype)
    return out


# --------------------------------------------------------------------------
# parts, one function each
# --------------------------------------------------------------------------

def embed(ids: torch.Tensor, table: torch.Tensor, hidden_size: int,
          scale_rounding: torch.dtype | None = None) -> torch.Tensor:
    """x = E[ids] * sqrt(hidden_size)  (src/wllm/models/llama.py:399-403,
    src/wllm/models/gemma.py:158-162).  The factor is a buffer that the
    reference casts to the model's dtype with the rest of the model
    (llama.py:397,651); `scale_rounding` names that dtype when it is narrower
    than the one computed in here (bfloat16: sqrt(2048) becomes 45.25).
    """
    scale = torch.tensor(hidden_size ** 0.5, dtype=torch.float32)
    if scale_rounding is not None:
        scale = scale.to(scale_rounding)
    return table[ids] * scale.to(table.dtype)


def rms_norm_one_plus_w(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    """h = x * rsqrt(mean(x^2) + eps) * (1 + w)  (src/wllm/models/gemma.py:41-51)."""
    variance = x.pow(2).mean(-1, keepdim=True)
    x = x * torch.rsqrt(variance + eps)
    return x * (1.0 + w)


def rope_cos_sin(positions: torch.Tensor, head_dim: int, theta: float,
                 dtype: torch.dtype) -> tuple[torch.Tensor, torch.Tensor]:
    """inv_freq[j] = 1 / theta^(2j/d); angles = pos * inv_freq; the table is the
    angles twice side by side (src/wllm/models/llama.py:52-62).  The reference
    builds inv_freq and the angles in float32; float64 is used here only when
    the whole oracle runs in float64.
    """
    base = torch.float64 if dtype == torch.float64 else torch.float32
    inv_freq = 1.0 / (theta ** (torch.arange(0, head_dim, 2, dtype=base) / head_dim))
    freqs = positions.to(base)[:, None] * inv_freq[None, :]
    emb = torch.cat((freqs, freqs), dim=-1)
    return emb.cos().to(dtype), emb.sin().to(dtype)


def rotate_half(x: torch.Tensor) -> torch.Tensor:
    """(x1, x2) -> (-x2, x1) on the two halves of the last axis
    (src/wllm/models/llama.py:47-49)."""
    x1, x2 = x.chunk(2, dim=-1)
    return torch.cat((-x2, x1), dim=-1)


def apply_rope(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> torch.Tensor:
    """x' = x*cos + rotate_half(x)*sin; x is [tokens, heads, d], cos/sin [tokens, d]
    (src/wllm/models/llama.py:65-71)."""
    return x * cos[:, None, :] + rotate_half(x) * sin[:, None, :]


def causal_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor,
                     head_dim: int) -> torch.Tensor:
    """q [T, nh, d], k/v [T, nkv, d] of one sequence.  Query head h reads KV
    head h // (nh // nkv) (src/wllm/models/llama.py:74-79,
    src/wllm/kernels/csrc/paged_attention.cu:44-45); scores are scaled by
    1/sqrt(head_dim) (llama.py:242; SDPA's default at llama.py:112); the query
    at position p sees keys 0..p (llama.py:112,190-192); softmax over the keys,
    then the weighted sum of v.
    """
    T, nh, d = q.shape
    nkv = k.shape[1]
    n_rep = nh // nkv
    k = k.repeat_interleave(n_rep, dim=1)
    v = v.repeat_interleave(n_rep, dim=1)
    scores = torch.einsum("qhd,khd->hqk", q, k) * (1.0 / math.sqrt(head_dim))
    allowed = torch.ones(T, T, dtype=torch.bool).tril()
    scores = scores.masked_fill(~allowed[None, :, :], float("-inf"))
    probs = torch.softmax(scores, dim=-1)
    return torch.einsum("hqk,khd->qhd", probs, v)


def gelu_tanh(z: torch.Tensor) -> torch.Tensor:
    """0.5 z (1 + tanh(sqrt(2/pi) (z + 0.044715 z^3))): what
    F.gelu(approximate="tanh") computes (src/wllm/models/gemma.py:62)."""
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z.pow(3))))


def geglu_mlp(h: torch.Tensor, w_gate: torch.Tensor, w_up: torch.Tensor,
              w_down: torch.Tensor) -> torch.Tensor:
    """down(gelu_tanh(gate(h)) * up(h)), no biases (src/wllm/models/gemma.py:54-62)."""
    return (gelu_tanh(h @ w_gate.T) * (h @ w_up.T)) @ w_down.T


def attention_block(h: torch.Tensor, weights: dict, prefix: str, cfg: dict,
                    cos: torch.Tensor, sin: torch.Tensor) -> torch.Tensor:
    """q/k/v projections (with bias only if attention_bias), views into heads,
    rotation of q and k, causal attention, output projection without bias
    (src/wllm/models/llama.py:95-115)."""
    nh, nkv, d = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"]
    T = h.shape[0]
    q = h @ weights[prefix + "q_proj.weight"].T
    k = h @ weights[prefix + "k_proj.weight"].T
    v = h @ weights[prefix + "v_proj.weight"].T
    if cfg["attention_bias"]:
        q = q + weights[prefix + "q_proj.bias"]
        k = k + weights[prefix + "k_proj.bias"]
        v = v + weights[prefix + "v_proj.bias"]
    q = apply_rope(q.view(T, nh, d), cos, sin)
    k = apply_rope(k.view(T, nkv, d), cos, sin)
    o = causal_attention(q, k, v.view(T, nkv, d), d)
    return o.reshape(T, nh * d) @ weights[prefix + "o_proj.weight"].T


def decoder_layer(x: torch.Tensor, weights: dict, i: int, cfg: dict,
                  cos: torch.Tensor, sin: torch.Tensor) -> torch.Tensor:
    """norm, attention, residual; norm, feed-forward, residual
    (src/wllm/models/gemma.py:83-93)."""
    p = f"model.layers.{i}."
    eps = cfg["rms_norm_eps"]
    h = rms_norm_one_plus_w(x, weights[p + "input_layernorm.weight"], eps)
    x = x + attention_block(h, weights, p + "self_attn.", cfg, cos, sin)
    h = rms_norm_one_plus_w(x, weights[p + "post_attention_layernorm.weight"], eps)
    return x + geglu_mlp(h, weights[p + "mlp.gate_proj.weight"], weights[p + "mlp.up_proj.weight"],
                         weights[p + "mlp.down_proj.weight"])


def forward_logits(cfg: dict, weights: dict, ids, positions=None,
                   scale_rounding: torch.dtype | None = None) -> torch.Tensor:
    """Logits [T, vocab] of one whole sequence (src/wllm/models/llama.py:405-415,
    432-446): embed and scale, positions 0..T-1 (`positions` moves them all, for
    the test that only distances count), the layers in order, the final norm,
    and the head: the embedding table itself, unscaled, when tied.
    """
    ids = torch.as_tensor(ids, dtype=torch.long)
    table = weights["model.embed_tokens.weight"]
    dtype = table.dtype
    x = embed(ids, table, cfg["hidden_size"], scale_rounding)
    if positions is None:
        positions = torch.arange(ids.shape[0])
    cos, sin = rope_cos_sin(torch.as_tensor(positions), cfg["head_dim"], cfg["rope_theta"], dtype)
    for i in range(cfg["num_hidden_layers"]):
        x = decoder_layer(x, weights, i, cfg, cos, sin)
    x = rms_norm_one_plus_w(x, weights["model.norm.weight"], cfg["rms_norm_eps"])
    head = table if cfg["tie_word_embeddings"] else weights["lm_head.weight"]
    return x @ head.T


def generate_greedy(cfg: dict, weights: dict, prompt: list[int], max_new_tokens: int,
                    scale_rounding: torch.dtype | None = None) -> list[int]:
    """Full recomputation at every token, argmax of the last row
    (src/wllm/models/llama.py:599-610)."""
    tokens = list(prompt)
    for _ in range(max_new_tokens):
        logits = forward_logits(cfg, weights, tokens, scale_rounding=scale_rounding)
        tokens.append(int(logits[-1].argmax()))
    return tokens[len(prompt):]
