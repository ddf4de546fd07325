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
#
# `round_to` (None, or torch.bfloat16) makes a function round where the reference's model rounds when
# it runs in that dtype: every torch operation of the reference returns a tensor of the model's dtype,
# so the value is rounded there and the arithmetic in here (float64, say) stands for the wider
# arithmetic inside the operation.  The run with `round_to=torch.bfloat16` beside the run without is
# what the tests take their bfloat16 bound from: how far the reference's own bfloat16 model is from
# the exact result.  One thing is left as the formulas intend it: the rotation's frequencies stay
# float32 (the reference's buffer `inv_freq` is cast with the model, src/wllm/models/llama.py:56,651,
# which would move the angles of late positions by whole radians).

def _r(x: torch.Tensor, round_to: torch.dtype | None) -> torch.Tensor:
    return x if round_to is None else x.to(round_to).to(x.dtype)


def embed(ids: torch.Tensor, table: torch.Tensor, hidden_size: int,
          scale_rounding: torch.dtype | None = None, round_to: torch.dtype | None = None) -> torch.Tensor:
    """x = E[ids] * sqrt(hidden_size)  (src/wllm/models/llama.py:399-403,
    src/wllm/models/gemma.py:158-162).  The factor is a buffer that the
    reference casts to the model's dtype with the rest of the model
    (llama.py:397,651); `scale_rounding` names that dtype when it is narrower
    than the one computed in here (bfloat16: sqrt(2048) becomes 45.25).
    """
    scale = torch.tensor(hidden_size ** 0.5, dtype=torch.float32)
    if scale_rounding is not None:
        scale = scale.to(scale_rounding)
    return _r(table[ids] * scale.to(table.dtype), round_to)


def rms_norm_one_plus_w(x: torch.Tensor, w: torch.Tensor, eps: float,
                        round_to: torch.dtype | None = None) -> torch.Tensor:
    """h = x * rsqrt(mean(x^2) + eps) * (1 + w)  (src/wllm/models/gemma.py:41-51).  The reference
    computes it in float32 and casts after the multiplication by (1 + w) (gemma.py:44,51): one rounding."""
    variance = x.pow(2).mean(-1, keepdim=True)
    x = x * torch.rsqrt(variance + eps)
    return _r(x * (1.0 + w), round_to)


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


def apply_rope(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor,
               round_to: torch.dtype | None = None) -> torch.Tensor:
    """x' = x*cos + rotate_half(x)*sin; x is [tokens, heads, d], cos/sin [tokens, d]
    (src/wllm/models/llama.py:65-71).  In a narrower dtype the table is cast to it (llama.py:67-68) and
    each of the two products and their sum is a tensor of its own."""
    cos, sin = _r(cos, round_to), _r(sin, round_to)
    return _r(_r(x * cos[:, None, :], round_to) + _r(rotate_half(x) * sin[:, None, :], round_to), round_to)


def causal_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor,
                     head_dim: int, round_to: torch.dtype | None = None, tamper=None) -> torch.Tensor:
    """q [T, nh, d], k/v [T, nkv, d] of one sequence.  Query head h reads KV
    head h // (nh // nkv) (src/wllm/models/llama.py:74-79,
    src/wllm/kernels/csrc/paged_attention.cu:44-45); scores are scaled by
    1/sqrt(head_dim) (llama.py:242; SDPA's default at llama.py:112); the query
    at position p sees keys 0..p (llama.py:112,190-192); softmax over the keys,
    then the weighted sum of v.  In a narrower dtype the reference's prefill hands tensors of that
    dtype to the library's attention (llama.py:112); what it rounds inside is the library's own
    matter, and is taken here as the common choice: scores and softmax wide, the probabilities
    rounded before the second product, the result rounded.  `tamper(allowed)` may change the
    mask of which key a query sees, for tests that show what a lost or a foreign key does.
    """
    T, nh, d = q.shape
    nkv = k.shape[1]
    n_rep = nh // nkv
    k = k.repeat_interleave(n_rep, dim=1)
    v = v.repeat_interleave(n_rep, dim=1)
    scores = torch.einsum("qhd,khd->hqk", q, k) * (1.0 / math.sqrt(head_dim))
    allowed = torch.ones(T, T, dtype=torch.bool).tril()
    if tamper is not None:
        allowed = tamper(allowed)
    scores = scores.masked_fill(~allowed[None, :, :], float("-inf"))
    probs = _r(torch.softmax(scores, dim=-1), round_to)
    return _r(torch.einsum("hqk,khd->qhd", probs, v), round_to)


def gelu_tanh(z: torch.Tensor) -> torch.Tensor:
    """0.5 z (1 + tanh(sqrt(2/pi) (z + 0.044715 z^3))): what
    F.gelu(approximate="tanh") computes (src/wllm/models/gemma.py:62)."""
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z.pow(3))))


def geglu_mlp(h: torch.Tensor, w_gate: torch.Tensor, w_up: torch.Tensor,
              w_down: torch.Tensor, round_to: torch.dtype | None = None) -> torch.Tensor:
    """down(gelu_tanh(gate(h)) * up(h)), no biases (src/wllm/models/gemma.py:54-62): five tensors
    (two projections, the activation, the product, the projection back), each in the model's dtype."""
    gate, up = _r(h @ w_gate.T, round_to), _r(h @ w_up.T, round_to)
    return _r(_r(_r(gelu_tanh(gate), round_to) * up, round_to) @ w_down.T, round_to)


def attention_block(h: torch.Tensor, weights: dict, prefix: str, cfg: dict,
                    cos: torch.Tensor, sin: torch.Tensor, round_to: torch.dtype | None = None,
                    tamper=None) -> torch.Tensor:
    """q/k/v projections (with bias only if attention_bias), views into heads,
    rotation of q and k, causal attention, output projection without bias
    (src/wllm/models/llama.py:95-115).  A projection with its bias is one operation (one rounding)."""
    nh, nkv, d = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"]
    T = h.shape[0]
    q = h @ weights[prefix + "q_proj.weight"].T
    k = h @ weights[prefix + "k_proj.weight"].T
    v = h @ weights[prefix + "v_proj.weight"].T
    if cfg["attention_bias"]:
        q = q + weights[prefix + "q_proj.bias"]
        k = k + weights[prefix + "k_proj.bias"]
        v = v + weights[prefix + "v_proj.bias"]
    q, k, v = _r(q, round_to), _r(k, round_to), _r(v, round_to)
    q = apply_rope(q.view(T, nh, d), cos, sin, round_to)
    k = apply_rope(k.view(T, nkv, d), cos, sin, round_to)
    o = causal_attention(q, k, v.view(T, nkv, d), d, round_to, tamper)
    return _r(o.reshape(T, nh * d) @ weights[prefix + "o_proj.weight"].T, round_to)


def decoder_layer(x: torch.Tensor, weights: dict, i: int, cfg: dict,
                  cos: torch.Tensor, sin: torch.Tensor, round_to: torch.dtype | None = None,
                  tamper=None) -> torch.Tensor:
    """norm, attention, residual; norm, feed-forward, residual
    (src/wllm/models/gemma.py:83-93).  `tamper(layer, allowed)`: see `causal_attention`."""
    p = f"model.layers.{i}."
    eps = cfg["rms_norm_eps"]
    layer_tamper = None if tamper is None else (lambda allowed: tamper(i, allowed))
    h = rms_norm_one_plus_w(x, weights[p + "input_layernorm.weight"], eps, round_to)
    x = _r(x + attention_block(h, weights, p + "self_attn.", cfg, cos, sin, round_to, layer_tamper), round_to)
    h = rms_norm_one_plus_w(x, weights[p + "post_attention_layernorm.weight"], eps, round_to)
    return _r(x + geglu_mlp(h, weights[p + "mlp.gate_proj.weight"], weights[p + "mlp.up_proj.weight"],
                            weights[p + "mlp.down_proj.weight"], round_to), round_to)


def forward_logits(cfg: dict, weights: dict, ids, positions=None,
                   scale_rounding: torch.dtype | None = None, round_to: torch.dtype | None = None,
                   tamper=None) -> torch.Tensor:
    """Logits [T, vocab] of one whole sequence (src/wllm/models/llama.py:405-415,
    432-446): embed and scale, positions 0..T-1 (`positions` moves them all, for
    the test that only distances count), the layers in order, the final norm,
    and the head: the embedding table itself, unscaled, when tied.  `round_to`: round where the
    reference's model of that dtype rounds (the logits too: they are a tensor of the model's dtype,
    llama.py:443-446), which implies `scale_rounding`.
    """
    ids = torch.as_tensor(ids, dtype=torch.long)
    table = weights["model.embed_tokens.weight"]
    dtype = table.dtype
    x = embed(ids, table, cfg["hidden_size"], scale_rounding or round_to, round_to)
    if positions is None:
        positions = torch.arange(ids.shape[0])
    cos, sin = rope_cos_sin(torch.as_tensor(positions), cfg["head_dim"], cfg["rope_theta"], dtype)
    for i in range(cfg["num_hidden_layers"]):
        x = decoder_layer(x, weights, i, cfg, cos, sin, round_to, tamper)
    x = rms_norm_one_plus_w(x, weights["model.norm.weight"], cfg["rms_norm_eps"], round_to)
    head = table if cfg["tie_word_embeddings"] else weights["lm_head.weight"]
    return _r(x @ head.T, round_to)


def generate_greedy(cfg: dict, weights: dict, prompt: list[int], max_new_tokens: int,
                    scale_rounding: torch.dtype | None = None) -> list[int]:
    """Full recomputation at every token, argmax of the last row
    (src/wllm/models/llama.py:599-610)."""
    tokens = list(prompt)
    for _ in range(max_new_tokens):
        logits = forward_logits(cfg, weights, tokens, scale_rounding=scale_rounding)
        tokens.append(int(logits[-1].argmax()))
    return tokens[len(prompt):]
