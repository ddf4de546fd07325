"""A plain sampler for one row of logits, written from the reference's
`sample` (src/wllm/engine/sampling.py:101-143), sort-based as it is there.  The one
change: where the reference draws with `torch.multinomial` (sampling.py:139), this
takes the uniform number `u` as an argument and inverts the cumulative distribution
in index order, which is how the engine draws; and it returns the probability
interval of every token so that a test can check a draw without depending on the
last bit of a sum.
"""
from __future__ import annotations

import numpy as np
import torch


def apply_repetition_penalty(logits: torch.Tensor, generated: list, penalty: float) -> torch.Tensor:
    """Positive logits of generated ids are divided by the penalty, negative ones
    multiplied; each distinct id once (sampling.py:45-58)."""
    logits = logits.clone()
    if penalty == 1.0 or not generated:
        return logits
    idx = torch.tensor(sorted(set(generated)), dtype=torch.long)
    row = logits[idx]
    logits[idx] = torch.where(row > 0, row / penalty, row * penalty)
    return logits


def keep_mask(scaled: torch.Tensor, top_k: int, top_p: float, min_p: float) -> torch.Tensor:
    """Which tokens survive top-k, top-p and min-p (sampling.py:61-98): on the
    descending sort of the scaled logits, rank < k; cumulative probability <= p
    except that rank 0 always stays; probability >= min_p * top probability."""
    vocab = scaled.shape[0]
    sorted_logits, sorted_idx = torch.sort(scaled, descending=True)
    keep = torch.ones(vocab, dtype=torch.bool)
    rank = torch.arange(vocab)
    if top_k > 0:
        keep &= rank < top_k
    probs = torch.softmax(sorted_logits, dim=-1)
    if top_p < 1.0:
        over = probs.cumsum(-1) > top_p
        over[0] = False
        keep &= ~over
    if min_p > 0.0:
        below = probs < min_p * probs[0]
        below[0] = False
        keep &= ~below
    out = torch.zeros(vocab, dtype=torch.bool)
    out[sorted_idx] = keep
    return out


def sample_row(logits: torch.Tensor, temperature: float, top_k: int, top_p: float, min_p: float,
               repetition_penalty: float, generated: list, u: float):
    """Returns (token, logprob, kept mask, (low, high) cumulative probability of each token
    among the kept ones in index order)."""
    logits = apply_repetition_penalty(logits.double(), generated, repetition_penalty)
    if temperature == 0.0:   # greedy: argmax of the penalised logits, logprob at temperature 1 (:125-131)
        token = int(logits.argmax())
        return token, float(torch.log_softmax(logits, -1)[token]), None, None
    scaled = logits / max(temperature, 1e-5)                       # :122-123
    logprobs = torch.log_softmax(scaled, -1)                       # before truncation (:130,142)
    keep = keep_mask(scaled, top_k, top_p, min_p)
    probs = torch.softmax(scaled.masked_fill(~keep, float("-inf")), -1)   # :136-137
    high = probs.cumsum(-1)
    low = high - probs
    token = int(torch.searchsorted(high, torch.tensor(u, dtype=high.dtype), right=True).clamp(max=len(high) - 1))
    return token, float(logprobs[token]), keep, (low, high)


def philox_uniform(seed: int, counter: int) -> float:
    """Philox4x32-10 with key (seed low, seed high) and counter (counter low, counter high, 0, 0);
    the first two output words make a 53-bit uniform number in [0, 1)."""
    m0, m1, w0, w1, mask = 0xD2511F53, 0xCD9E8D57, 0x9E3779B9, 0xBB67AE85, 0xFFFFFFFF
    ctr = [counter & mask, (counter >> 32) & mask, 0, 0]
    k0, k1 = seed & mask, (seed >> 32) & mask
    for _ in range(10):
        p0, p1 = m0 * ctr[0], m1 * ctr[2]
        ctr = [((p1 >> 32) ^ ctr[1] ^ k0) & mask, p1 & mask, ((p0 >> 32) ^ ctr[3] ^ k1) & mask, p0 & mask]
        k0, k1 = (k0 + w0) & mask, (k1 + w1) & mask
    return (((ctr[0] << 32) | ctr[1]) >> 11) / float(1 << 53)
