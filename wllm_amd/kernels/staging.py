"""Small arrays from the host to the device without making the host wait.

A copy from ordinary host memory waits until everything enqueued before it on the stream has
run, which would stop the host at every step; a copy from page-locked memory is only enqueued.
The page-locked buffer comes from torch's caching allocator, which does not hand it out again
before the copy has run.
"""
from __future__ import annotations

import numpy as np
import torch


def pack_int32(arrays: list, device):
    """Concatenates int32 arrays, copies them to the device at once and returns the
    device views in order."""
    sizes = [a.size for a in arrays]
    total = sum(sizes)
    host = torch.empty(max(total, 1), dtype=torch.int32, pin_memory=(torch.device(device).type == "cuda"))
    buf = host.numpy()
    o = 0
    for a, s in zip(arrays, sizes):
        buf[o:o + s] = a.reshape(-1)
        o += s
    dev = host.to(device, non_blocking=True)
    views, o = [], 0
    for a, s in zip(arrays, sizes):
        views.append(dev[o:o + s].view(a.shape))
        o += s
    return views


def pack_words(arrays: list, device):
    """The same for arrays of 4-byte and 8-byte numbers of any kind (int32, float32, int64): each
    comes back as a device tensor of its own dtype and shape.  8-byte arrays must come first."""
    words = [np.ascontiguousarray(a).reshape(-1).view(np.int32) for a in arrays]
    views = pack_int32(words, device)
    out = []
    for a, v in zip(arrays, views):
        out.append(v.view(getattr(torch, a.dtype.name)).view(a.shape))
    return out
