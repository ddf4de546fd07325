"""A plain emulation of every kernel's contract, in ordinary torch arithmetic.

It has two uses.  On a machine without a GPU it stands in for the kernel library
so that the engine's bookkeeping (cache, batching, scheduling) can be compared
with the plain implementation.  On the GPU it is each kernel's reference: the
`-m gpu` tests run a kernel and its emulation on the same operands.  It follows
the contracts written in `wllm_amd/kernels/ops.py`, not the kernels' code, and
computes in float64 when `precise` is set.
"""
from __future__ import annotations

import math

import torch


class EmulatedKernels:
    def __init__(self, precise: bool = False, splits: int = 1):
        self.acc = torch.float64 if precise else torch.float32
        self.calls = {}
        self.splits = splits        # into how many partial sums `linear` is asked to split

    def _count(self, name):
        self.calls[name] = self.calls.get(name, 0) + 1

    def run_registered(self, op, args, kwargs):
        """An operation that went through `ops.register_op`: the framework's own have their emulation
        here under their name; one that a part registered brings its own."""
        own = getattr(self, op.name, None)
        if own is not None:
            own(*args, **kwargs)
            return
        self._count(op.name)
        if op.emulate is None:
            raise NotImplementedError(f"operation {op.name!r} was registered without an emulation")
        op.emulate(*args, **kwargs)

    def embed_lookup(self, ids, table, scale, out):
        self._count("embed_lookup")
        out.copy_((table[ids.long()].to(self.acc) * scale).to(out.dtype))

    def feed_tokens(self, ids, dst, src, source):
        self._count("feed_tokens")
        for d, s in zip(dst.tolist(), src.tolist()):
            if 0 <= d < ids.shape[0] and 0 <= s < source.shape[0]:
                ids[d] = source[s]

    def rms_norm(self, x, weight, eps, offset, out, delta, rows):
        self._count("rms_norm")
        if delta is not None and delta.dim() == 3:
            total = delta[0].to(torch.float32)
            for p in range(1, delta.shape[0]):
                total = total + delta[p]
            delta = total
        if rows is None:
            v = x.to(self.acc)
            if delta is not None:
                v = v + delta.to(self.acc)
                x.copy_(v.to(x.dtype))
                v = x.to(self.acc)  # the kernel normalises what it wrote back
        else:
            idx = rows.long()
            v = x[idx].to(self.acc)
            if delta is not None:
                v = (v + delta[idx].to(self.acc)).to(x.dtype).to(self.acc)
        var = v.pow(2).mean(-1, keepdim=True)
        y = v * torch.rsqrt(var + eps) * (offset + weight.to(self.acc))
        out.copy_(y.to(out.dtype))

    fused_qkv = True        # whether the emulation offers the fused projection and rotation
    fused_residual = True   # and the product that adds into the residual stream

    def linear_residual_takes(self, rows, dtype, out_features, in_features):
        return self.fused_residual and rows <= 16 and out_features % 16 == 0

    def linear_residual(self, x, weight, tiles, residual, sumsq):
        self._count("linear_residual")
        self._same_numbers(weight, tiles, 1)
        new = residual.to(self.acc) + x.to(self.acc) @ weight.to(self.acc).T
        residual.copy_(new.to(torch.float32))
        sumsq.copy_((residual.to(self.acc) ** 2).view(residual.shape[0], -1, 16).sum(-1).to(torch.float32))

    def qkv_rope_takes(self, rows, dtype, in_features, head_dim, rotary_dim):
        return self.fused_qkv and rotary_dim == head_dim and rows <= 32

    def qkv_rope(self, x, weight, tiles, qkv, bias, positions, inv_freq, slots, cache, num_heads, num_kv_heads,
                 head_dim, page_size):
        self._count("qkv_rope")
        self._same_numbers(weight, tiles, 1)
        # the kernel rotates the float32 sums, not their rounding to the activation dtype: hand them
        # on as a stack of one partial sum
        pre = (x.to(self.acc) @ weight.to(self.acc).T).to(torch.float32)[None]
        self.rope_and_cache_write(qkv, bias, positions, inv_freq, slots, cache, num_heads, num_kv_heads, head_dim,
                                  head_dim if inv_freq is not None else 0, page_size, parts=pre)
        self.calls["rope_and_cache_write"] -= 1

    def rope_and_cache_write(self, qkv, bias, positions, inv_freq, slots, cache, num_heads, num_kv_heads,
                             head_dim, rotary_dim, page_size, parts=None):
        self._count("rope_and_cache_write")
        n = qkv.shape[0]
        heads = num_heads + 2 * num_kv_heads
        if parts is not None:
            total = parts[0]
            for p in range(1, parts.shape[0]):
                total = total + parts[p]
            v = total.to(self.acc)
        else:
            v = qkv.to(self.acc)
        if bias is not None:
            v = v + bias.to(self.acc)
        v = v.view(n, heads, head_dim).clone()
        if inv_freq is not None:
            half = rotary_dim // 2
            ang = positions.to(torch.float32)[:, None] * inv_freq[None, :]          # float32 angles
            cos, sin = ang.cos().to(self.acc)[:, None, :], ang.sin().to(self.acc)[:, None, :]
            r = num_heads + num_kv_heads                                              # queries and keys
            x1 = v[:, :r, :half].clone()
            x2 = v[:, :r, half:rotary_dim].clone()
            v[:, :r, :half] = x1 * cos - x2 * sin
            v[:, :r, half:rotary_dim] = x2 * cos + x1 * sin
        qkv.copy_(v.view(n, -1).to(qkv.dtype))
        if cache is not None:
            rows = qkv.view(n, heads, head_dim)
            page = (slots // page_size).long()
            off = (slots % page_size).long()
            k = rows[:, num_heads:num_heads + num_kv_heads]                           # [n, nkv, d]
            val = rows[:, num_heads + num_kv_heads:]
            kview = cache[:, 0].view(cache.shape[0], num_kv_heads, page_size, head_dim)
            vview = cache[:, 1].view(cache.shape[0], num_kv_heads, head_dim, page_size)
            kview[page, :, off, :] = k
            vview[page, :, :, off] = val

    def paged_attention(self, qkv, cache, block_tables, token_segment, seg_q_start, seg_q_len, seg_ctx_len, out,
                        num_heads, num_kv_heads, head_dim, page_size, scale, window, max_q_len, max_ctx_len,
                        plan=None):
        self._count("paged_attention")
        n = qkv.shape[0]
        n_rep = num_heads // num_kv_heads
        q_all = qkv.view(n, num_heads + 2 * num_kv_heads, head_dim)[:, :num_heads].to(self.acc)
        pages = cache.shape[0]
        kview = cache[:, 0].view(pages, num_kv_heads, page_size, head_dim)
        vview = cache[:, 1].view(pages, num_kv_heads, head_dim, page_size)
        for s in range(block_tables.shape[0]):
            q0, ql, cl = int(seg_q_start[s]), int(seg_q_len[s]), int(seg_ctx_len[s])
            if ql == 0:
                continue
            npages = -(-cl // page_size)
            ids = block_tables[s, :npages].long()
            k = kview[ids].permute(0, 2, 1, 3).reshape(npages * page_size, num_kv_heads, head_dim)[:cl].to(self.acc)
            v = vview[ids].permute(0, 3, 1, 2).reshape(npages * page_size, num_kv_heads, head_dim)[:cl].to(self.acc)
            k = k.repeat_interleave(n_rep, dim=1)
            v = v.repeat_interleave(n_rep, dim=1)
            q = q_all[q0:q0 + ql]
            pos = torch.arange(cl - ql, cl, device=q.device)
            key = torch.arange(cl, device=q.device)
            allowed = key[None, :] <= pos[:, None]
            if window:
                allowed &= key[None, :] > pos[:, None] - window
            scores = torch.einsum("qhd,khd->hqk", q, k) * scale
            # keys outside the window may hold NaN of pages given back: mask by selection, not by addition
            scores = torch.where(allowed[None], scores, torch.full_like(scores, float("-inf")))
            probs = torch.softmax(scores, dim=-1)
            v = torch.where(torch.isnan(v), torch.zeros_like(v), v) if window else v
            o = torch.einsum("hqk,khd->qhd", probs, v)
            out[q0:q0 + ql] = o.reshape(ql, num_heads * head_dim).to(out.dtype)

    def plan_paged_attention(self, *args):
        return None

    def linear_splits(self, rows, out_features, in_features, dtype):
        return self.splits

    def tile_weight(self, weight, tiles):
        """bfloat16: [n, k] -> [band][step][g][i][8]: lane 16g + i of a wavefront holds w[16 band + i][32 step + 8g .. +8].
        float32: [n, k] -> [band][chunk][g][i][4] with rows and keys padded with zeros to multiples of 16."""
        n, k = weight.shape
        if weight.dtype == torch.float32:
            padded = torch.zeros(-(-n // 16) * 16, -(-k // 16) * 16, dtype=weight.dtype, device=weight.device)
            padded[:n, :k] = weight
            tiles.copy_(padded.view(-1, 16, padded.shape[1] // 16, 4, 4).permute(0, 2, 3, 1, 4).reshape(-1))
            return
        padded = torch.zeros(-(-n // 16) * 16, k, dtype=weight.dtype, device=weight.device)
        padded[:n] = weight
        tiles.copy_(padded.view(-1, 16, k // 32, 4, 8).permute(0, 2, 3, 1, 4).reshape(-1))

    def _same_numbers(self, weight, tiles, halves):
        """A tile-major copy must hold the weight's numbers: the emulation computes from the weight."""
        if tiles is None:
            return
        if weight.dtype == torch.float32:
            n, k = weight.shape
            kp = -(-k // 16) * 16
            back = tiles.view(-1, kp // 16, 4, 16, 4).permute(0, 3, 1, 2, 4).reshape(-1, kp)[:n, :k]
            assert torch.equal(back, weight), "the tile-major copy differs from the weight"
            return
        n, k = weight.shape[0] // halves, weight.shape[1]
        size = -(-n // 16) * 16 * k
        for h in range(halves):
            back = tiles[h * size:(h + 1) * size].view(-1, k // 32, 4, 16, 8).permute(0, 3, 1, 2, 4).reshape(-1, k)[:n]
            assert torch.equal(back, weight[h * n:(h + 1) * n]), "the tile-major copy differs from the weight"

    def linear(self, x, weight, out, tiles=None):
        self._count("linear")
        self._same_numbers(weight, tiles, 1)
        if out.dim() == 3:
            k = x.shape[1]
            edges = [round(i * k / out.shape[0]) for i in range(out.shape[0] + 1)]
            for p in range(out.shape[0]):
                a, b = edges[p], edges[p + 1]
                out[p].copy_((x[:, a:b].to(self.acc) @ weight[:, a:b].to(self.acc).T).to(out.dtype))
            return
        out.copy_((x.to(self.acc) @ weight.to(self.acc).T).to(out.dtype))

    fused_norm = True       # and the gated product with the norm on load

    def gated_linear_norm_takes(self, rows, dtype, in_features):
        return self.fused_norm and rows <= 16

    def gated_linear_norm(self, x, weight, out, activation, tiles=None):
        self._count("gated_linear_norm")
        self._same_numbers(weight, tiles, 2)
        r = x.residual.to(self.acc)
        # the mean square comes from the sums the producer left, not from the residual itself
        inv = torch.rsqrt(x.sumsq.to(self.acc).sum(-1, keepdim=True) / r.shape[1] + x.eps)
        h = (r * inv * (x.offset + x.weight.to(self.acc))).to(x.dtype)
        gu = (h.to(self.acc) @ weight.to(self.acc).T)
        self.gated_activation(gu, out, activation)
        self.calls["gated_activation"] -= 1

    def gated_linear(self, x, weight, out, activation, scratch, tiles=None):
        self._count("gated_linear")
        self._same_numbers(weight, tiles, 2)
        gu = (x.to(self.acc) @ weight.to(self.acc).T)
        self.gated_activation(gu, out, activation)

    def gated_activation(self, gate_up, out, activation):
        self._count("gated_activation")
        i = gate_up.shape[1] // 2
        g, u = gate_up[:, :i].to(self.acc), gate_up[:, i:].to(self.acc)
        if activation == "gelu_tanh":
            a = 0.5 * g * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (g + 0.044715 * g.pow(3))))
        elif activation == "silu":
            a = g * torch.sigmoid(g)
        else:
            raise ValueError(activation)
        out.copy_((a * u).to(out.dtype))

    def argmax_rows(self, logits, out):
        self._count("argmax_rows")
        out.copy_(logits.argmax(dim=-1).to(torch.int32))

    def sample_rows(self, logits, params, seeds, penalty_ids, penalty_offsets, out_tokens, out_logprobs,
                    truncations=True):
        from plain.sampling_plain import philox_uniform, sample_row
        self._count("sample_rows")
        for r in range(logits.shape[0]):
            t, k, p, mp, pen = (float(x) for x in params[r])
            gen = []
            if penalty_ids is not None:
                gen = penalty_ids[int(penalty_offsets[r]):int(penalty_offsets[r + 1])].tolist()
            u = philox_uniform(int(seeds[r, 0]), int(seeds[r, 1]))
            tok, lp, _, _ = sample_row(logits[r].cpu(), t, int(k), p, mp, pen, gen, u)
            out_tokens[r] = tok
            out_logprobs[r] = lp
