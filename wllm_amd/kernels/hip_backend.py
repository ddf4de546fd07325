"""Calls into the kernel library: tensors to raw pointers, the current stream, error codes
to exceptions.  Shapes were checked in `ops`; what is checked here is that tensors live
on the GPU, since a host pointer handed to a kernel faults the device."""
from __future__ import annotations

import ctypes
from ctypes import c_float, c_int, c_longlong, c_void_p

import numpy as np
import torch

from wllm_amd.kernels.attention_plan import AttentionPlan, build_work_items
from wllm_amd.kernels import ops
from wllm_amd.kernels.ops import ACTIVATIONS
from wllm_amd.kernels.library import load
from wllm_amd.kernels.staging import pack_int32


class KernelError(RuntimeError):
    """A kernel launch failed or a kernel refused its operands."""


# torch's own shortcut to the current stream's handle (what its compiled kernels call)
_raw_current_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _ptr(t):
    return c_void_p(t.data_ptr()) if t is not None else c_void_p(0)


_SIGNATURES = {
    "wllm_gemm_residual": [c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_int, c_int, c_int, c_void_p],
    "wllm_qkv_rope": [c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_longlong,
                      c_int, c_int, c_int, c_int, c_int, c_int, c_void_p],
    "wllm_rms_norm": [c_void_p, c_void_p, c_int, c_int, c_longlong, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int,
                      c_float, c_float, c_void_p],
    "wllm_rope_cache_write": [c_void_p, c_int, c_void_p, c_int, c_longlong, c_void_p, c_void_p, c_void_p, c_void_p,
                              c_void_p, c_longlong, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p],
    "wllm_gemm_skinny_gated": [c_void_p, c_void_p, c_int, c_void_p, c_int, c_int, c_int, c_int, c_int, c_void_p],
    "wllm_gemm_skinny_gated_norm": [c_void_p, c_void_p, c_int, c_void_p, c_float, c_float, c_void_p, c_int, c_void_p, c_int,
                                    c_int, c_int, c_int, c_void_p],
    "wllm_tile_weight": [c_void_p, c_void_p, c_int, c_int, c_void_p],
    "wllm_paged_attention_generic": [c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                     c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int,
                                     c_float, c_int, c_void_p],
    "wllm_paged_attention_generic_chunk_keys": [],
    "wllm_paged_attention_mfma": [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_int, c_void_p, c_void_p,
                                  c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_float,
                                  c_int, c_void_p],
    "wllm_paged_attention_mfma_f32": [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_int, c_void_p, c_void_p,
                                      c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_float, c_int, c_void_p],
    "wllm_paged_attention_prefill_f32": [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_void_p, c_void_p, c_void_p,
                                         c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_float, c_int,
                                         c_void_p],
    "wllm_paged_attention_prefill": [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_void_p, c_void_p, c_void_p,
                                     c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_float, c_int,
                                     c_void_p],
    "wllm_gemm_tile": [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_void_p],
    "wllm_split_sum": [c_void_p, c_void_p, c_int, c_longlong, c_int, c_void_p],
    "wllm_gemm_generic": [c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_int, c_void_p, c_int, c_int, c_int, c_void_p],
    "wllm_tile_weight_f32": [c_void_p, c_void_p, c_int, c_int, c_void_p],
    "wllm_gemm_f32_segments": [c_int, c_int, c_int],
    "wllm_argmax_rows": [c_void_p, c_void_p, c_void_p, c_int, c_int, c_void_p],
    "wllm_gemm_skinny": [c_void_p, c_void_p, c_int, c_void_p, c_int, c_void_p, c_int, c_int, c_int, c_int, c_int,
                         c_void_p],
    "wllm_sample_rows": [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_void_p],
    "wllm_sample_rows_split": [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int,
                               c_int, c_int, c_void_p],
    "wllm_sample_split_row_words": [],
}


class HipBackend:
    def __init__(self):
        if not torch.cuda.is_available():
            raise KernelError("no GPU is visible; the kernels run on gfx950 only and there is no other path")
        self.lib = load()
        self._device_index = torch.cuda.current_device()
        self._partial_o = None
        self._slots_of = {}                # device -> workgroups of the prompt kernel it runs at once
        self._gemm_partials = None
        self._argmax_scratch = None
        self._sample_scratch = None
        self._partial_ml = None
        self._generic_partial_o = None
        self._registered: dict = {}
        self.library_events = None      # a list: every library product is bracketed by a pair of timing events
        for name, argtypes in _SIGNATURES.items():
            fn = getattr(self.lib, name)
            fn.argtypes = argtypes
            fn.restype = c_int

    @staticmethod
    def _on_gpu(*tensors) -> None:
        for t in tensors:
            if t is not None and not t.is_cuda:
                raise KernelError("a kernel operand is not on the GPU")

    def _stream(self) -> c_void_p:
        # the raw handle of torch's current stream on this process's GPU, asked for at every launch
        if _raw_current_stream is not None:
            return c_void_p(_raw_current_stream(self._device_index))
        return c_void_p(torch.cuda.current_stream().cuda_stream)

    @staticmethod
    def _check(code: int, what: str) -> None:
        if code == -1:
            raise KernelError(f"{what}: the kernel does not take these sizes")
        if code != 0:
            raise KernelError(f"{what}: HIP error {code}")

    def run_registered(self, op, args, kwargs) -> None:
        """An operation that a part registered (`ops.register_op`): its entry point is looked up once in
        its library, given its signature, and launched on the current stream."""
        fn = self._registered.get(op.name)
        if fn is None or fn[0] is not op:
            lib = op.library() if op.library is not None else self.lib
            entry = getattr(lib, op.entry_point)
            entry.argtypes = op.argtypes
            entry.restype = c_int
            fn = self._registered[op.name] = (op, entry)
        self._on_gpu(*[a for a in list(args) + list(kwargs.values()) if isinstance(a, torch.Tensor)])
        self._check(op.launch(fn[1], self._stream(), *args, **kwargs), op.name)

    def rms_norm(self, x, weight, eps, offset, out, delta, rows):
        self._on_gpu(x, weight, out, delta, rows)
        splits, stride = 1, 0
        if delta is not None and delta.dim() == 3:
            splits, stride = delta.shape[0], delta.shape[1] * delta.shape[2]
        self._check(self.lib.wllm_rms_norm(
            _ptr(x), _ptr(delta), int(delta is not None and delta.dtype == torch.bfloat16), splits, stride,
            _ptr(weight), _ptr(rows), _ptr(out), int(out.dtype == torch.bfloat16), out.shape[0], x.shape[1], eps,
            offset, self._stream()), "rms_norm")

    def rope_and_cache_write(self, qkv, bias, positions, inv_freq, slots, cache, num_heads, num_kv_heads, head_dim,
                             rotary_dim, page_size, parts=None):
        self._on_gpu(qkv, bias, positions, inv_freq, slots, cache, parts)
        splits, stride = (parts.shape[0], parts.shape[1] * parts.shape[2]) if parts is not None else (0, 0)
        self._check(self.lib.wllm_rope_cache_write(
            _ptr(qkv), int(qkv.dtype == torch.bfloat16), _ptr(parts), splits, stride, _ptr(bias), _ptr(positions),
            _ptr(inv_freq), _ptr(slots),
            _ptr(cache), cache.shape[0] if cache is not None else 0, qkv.shape[0], num_heads, num_kv_heads, head_dim,
            rotary_dim, page_size, self._stream()), "rope_and_cache_write")

    RESIDUAL_MAX_K = 4096

    def linear_residual_takes(self, rows: int, dtype, out_features: int, in_features: int) -> bool:
        """The product that adds into the residual stream: bfloat16, at most 16 rows, whole bands of
        16 columns.  Its workgroups are the bands; with a long K axis there are too few of them for the
        weight to stream from all compute units, and the split product with its norm kernel is faster."""
        return (dtype == torch.bfloat16 and 1 <= rows <= 16 and out_features % 16 == 0 and in_features % 32 == 0
                and in_features <= self.RESIDUAL_MAX_K)

    def linear_residual(self, x, weight, tiles, residual, sumsq):
        self._on_gpu(x, weight, tiles, residual, sumsq)
        w, tiled = (tiles, 1) if tiles is not None else (weight, 0)
        self._check(self.lib.wllm_gemm_residual(_ptr(x), _ptr(w), tiled, _ptr(residual), _ptr(sumsq), x.shape[0],
                                                weight.shape[0], x.shape[1], self._stream()), "linear_residual")

    @staticmethod
    def qkv_rope_takes(rows: int, dtype, in_features: int, head_dim: int, rotary_dim: int) -> bool:
        """The fused projection, rotation and cache write: bfloat16, at most 32 tokens, heads of a
        multiple of 32 that are rotated whole."""
        return (dtype == torch.bfloat16 and 1 <= rows <= 32 and in_features % 32 == 0 and head_dim % 32 == 0
                and rotary_dim == head_dim)

    def qkv_rope(self, x, weight, tiles, qkv, bias, positions, inv_freq, slots, cache, num_heads, num_kv_heads,
                 head_dim, page_size):
        self._on_gpu(x, weight, tiles, qkv, bias, positions, inv_freq, slots, cache)
        w, tiled = (tiles, 1) if tiles is not None else (weight, 0)
        self._check(self.lib.wllm_qkv_rope(
            _ptr(x), _ptr(w), tiled, _ptr(bias), _ptr(positions), _ptr(inv_freq), _ptr(slots), _ptr(qkv), _ptr(cache),
            cache.shape[0] if cache is not None else 0, x.shape[0], x.shape[1], num_heads, num_kv_heads, head_dim,
            page_size, self._stream()), "qkv_rope")

    @staticmethod
    def mfma_attention_takes(dtype, head_dim: int, page_size: int) -> bool:
        """The matrix-core kernels: bfloat16 or float32 (each with the instruction of its own type), head sizes
        32..256 in steps of 32, pages of a multiple of 4."""
        return (dtype in (torch.bfloat16, torch.float32) and head_dim % 32 == 0 and 32 <= head_dim <= 256
                and page_size % 4 == 0)

    def plan_paged_attention(self, host_q_len, host_ctx_len, num_heads, num_kv_heads, head_dim, page_size, window,
                             dtype, device):
        if not self.mfma_attention_takes(dtype, head_dim, page_size):
            return None
        group, slots_of_device = num_heads // num_kv_heads, self._workgroup_slots(device)
        items, reduces, slots, prefill, prefill_rows = build_work_items(
            host_q_len, host_ctx_len, group, num_kv_heads, window, page_size, workgroup_slots=slots_of_device)
        if dtype == torch.float32 and 0 < prefill.shape[0] < slots_of_device // 2:
            # float32 and few blocks of 64 rows (a prompt of some hundred tokens): tiles of 16 rows fill the device
            # better than the blocks would (512 tokens of 8 heads: 43 against 96 us).  With so few blocks the tiles
            # are few too (at most four a block) and so are their chunks (the blocks' keys were not worth cutting).
            items, reduces, slots, prefill, prefill_rows = build_work_items(
                host_q_len, host_ctx_len, group, num_kv_heads, window, page_size, workgroup_slots=slots_of_device,
                tiles_only=True)
        flat = np.concatenate([items.reshape(-1), reduces.reshape(-1), prefill.reshape(-1)])
        dev = pack_int32([flat], device)[0]
        n_i, n_r, n_p = items.shape[0], reduces.shape[0], prefill.shape[0]
        self._ensure_partials(slots, head_dim, device)
        a, b = n_i * 8, (n_i + n_r) * 8
        return AttentionPlan(dev[:a].view(n_i, 8), dev[a:b].view(n_r, 8) if n_r else None, n_i, n_r, slots,
                             self._partial_o, self._partial_ml, dev[b:].view(n_p, 8) if n_p else None, n_p,
                             prefill_rows)

    def _workgroup_slots(self, device) -> int:
        """Workgroups of the kernel for prompt portions that the device runs at once: two a compute unit."""
        key = torch.device(device)
        if key not in self._slots_of:
            self._slots_of[key] = 2 * torch.cuda.get_device_properties(key).multi_processor_count
        return self._slots_of[key]

    def static_attention_plan(self, segments, num_heads, num_kv_heads, head_dim, page_size, window, dtype, device,
                              max_context: int, max_total_keys: int):
        """A plan of fixed shape for a captured decode graph of `segments` requests of one token."""
        if not self.mfma_attention_takes(dtype, head_dim, page_size):
            return None
        from wllm_amd.kernels.attention_plan import KEY_CHUNK, StaticAttentionPlan, row_tiles
        group = num_heads // num_kv_heads
        fixed = -(-max_context // KEY_CHUNK)
        max_slots = (max_total_keys // KEY_CHUNK + 2 * segments) * num_kv_heads * row_tiles(1, group)
        return StaticAttentionPlan(segments, group, num_kv_heads, window, fixed, max_slots, head_dim, device)

    def _ensure_partials(self, slots: int, head_dim: int, device) -> None:
        need = max(1, slots) * 16 * head_dim
        if self._partial_o is None or self._partial_o.numel() < need or self._partial_o.device != torch.device(device):
            self._partial_o = torch.empty(need, dtype=torch.float32, device=device)
        need = max(1, slots) * 16 * 2
        if self._partial_ml is None or self._partial_ml.numel() < need or self._partial_ml.device != torch.device(device):
            self._partial_ml = torch.empty(need, dtype=torch.float32, device=device)

    GENERIC_PARTIAL_FLOATS = 1 << 25       # 128 MiB of partial results for the general attention kernel

    def paged_attention(self, qkv, cache, block_tables, token_segment, seg_q_start, seg_q_len, seg_ctx_len, out,
                        num_heads, num_kv_heads, head_dim, page_size, scale, window, max_q_len, max_ctx_len,
                        plan=None):
        self._on_gpu(qkv, cache, block_tables, token_segment, seg_q_start, seg_q_len, seg_ctx_len, out)
        if plan is not None:
            if not self.mfma_attention_takes(qkv.dtype, head_dim, page_size):
                raise KernelError("paged_attention: a plan was given for sizes the matrix-core kernel does not take")
            if qkv.dtype == torch.float32:
                if plan.num_prefill:
                    self._check(self.lib.wllm_paged_attention_prefill_f32(
                        _ptr(qkv), _ptr(cache), _ptr(block_tables), _ptr(plan.prefill_items), plan.num_prefill,
                        plan.prefill_rows, _ptr(seg_q_start), _ptr(seg_q_len), _ptr(seg_ctx_len), _ptr(out),
                        _ptr(plan.partial_o), _ptr(plan.partial_ml), num_heads, num_kv_heads, head_dim, page_size,
                        block_tables.shape[1], scale, window, self._stream()),
                        "paged_attention (prompt portions, matrix cores, float32)")
                if plan.num_items == 0 and plan.num_reduce == 0:
                    return
                self._check(self.lib.wllm_paged_attention_mfma_f32(
                    _ptr(qkv), _ptr(cache), _ptr(block_tables), _ptr(plan.items), _ptr(plan.live_items), plan.num_items,
                    _ptr(plan.reduce_items), plan.num_reduce, _ptr(seg_q_start), _ptr(seg_q_len), _ptr(out),
                    _ptr(plan.partial_o), _ptr(plan.partial_ml), num_heads, num_kv_heads, head_dim, page_size,
                    block_tables.shape[1], scale, window, self._stream()), "paged_attention (matrix cores, float32)")
                return
            if plan.num_prefill:
                self._check(self.lib.wllm_paged_attention_prefill(
                    _ptr(qkv), _ptr(cache), _ptr(block_tables), _ptr(plan.prefill_items), plan.num_prefill,
                    plan.prefill_rows,
                    _ptr(seg_q_start), _ptr(seg_q_len), _ptr(seg_ctx_len), _ptr(out), _ptr(plan.partial_o),
                    _ptr(plan.partial_ml), num_heads, num_kv_heads,
                    head_dim, page_size, block_tables.shape[1], scale, window, self._stream()),
                    "paged_attention (prompt portions, matrix cores)")
            if plan.num_items == 0 and plan.num_reduce == 0:
                return
            self._check(self.lib.wllm_paged_attention_mfma(
                _ptr(qkv), _ptr(cache), _ptr(block_tables), _ptr(plan.items),
                _ptr(plan.live_items), plan.num_items, _ptr(plan.reduce_items),
                plan.num_reduce, _ptr(seg_q_start), _ptr(seg_q_len), _ptr(seg_ctx_len), _ptr(out),
                _ptr(plan.partial_o), _ptr(plan.partial_ml), num_heads, num_kv_heads, head_dim, page_size,
                block_tables.shape[1], scale, window, self._stream()), "paged_attention (matrix cores)")
            return
        if head_dim % 4 or head_dim > 256:
            raise KernelError(f"paged_attention: head_dim {head_dim} is not a multiple of 4 up to 256")
        # The general kernel cuts a token's keys into chunks and leaves the chunks of a token that has
        # several in a buffer for a second kernel.  The buffer is made once at a fixed size (captured
        # graphs hold its address); the tokens of a step run in as many launches as it takes.
        longest = block_tables.shape[1] * page_size
        max_ctx_len = min(max_ctx_len, longest) if max_ctx_len > 0 else longest
        chunks = -(-max_ctx_len // self.lib.wllm_paged_attention_generic_chunk_keys())
        per_token = num_heads * chunks * (head_dim + 2)
        if per_token > self.GENERIC_PARTIAL_FLOATS:
            raise KernelError(f"paged_attention: one token of {num_heads} heads over {max_ctx_len} keys needs "
                              f"{per_token} floats of partial results, {self.GENERIC_PARTIAL_FLOATS} are reserved")
        if self._generic_partial_o is None or self._generic_partial_o.device != qkv.device:
            self._generic_partial_o = torch.empty(self.GENERIC_PARTIAL_FLOATS, dtype=torch.float32, device=qkv.device)
        partial_tokens = self.GENERIC_PARTIAL_FLOATS // per_token
        partial_ml = self._generic_partial_o[partial_tokens * num_heads * chunks * head_dim:]
        self._check(self.lib.wllm_paged_attention_generic(
            _ptr(qkv), _ptr(cache), int(qkv.dtype == torch.bfloat16), _ptr(block_tables), _ptr(token_segment),
            _ptr(seg_q_start), _ptr(seg_q_len), _ptr(seg_ctx_len), _ptr(out), _ptr(self._generic_partial_o),
            _ptr(partial_ml), partial_tokens, max_ctx_len, qkv.shape[0], num_heads, num_kv_heads,
            head_dim, page_size, block_tables.shape[1], scale, window, self._stream()), "paged_attention")

    @staticmethod
    def skinny_split(n: int, k: int) -> int:
        """Over how many workgroups the K axis of a few-row product is split: enough that about
        2,000 wavefronts stream weights at once, a function of the weight's shape only."""
        tiles = -(-n // 16)
        splits = 1
        while tiles * splits < 1536 and k % (splits * 2) == 0 and (k // (splits * 2)) % 32 == 0 \
                and k // (splits * 2) >= 256:
            splits *= 2
        return splits

    # splits * N stays below 3072 * 16 by the rule of `skinny_split`; 64 rows of float32 of that
    GEMM_PARTIAL_FLOATS = 3072 * 16 * 64

    def _gemm_partial(self, count: int, device) -> torch.Tensor:
        """The buffer of split sums.  It is allocated once at its largest size and never again,
        because captured graphs hold its address."""
        if count > self.GEMM_PARTIAL_FLOATS:
            raise KernelError(f"split-sum buffer: {count} floats needed, {self.GEMM_PARTIAL_FLOATS} reserved")
        if self._gemm_partials is None or self._gemm_partials.device != device:
            self._gemm_partials = torch.empty(self.GEMM_PARTIAL_FLOATS, dtype=torch.float32, device=device)
        return self._gemm_partials

    SKINNY_CHUNK = {1: 1024, 2: 512, 3: 256, 4: 256}     # K elements of x staged at a time, by row tiles
    GATED_CHUNK = {1: 256, 2: 256, 3: 256, 4: 256}       # the same per half of K in the gated product

    @staticmethod
    def skinny_takes(dtype, rows: int, in_features: int) -> bool:
        return dtype == torch.bfloat16 and rows <= 64 and in_features % 32 == 0

    # The tiled matrix-core product (`gemm_tile.hip`) for the rows of a mixed step or a large decode
    # batch.  Measured against the library's product it is ahead where the output has few columns and
    # the K axis is long, so that the library's tiles leave compute units idle and a split of the K axis
    # fills them (the down projection: 1.3 to 1.6 times as fast at 128 to 1,024 rows), and for the gated
    # product, which it writes once, up to 256 rows (at 512 rows it takes 84 us in a mixed step where
    # the library's product and the activation kernel take 69).  With these two the decode step of 256
    # requests is 5% and the stress workload 2% faster.  The projections of the attention block are
    # twice as fast alone (K axis of 2,048 in four pieces at 128 to 512 rows), but the rotation and the
    # norm that then add the pieces lose more than that: left to the library.
    TILE_MAX_ROWS = 1024
    F32_FEW_ROWS = 64         # rows up to which the float32 product streams its weights a band a wavefront
    TILE_LONG_K = 8192
    TILE_GATED_MAX_ROWS = 256

    @staticmethod
    def tile_splits(n: int, k: int, rows: int = 128) -> int:
        """Over how many workgroups the tiled product splits the K axis: a function of the weight's
        shape up to 640 rows, so that a row's sums do not depend on the step's other rows there.
        More rows fill the machine with fewer pieces, and every piece is a stack of partial sums to
        write and to read: halved while the launch has more than 640 workgroups (the down projection
        of 2,048 x 16,384 with the norm after it, 4 pieces against 8: 78 against 92 us at 1,024 rows,
        70 against 80 at 896, 68 against 70 at 768, but 67 against 64 at 640; that of 3,072 x 24,576:
        184 us with 2 pieces against 215 with 8 at 1,024 rows, 155 with 4 against 164 at 768)."""
        tiles = -(-n // 128)
        splits = 1
        while tiles * splits * 2 < 256 and k % (128 * splits) == 0 and k // (2 * splits) >= 512:
            splits *= 2
        row_tiles = -(-rows // 128)
        while splits > 2 and row_tiles > 5 and tiles * row_tiles * splits > 640:
            splits //= 2
        return splits

    def tile_takes(self, dtype, rows: int, out_features: int, in_features: int) -> bool:
        return (dtype == torch.bfloat16 and 64 < rows <= self.TILE_MAX_ROWS and in_features >= self.TILE_LONG_K
                and in_features % 64 == 0 and self.tile_splits(out_features, in_features, rows) > 1
                and max(rows, out_features) * in_features * 2 < 2 ** 32)

    def linear_splits(self, rows, out_features, in_features, dtype) -> int:
        if self.skinny_takes(dtype, rows, in_features):
            return self.skinny_split(out_features, in_features)
        if self.tile_takes(dtype, rows, out_features, in_features):
            return self.tile_splits(out_features, in_features, rows)
        if dtype == torch.float32 and rows <= self.F32_FEW_ROWS:
            return self.lib.wllm_gemm_f32_segments(rows, out_features, in_features)
        return 1

    def tile_weight(self, weight, tiles) -> None:
        self._on_gpu(weight, tiles)
        if weight.dtype == torch.float32:
            self._check(self.lib.wllm_tile_weight_f32(_ptr(weight), _ptr(tiles), weight.shape[0], weight.shape[1],
                                                      self._stream()), "tile_weight (float32)")
            return
        self._check(self.lib.wllm_tile_weight(_ptr(weight), _ptr(tiles), weight.shape[0], weight.shape[1], self._stream()),
                    "tile_weight")

    def _skinny(self, x, weight, out, tiles=None) -> None:
        m, k = x.shape
        n = weight.shape[0]
        splits = self.skinny_split(n, k)
        chunk = self.SKINNY_CHUNK[min(4, -(-m // 16))]
        w, tiled = (tiles, 1) if tiles is not None else (weight, 0)
        if out.dim() == 3:      # the caller adds the partial sums later
            self._check(self.lib.wllm_gemm_skinny(_ptr(x), _ptr(w), tiled, c_void_p(0), 0, _ptr(out), m, n, k, splits,
                                                  chunk, self._stream()), "linear (few rows, partial sums)")
            return
        partial = self._gemm_partial(splits * m * n, x.device) if splits > 1 else None
        self._check(self.lib.wllm_gemm_skinny(_ptr(x), _ptr(w), tiled, _ptr(out), int(out.dtype == torch.bfloat16),
                                              _ptr(partial), m, n, k, splits, chunk, self._stream()),
                    "linear (few rows, matrix cores)")

    def linear(self, x, weight, out, tiles=None):
        self._on_gpu(x, weight, out, tiles)
        m, k = x.shape
        if x.dtype == torch.bfloat16:
            if self.skinny_takes(x.dtype, m, k):
                self._skinny(x, weight, out, tiles)
                return
            if self.tile_takes(x.dtype, m, weight.shape[0], k):
                # some hundred rows and a long K axis: the tiled product, its K axis in pieces whose
                # sums the caller adds, or a kernel here in their order
                n, splits = weight.shape[0], self.tile_splits(weight.shape[0], k, m)
                stack = out if out.dim() == 3 else torch.empty((splits, m, n), dtype=torch.float32, device=x.device)
                self._check(self.lib.wllm_gemm_tile(_ptr(x), _ptr(weight), None, _ptr(stack), m, n, k, splits, 0,
                                                    self._stream()), "linear (tiles, partial sums)")
                if out.dim() == 2:
                    self._check(self.lib.wllm_split_sum(_ptr(stack), _ptr(out), int(out.dtype == torch.bfloat16), m * n, splits,
                                                        self._stream()), "linear (sum of partial sums)")
                return
            if k % 32 == 0 and out.dtype == torch.float32 and self.skinny_split(weight.shape[0], k) == 1:
                # float32 results from bfloat16 operands (logits at many rows): the few-row kernel with a
                # workgroup per 64 rows, placed so that the weights come from HBM once
                self._skinny(x, weight, out, tiles)
                return
            if k % 32 == 0 and out.dtype == torch.float32:
                for r in range(0, m, 64):
                    self._skinny(x[r:r + 64], weight, out[r:r + 64], tiles)
                return
            if out.dtype == torch.bfloat16 and m > 64:
                # many rows: the library's matrix-core product (float32 accumulation)
                if self.library_events is not None:     # a measurement asked for the library's share of a step
                    begin, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                    begin.record()
                    torch.mm(x, weight.t(), out=out)
                    end.record()
                    self.library_events.append((begin, end))
                    return
                torch.mm(x, weight.t(), out=out)
                return
        # float32, few rows, a long K axis: the segments of K are summed by wavefronts of their own
        if x.dtype == torch.float32 and m <= self.F32_FEW_ROWS:
            n = weight.shape[0]
            segments = self.lib.wllm_gemm_f32_segments(m, n, k)
            if out.dim() == 3:      # the caller adds the segments' sums later
                self._check(self.lib.wllm_gemm_generic(_ptr(x), _ptr(weight), _ptr(tiles), 0, c_void_p(0), 0, _ptr(out), m, n, k,
                                                       self._stream()), "linear (float32, partial sums)")
                return
            if segments > 1 and segments * m * n > self.GEMM_PARTIAL_FLOATS:
                # more partial sums than the buffer holds: some rows at a time; a row's sums do not
                # depend on the rows beside it
                rows = self.GEMM_PARTIAL_FLOATS // (segments * n)
                if rows < 1:
                    raise KernelError(f"linear: {segments} segments of {n} columns need more than the "
                                      f"{self.GEMM_PARTIAL_FLOATS} floats of the split-sum buffer for one row")
                for r in range(0, m, rows):
                    self._generic(x[r:r + rows], weight, out[r:r + rows], segments, tiles)
                return
            self._generic(x, weight, out, segments, tiles)
            return
        self._generic(x, weight, out, 1)

    def _generic(self, x, weight, out, segments: int, tiles=None) -> None:
        m, n = x.shape[0], weight.shape[0]
        partial = self._gemm_partial(segments * m * n, x.device) if segments > 1 else None
        self._check(self.lib.wllm_gemm_generic(
            _ptr(x), _ptr(weight), _ptr(tiles) if x.dtype == torch.float32 else c_void_p(0), int(x.dtype == torch.bfloat16),
            _ptr(out), int(out.dtype == torch.bfloat16),
            _ptr(partial), m, n, x.shape[1], self._stream()), "linear")

    def gated_linear(self, x, weight, out, activation, scratch, tiles=None):
        self._on_gpu(x, weight, out, scratch, tiles)
        m, k = x.shape
        w, tiled = (tiles, 1) if tiles is not None else (weight, 0)
        if self.skinny_takes(x.dtype, m, k) and k % 64 == 0:
            self._check(self.lib.wllm_gemm_skinny_gated(
                _ptr(x), _ptr(w), tiled, _ptr(out), m, out.shape[1], k, ACTIVATIONS[activation],
                self.GATED_CHUNK[-(-m // 16)], self._stream()), "gated_linear (few rows, matrix cores)")
            return
        n = out.shape[1]
        if (x.dtype == torch.bfloat16 and 64 < m <= self.TILE_GATED_MAX_ROWS and k % 64 == 0
                and max(m, 2 * n) * k * 2 < 2 ** 32):
            # some hundred rows: the tiled product with the activation in its registers
            self._check(self.lib.wllm_gemm_tile(_ptr(x), _ptr(weight), _ptr(out), None, m, n, k, 1,
                                                1 + ACTIVATIONS[activation], self._stream()),
                        "gated_linear (tiles)")
            return
        # (the tile-major copy of a stacked float32 matrix is that of the one matrix it is; a bfloat16 one's
        # halves are tiled each by itself, which only the gated kernels above read)
        self.linear(x, weight, scratch, tiles if x.dtype == torch.float32 else None)
        ops.call("gated_activation", scratch, out, activation)

    @staticmethod
    def gated_linear_norm_takes(rows: int, dtype, in_features: int) -> bool:
        """The gated product with the norm folded into its load of x: bfloat16, at most 16 rows,
        input size a multiple of 512 (whole chunks of 256 keys per half of the K axis)."""
        return dtype == torch.bfloat16 and 1 <= rows <= 16 and in_features % 512 == 0

    def gated_linear_norm(self, x, weight, out, activation, tiles=None):
        self._on_gpu(x.residual, x.sumsq, x.weight, weight, out, tiles)
        w, tiled = (tiles, 1) if tiles is not None else (weight, 0)
        self._check(self.lib.wllm_gemm_skinny_gated_norm(
            _ptr(x.residual), _ptr(x.sumsq), x.sumsq.shape[1], _ptr(x.weight), x.eps, x.offset, _ptr(w), tiled,
            _ptr(out), x.shape[0], out.shape[1], x.shape[1], ACTIVATIONS[activation], self._stream()),
            "gated_linear (norm on load)")

    ARGMAX_ROWS = 4096       # rows per launch; the scratch (64 words a row) is allocated once

    def argmax_rows(self, logits, out):
        self._on_gpu(logits, out)
        if self._argmax_scratch is None or self._argmax_scratch.device != logits.device:
            self._argmax_scratch = torch.empty(self.ARGMAX_ROWS * 64, dtype=torch.int32, device=logits.device)
        for r in range(0, logits.shape[0], self.ARGMAX_ROWS):
            rows = min(self.ARGMAX_ROWS, logits.shape[0] - r)
            self._check(self.lib.wllm_argmax_rows(_ptr(logits[r:r + rows]), _ptr(out[r:r + rows]),
                                                  _ptr(self._argmax_scratch), rows, logits.shape[1], self._stream()),
                        "argmax_rows")

    SAMPLE_SPLIT_ROWS = 256     # up to this many rows each row is spread over many workgroups

    def sample_rows(self, logits, params, seeds, penalty_ids, penalty_offsets, out_tokens, out_logprobs,
                    truncations=True):
        self._on_gpu(logits, params, seeds, penalty_ids, penalty_offsets, out_tokens, out_logprobs)
        rows, vocab = logits.shape
        if rows <= self.SAMPLE_SPLIT_ROWS:
            # a decode step's few rows: one workgroup a row would leave the chip idle
            if self._sample_scratch is None or self._sample_scratch.device != logits.device:
                words = self.lib.wllm_sample_split_row_words()
                self._sample_scratch = torch.empty(self.SAMPLE_SPLIT_ROWS * words, dtype=torch.int64,
                                                   device=logits.device)
            self._check(self.lib.wllm_sample_rows_split(
                _ptr(logits), _ptr(params), _ptr(seeds), _ptr(penalty_ids), _ptr(penalty_offsets), _ptr(out_tokens),
                _ptr(out_logprobs), _ptr(self._sample_scratch), rows, vocab, int(bool(truncations)), self._stream()),
                "sample_rows (rows spread over workgroups)")
            return
        self._check(self.lib.wllm_sample_rows(
            _ptr(logits), _ptr(params), _ptr(seeds), _ptr(penalty_ids), _ptr(penalty_offsets), _ptr(out_tokens),
            _ptr(out_logprobs), rows, vocab, self._stream()), "sample_rows")
