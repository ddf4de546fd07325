// Paged attention for any element type, head size (a multiple of 4, at most 256), page size
// and grouping of heads, in float32 arithmetic throughout.  It is the kernel of the float32
// path and of sizes the matrix-core kernels refuse.
//
// A token at position p (from its segment: p = ctx_len - q_len + i) sees keys lo..p with
// lo = max(0, p - window + 1).  The keys are cut into chunks of kChunkKeys keys counted from
// key 0, so a chunk's boundaries depend on the key index alone.  One workgroup takes one
// (token, key/value head, chunk); its eight wavefronts take 16 keys each, and a wavefront's
// work is two trips to memory: the rows of its 16 keys (lane = key and quarter of the
// head, 16-byte loads) and, asked for once the scores are made, their values from the transposed
// page ([head_dim, page_size]; lane = element of the head, four consecutive keys a load where pages
// are a multiple of four keys).  Keys and values are not held at once: at a head of 256 that is 126
// registers instead of 168 and two workgroups a compute unit instead of one, which hide each other's trips.
// The query heads of the group, up to 8 at a time, share each key and value read.  The
// wavefronts' (maximum, sum, weighted sum) are merged through shared memory in wavefront
// order.  A token whose keys lie in one chunk is finished there; otherwise the chunk's
// unnormalised result goes to a partial buffer and a second kernel combines a token's chunks in
// ascending order.  The order of every sum is fixed by the key index, so a query's result does
// not depend on what else is in the batch, nor on whether it is decoded alone or inside a prompt.
#include "common.h"

constexpr int kGroupMax = 8;          // query heads handled per pass over the keys
constexpr int kChunkKeys = 128;       // keys per workgroup
constexpr int kTileKeys = 16;         // keys per wavefront
constexpr int kWaves = kChunkKeys / kTileKeys;
constexpr int kMaxHeadDim = 256;
constexpr int kMergeHeads = 4;        // heads whose weighted sums the wavefronts merge at a time

template <typename T> struct Vec4;
template <> struct Vec4<float> {
    float4 v;
    __device__ __forceinline__ float get(int i) const { return i == 0 ? v.x : (i == 1 ? v.y : (i == 2 ? v.z : v.w)); }
    __device__ __forceinline__ void zero() { v = make_float4(0.f, 0.f, 0.f, 0.f); }
    __device__ __forceinline__ void load(const float* p) { v = *reinterpret_cast<const float4*>(p); }
    __device__ __forceinline__ void gather(const float* p0, const float* p1, const float* p2, const float* p3) {
        v = make_float4(*p0, *p1, *p2, *p3);
    }
};
template <> struct Vec4<bf16> {
    uint2 v;
    __device__ __forceinline__ float get(int i) const {
        const uint32_t w = i < 2 ? v.x : v.y;
        return __uint_as_float((i & 1) ? (w & 0xffff0000u) : (w << 16));
    }
    __device__ __forceinline__ void zero() { v = make_uint2(0u, 0u); }
    __device__ __forceinline__ void load(const bf16* p) { v = *reinterpret_cast<const uint2*>(p); }
    __device__ __forceinline__ void gather(const bf16* p0, const bf16* p1, const bf16* p2, const bf16* p3) {
        v = make_uint2(static_cast<uint32_t>(p0->bits) | (static_cast<uint32_t>(p1->bits) << 16),
                       static_cast<uint32_t>(p2->bits) | (static_cast<uint32_t>(p3->bits) << 16));
    }
};

// NV: groups of four elements of a key's row per lane (head_dim <= 16 * NV); DPL: elements of the
// head per lane in the weighted sum (head_dim <= 64 * DPL); VEC4: pages hold a multiple of four
// keys, so four consecutive keys' values of one element are one load.
template <typename T, int NV, int DPL, bool VEC4>
__global__ void __launch_bounds__(kWave * kWaves, 4)
paged_attention_generic_kernel(const T* __restrict__ qkv, const T* __restrict__ cache,
                               const int* __restrict__ block_tables, const int* __restrict__ token_segment,
                               const int* __restrict__ seg_q_start, const int* __restrict__ seg_q_len,
                               const int* __restrict__ seg_ctx_len, T* __restrict__ out,
                               float* __restrict__ partial_o, float* __restrict__ partial_ml, int token_begin,
                               int max_chunks, int num_heads, int num_kv_heads, int head_dim, int page_size,
                               int max_pages, float scale, int window, int group_begin) {
    const int token = token_begin + blockIdx.x, kvh = blockIdx.y, chunk = blockIdx.z;
    const int seg = token_segment[token];
    const int q_len = seg_q_len[seg], ctx = seg_ctx_len[seg];
    const int pos = ctx - q_len + (token - seg_q_start[seg]);
    const int lo = window > 0 ? max(0, pos - window + 1) : 0;
    const int c_lo = lo / kChunkKeys, c_hi = min(pos / kChunkKeys, max_chunks - 1);   // the bound keeps every access inside the buffers
    if (chunk < c_lo || chunk > c_hi) return;
    // the caller's bound on the context lengths was below this token's: its keys beyond the bound are not
    // read, and its result is made NaN (through the last chunk's sums), not a number that looks right
    const bool cut_short = pos / kChunkKeys > max_chunks - 1;

    extern __shared__ float smem[];
    const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
    const int group = num_heads / num_kv_heads;
    const int g_count = min(kGroupMax, group - group_begin);   // heads of this pass
    const int* table = block_tables + static_cast<size_t>(seg) * max_pages;
    const int width = (num_heads + 2 * num_kv_heads) * head_dim;
    const size_t page_elems = static_cast<size_t>(2) * num_kv_heads * page_size * head_dim;
    const size_t k_off = static_cast<size_t>(kvh) * page_size * head_dim;
    const size_t v_off = (static_cast<size_t>(num_kv_heads) + kvh) * page_size * head_dim;

    // shared memory: queries [g][d] | per wave probabilities [g][16] | per wave page offsets [16], slots [16]
    float* q_s = smem;
    float* p_s = q_s + kGroupMax * head_dim + wave * (kGroupMax * kTileKeys);
    long long* koff_all = reinterpret_cast<long long*>(q_s + kGroupMax * head_dim + kWaves * kGroupMax * kTileKeys);
    long long* koff_s = koff_all + wave * kTileKeys;
    int* slot_s = reinterpret_cast<int*>(koff_all + kWaves * kTileKeys) + wave * kTileKeys;

    const T* qrow = qkv + static_cast<size_t>(token) * width + static_cast<size_t>(kvh * group + group_begin) * head_dim;
    for (int i = threadIdx.x; i < g_count * head_dim; i += blockDim.x) q_s[i] = to_float(qrow[i]);

    // ---- this wavefront's 16 keys: where they are ----
    const int key0 = chunk * kChunkKeys + wave * kTileKeys;
    const int j = lane / 4, c = lane % 4;                    // key of the tile, quarter of its row
    const int key = key0 + j;
    const bool valid = key >= lo && key <= pos;
    long long page_base = 0;
    int slot = 0;
    if (valid) {
        slot = key % page_size;
        page_base = static_cast<long long>(table[key / page_size]) * static_cast<long long>(page_elems);
    }
    if (c == 0) {
        koff_s[j] = page_base;
        slot_s[j] = slot;
    }
    // ---- loads: the keys' rows, then the values ----
    const int n4 = head_dim / 4;
    Vec4<T> kvec[NV];
    {
        const T* krow = cache + page_base + k_off + static_cast<size_t>(slot) * head_dim;
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            const int idx = i * 4 + c;
            if (valid && idx < n4) kvec[i].load(krow + idx * 4);
            else kvec[i].zero();
        }
    }
    __syncthreads();                       // queries, offsets and slots are in shared memory
    // ---- scores: a lane's part of the dot products, then the sum over the four lanes of a key ----
    float s[kGroupMax];
#pragma unroll
    for (int g = 0; g < kGroupMax; ++g) s[g] = 0.f;
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const int idx = i * 4 + c;
        if (idx < n4) {
#pragma unroll
            for (int g = 0; g < kGroupMax; ++g) {
                if (g < g_count) {
                    const float4 qv = *reinterpret_cast<const float4*>(q_s + g * head_dim + idx * 4);
                    s[g] = fmaf(qv.x, kvec[i].get(0), s[g]);
                    s[g] = fmaf(qv.y, kvec[i].get(1), s[g]);
                    s[g] = fmaf(qv.z, kvec[i].get(2), s[g]);
                    s[g] = fmaf(qv.w, kvec[i].get(3), s[g]);
                }
            }
        }
    }
    float m[kGroupMax], l[kGroupMax];
#pragma unroll
    for (int g = 0; g < kGroupMax; ++g) {
        m[g] = -INFINITY;
        l[g] = 0.f;
        if (g < g_count) {
            float t = s[g];
            t += __shfl_xor(t, 1, kWave);
            t += __shfl_xor(t, 2, kWave);
            const float sc = valid ? t * scale : -INFINITY;
            m[g] = wave_max(sc);
            const float p = valid ? expf(sc - m[g]) : 0.f;        // m is finite if any key of the tile is valid
            l[g] = wave_sum(c == 0 ? p : 0.f);
            if (c == 0) p_s[g * kTileKeys + j] = p;
        }
    }
    const int keys_before = key0 < lo ? lo - key0 : 0;                     // keys of the tile below the window
    const int keys_end = min(kTileKeys, pos - key0 + 1);                   // keys of the tile up to the token's own
    Vec4<T> vvec[DPL][kTileKeys / 4];
#pragma unroll
    for (int k = 0; k < DPL; ++k) {
        const int d = lane + k * kWave;
#pragma unroll
        for (int jj = 0; jj < kTileKeys / 4; ++jj) {
            const int j0 = jj * 4;
            vvec[k][jj].zero();
            if (d < head_dim && j0 < keys_end && j0 + 4 > keys_before) {
                if (VEC4) {
                    // four consecutive keys lie in one page; the first valid one says which
                    const int jv = max(j0, keys_before);
                    vvec[k][jj].load(cache + koff_s[jv] + v_off + static_cast<size_t>(d) * page_size + (slot_s[jv] - (jv - j0)));
                } else {
                    const T* p[4];
#pragma unroll
                    for (int u = 0; u < 4; ++u) {
                        const int ju = min(max(j0 + u, keys_before), keys_end - 1);     // an invalid key reads a valid one's
                        p[u] = cache + koff_s[ju] + v_off + static_cast<size_t>(d) * page_size + slot_s[ju];
                    }
                    vvec[k][jj].gather(p[0], p[1], p[2], p[3]);
                }
            }
        }
    }

    // lanes read below what other lanes of the wavefront wrote above: no reordering by the
    // scheduler, and the compiler is told that the memory changed
    __builtin_amdgcn_wave_barrier();
    asm volatile("" ::: "memory");

    // ---- weighted sum: lane = element of the head; the keys in ascending order ----
    float acc[kGroupMax][DPL];
#pragma unroll
    for (int g = 0; g < kGroupMax; ++g)
#pragma unroll
        for (int k = 0; k < DPL; ++k) acc[g][k] = 0.f;
#pragma unroll
    for (int jj = 0; jj < kTileKeys / 4; ++jj) {
#pragma unroll
        for (int g = 0; g < kGroupMax; ++g) {
            if (g < g_count) {
                const float4 pv = *reinterpret_cast<const float4*>(p_s + g * kTileKeys + jj * 4);
                const float pj[4] = {pv.x, pv.y, pv.z, pv.w};
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    const int ju = jj * 4 + u;
                    const bool live = ju >= keys_before && ju < keys_end;      // a stale slot may hold anything
#pragma unroll
                    for (int k = 0; k < DPL; ++k) {
                        const float vf = live ? vvec[k][jj].get(u) : 0.f;
                        acc[g][k] = fmaf(pj[u], vf, acc[g][k]);
                    }
                }
            }
        }
    }

    // ---- merge the wavefronts, in their order: (m, l) of all heads at once, the weighted sums of
    // kMergeHeads heads at a time through one buffer of [waves][kMergeHeads][head_dim] (two barriers a
    // batch of heads: a head at a time they were 16 barriers for a group of 8, a third of the kernel) ----
    __syncthreads();
    float* ml_s = smem;                                              // [waves][g][2]
    float* acc_s = smem + kWaves * kGroupMax * 2;                    // [waves][kMergeHeads][head_dim]
    if (lane == 0) {
#pragma unroll
        for (int g = 0; g < kGroupMax; ++g) {
            ml_s[(wave * kGroupMax + g) * 2] = m[g];
            ml_s[(wave * kGroupMax + g) * 2 + 1] = l[g];
        }
    }
    const bool whole = c_lo == c_hi;                                 // the token's only chunk: finish here
    const int head0 = kvh * group + group_begin;
    T* orow = out + static_cast<size_t>(token) * num_heads * head_dim + static_cast<size_t>(head0) * head_dim;
    const size_t part_row = (static_cast<size_t>(blockIdx.x) * num_heads + head0) * max_chunks + chunk;
    const size_t part_stride = max_chunks;                          // between two heads of a token
#pragma unroll
    for (int g0 = 0; g0 < kGroupMax; g0 += kMergeHeads) {
        if (g0 >= g_count) break;
#pragma unroll
        for (int gi = 0; gi < kMergeHeads; ++gi) {
#pragma unroll
            for (int k = 0; k < DPL; ++k) {
                const int d = lane + k * kWave;
                if (d < head_dim && g0 + gi < g_count) acc_s[(wave * kMergeHeads + gi) * head_dim + d] = acc[g0 + gi][k];
            }
        }
        __syncthreads();
        for (int e = threadIdx.x; e < kMergeHeads * head_dim; e += blockDim.x) {
            const int gi = e / head_dim, d = e - gi * head_dim, g = g0 + gi;
            if (g >= g_count) continue;
            float mm = -INFINITY;
            for (int w = 0; w < kWaves; ++w) mm = fmaxf(mm, ml_s[(w * kGroupMax + g) * 2]);
            float num = 0.f, den = 0.f;
            for (int w = 0; w < kWaves; ++w) {
                const float mw = ml_s[(w * kGroupMax + g) * 2];
                const float f = mw == -INFINITY ? 0.f : expf(mw - mm);
                num = fmaf(acc_s[(w * kMergeHeads + gi) * head_dim + d], f, num);
                den = fmaf(ml_s[(w * kGroupMax + g) * 2 + 1], f, den);
            }
            if (cut_short) num = __builtin_nanf("");
            if (whole) {
                orow[g * head_dim + d] = from_float<T>(num / den);
            } else {
                const size_t row = part_row + g * part_stride;
                partial_o[row * head_dim + d] = num;
                if (d == 0) {
                    partial_ml[row * 2] = mm;
                    partial_ml[row * 2 + 1] = den;
                }
            }
        }
        __syncthreads();
    }
}

// Combines the chunks of the tokens whose keys span more than one, in ascending order of the chunks.
// One workgroup per (token, head); a thread per element of the head.
template <typename T>
__global__ void __launch_bounds__(kMaxHeadDim)
paged_attention_generic_reduce_kernel(const float* __restrict__ partial_o, const float* __restrict__ partial_ml,
                                      const int* __restrict__ token_segment, const int* __restrict__ seg_q_start,
                                      const int* __restrict__ seg_q_len, const int* __restrict__ seg_ctx_len,
                                      T* __restrict__ out, int token_begin, int max_chunks, int num_heads, int head_dim,
                                      int window) {
    const int token = token_begin + blockIdx.x, head = blockIdx.y;
    const int seg = token_segment[token];
    const int pos = seg_ctx_len[seg] - seg_q_len[seg] + (token - seg_q_start[seg]);
    const int lo = window > 0 ? max(0, pos - window + 1) : 0;
    const int c_lo = lo / kChunkKeys, c_hi = min(pos / kChunkKeys, max_chunks - 1);   // the bound keeps every access inside the buffers
    if (c_lo == c_hi) return;
    const size_t row0 = (static_cast<size_t>(blockIdx.x) * num_heads + head) * max_chunks;
    float mm = -INFINITY;
    for (int ch = c_lo; ch <= c_hi; ++ch) mm = fmaxf(mm, partial_ml[(row0 + ch) * 2]);
    const int d = threadIdx.x;
    if (d >= head_dim) return;
    float num = 0.f, den = 0.f;
    for (int ch = c_lo; ch <= c_hi; ++ch) {
        const float f = expf(partial_ml[(row0 + ch) * 2] - mm);
        num = fmaf(partial_o[(row0 + ch) * head_dim + d], f, num);
        den = fmaf(partial_ml[(row0 + ch) * 2 + 1], f, den);
    }
    out[(static_cast<size_t>(token) * num_heads + head) * head_dim + d] = from_float<T>(num / den);
}

static size_t generic_smem_bytes(int head_dim) {
    const size_t main_part = sizeof(float) * (kGroupMax * head_dim + kWaves * kGroupMax * kTileKeys) +
                             sizeof(long long) * kWaves * kTileKeys + sizeof(int) * kWaves * kTileKeys;
    const size_t merge = sizeof(float) * (kWaves * kGroupMax * 2 + kWaves * kMergeHeads * head_dim);
    return main_part > merge ? main_part : merge;
}

// Floats of the two partial buffers one token needs when its keys may span `max_chunks` chunks.
WLLM_API int wllm_paged_attention_generic_chunk_keys() { return kChunkKeys; }

// Returns 0, a HIP error code, or -1 for a size the kernel does not take.  `max_ctx_len` bounds every
// segment's context length (it sets the number of chunks in the grid; the lengths themselves are in
// device memory, so a bound that is too low shows as NaN in the tokens it cuts short).  partial_o holds
// partial_tokens * num_heads * max_chunks * head_dim floats and partial_ml partial_tokens * num_heads *
// max_chunks * 2, with max_chunks = ceil(max_ctx_len / chunk keys); the tokens run in launches of
// at most `partial_tokens`.
WLLM_API int wllm_paged_attention_generic(const void* qkv, const void* cache, int is_bf16, const int* block_tables,
                                          const int* token_segment, const int* seg_q_start, const int* seg_q_len,
                                          const int* seg_ctx_len, void* out, void* partial_o, void* partial_ml,
                                          int partial_tokens, int max_ctx_len, int n, int num_heads, int num_kv_heads,
                                          int head_dim, int page_size, int max_pages, float scale, int window,
                                          hipStream_t stream) {
    if (head_dim <= 0 || head_dim % 4 != 0 || head_dim > kMaxHeadDim || num_heads % num_kv_heads != 0) return -1;
    if (partial_tokens < 1 || max_ctx_len < 1 || !partial_o || !partial_ml) return -1;
    const int group = num_heads / num_kv_heads;
    const int max_chunks = (max_ctx_len + kChunkKeys - 1) / kChunkKeys;
    if (max_chunks > 65535 || num_kv_heads > 65535 || num_heads > 65535) return -1;
    const size_t smem = generic_smem_bytes(head_dim);
    const int nv = head_dim <= 64 ? 4 : (head_dim <= 128 ? 8 : 16);
    const bool vec4 = page_size % 4 == 0;
    for (int t0 = 0; t0 < n; t0 += partial_tokens) {
        const int tokens = n - t0 < partial_tokens ? n - t0 : partial_tokens;
        const dim3 grid(tokens, num_kv_heads, max_chunks);
        for (int gb = 0; gb < group; gb += kGroupMax) {
#define LAUNCH(T, NV, DPL, V4)                                                                                          \
    paged_attention_generic_kernel<T, NV, DPL, V4><<<grid, kWave * kWaves, smem, stream>>>(                              \
        static_cast<const T*>(qkv), static_cast<const T*>(cache), block_tables, token_segment, seg_q_start, seg_q_len,  \
        seg_ctx_len, static_cast<T*>(out), static_cast<float*>(partial_o), static_cast<float*>(partial_ml), t0,         \
        max_chunks, num_heads, num_kv_heads, head_dim, page_size, max_pages, scale, window, gb)
#define LAUNCH_SIZES(T, V4)                         \
    if (nv == 4) LAUNCH(T, 4, 1, V4);               \
    else if (nv == 8) LAUNCH(T, 8, 2, V4);          \
    else LAUNCH(T, 16, 4, V4)
            if (is_bf16) {
                if (vec4) { LAUNCH_SIZES(bf16, true); } else { LAUNCH_SIZES(bf16, false); }
            } else {
                if (vec4) { LAUNCH_SIZES(float, true); } else { LAUNCH_SIZES(float, false); }
            }
#undef LAUNCH_SIZES
#undef LAUNCH
            if (const int err = launch_status()) return err;
        }
        if (max_chunks > 1) {
            const dim3 rgrid(tokens, num_heads);
            if (is_bf16)
                paged_attention_generic_reduce_kernel<bf16><<<rgrid, kMaxHeadDim, 0, stream>>>(
                    static_cast<const float*>(partial_o), static_cast<const float*>(partial_ml), token_segment, seg_q_start,
                    seg_q_len, seg_ctx_len, static_cast<bf16*>(out), t0, max_chunks, num_heads, head_dim, window);
            else
                paged_attention_generic_reduce_kernel<float><<<rgrid, kMaxHeadDim, 0, stream>>>(
                    static_cast<const float*>(partial_o), static_cast<const float*>(partial_ml), token_segment, seg_q_start,
                    seg_q_len, seg_ctx_len, static_cast<float*>(out), t0, max_chunks, num_heads, head_dim, window);
            if (const int err = launch_status()) return err;
        }
    }
    return 0;
}
