// Paged attention for any element type, head size (a multiple of 4, at most 256), page size
// and grouping of heads, in float32 arithmetic throughout.  It is the kernel of the float32
// path and of sizes the matrix-core kernels refuse.
//
// One workgroup (16 wavefronts) per (token, key/value head).  The token's position p follows
// from its segment: p = ctx_len - q_len + i; it sees keys lo..p with lo = max(0, p - window + 1).
// Each wavefront takes tiles of 64 consecutive keys: lane = key for the scores (a lane reads
// its key's row of the page, [page_size, head_dim]), lane = element of the head for the
// weighted sum (a lane reads its row of the transposed values, [head_dim, page_size]).  The
// query heads of the group, up to 8 at a time, share each key and value read.  Running maximum,
// running sum and accumulator are kept per wavefront and merged through shared memory; the
// order of all sums is fixed by the key index, so a query's result does not depend on what
// else is in the batch.
#include "common.h"

constexpr int kGroupMax = 8;     // query heads handled per pass over the keys
constexpr int kWaves = 16;      // a decode step has few (token, key/value head) pairs: many wavefronts each
constexpr int kMaxHeadDim = 256;

template <typename T> struct Vec4;
template <> struct Vec4<float> {
    float4 v;
    __device__ __forceinline__ float get(int i) const { return i == 0 ? v.x : (i == 1 ? v.y : (i == 2 ? v.z : v.w)); }
};
template <> struct Vec4<bf16> {
    uint2 v;
    __device__ __forceinline__ float get(int i) const {
        const uint32_t w = i < 2 ? v.x : v.y;
        return __uint_as_float((i & 1) ? (w & 0xffff0000u) : (w << 16));
    }
};

template <typename T, int DPL>   // DPL: elements of the head per lane (head_dim <= 64*DPL)
__global__ void __launch_bounds__(kWave * kWaves)
paged_attention_generic_kernel(const T* __restrict__ qkv, const T* __restrict__ cache,
                               const int* __restrict__ block_tables, const int* __restrict__ token_segment,
                               const int* __restrict__ seg_q_start, const int* __restrict__ seg_q_len,
                               const int* __restrict__ seg_ctx_len, T* __restrict__ out, int num_heads,
                               int num_kv_heads, int head_dim, int page_size, int max_pages, float scale,
                               int window, int group_begin) {
    extern __shared__ float smem[];
    const int token = blockIdx.x, kvh = blockIdx.y;
    const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
    const int group = num_heads / num_kv_heads;
    const int g_count = min(kGroupMax, group - group_begin);   // heads of this pass
    const int seg = token_segment[token];
    const int q_len = seg_q_len[seg], ctx = seg_ctx_len[seg];
    const int pos = ctx - q_len + (token - seg_q_start[seg]);
    const int lo = window > 0 ? max(0, pos - window + 1) : 0;
    const int* table = block_tables + static_cast<size_t>(seg) * max_pages;
    const int width = (num_heads + 2 * num_kv_heads) * head_dim;
    const size_t page_elems = static_cast<size_t>(2) * num_kv_heads * page_size * head_dim;
    const size_t k_off = static_cast<size_t>(kvh) * page_size * head_dim;
    const size_t v_off = (static_cast<size_t>(num_kv_heads) + kvh) * page_size * head_dim;

    // shared memory: queries [g][d] | per wave probabilities [g][64] | per wave key offsets [64] x2
    float* q_s = smem;
    float* p_s = q_s + kGroupMax * head_dim + wave * (kGroupMax * kWave);
    long long* koff_all = reinterpret_cast<long long*>(q_s + kGroupMax * head_dim + kWaves * kGroupMax * kWave);
    long long* koff_s = koff_all + wave * kWave;
    int* slot_s = reinterpret_cast<int*>(koff_all + kWaves * kWave) + wave * kWave;

    const T* qrow = qkv + static_cast<size_t>(token) * width + static_cast<size_t>(kvh * group + group_begin) * head_dim;
    for (int i = threadIdx.x; i < g_count * head_dim; i += blockDim.x) q_s[i] = to_float(qrow[i]);
    __syncthreads();

    float m[kGroupMax], l[kGroupMax], acc[kGroupMax][DPL];
#pragma unroll
    for (int g = 0; g < kGroupMax; ++g) {
        m[g] = -INFINITY;
        l[g] = 0.f;
#pragma unroll
        for (int k = 0; k < DPL; ++k) acc[g][k] = 0.f;
    }

    const int num_tiles = (pos - lo + kWave) / kWave;    // ceil((pos - lo + 1) / 64)
    for (int tile = wave; tile < num_tiles; tile += kWaves) {
        const int key = lo + tile * kWave + lane;
        const bool valid = key <= pos;
        float s[kGroupMax];
#pragma unroll
        for (int g = 0; g < kGroupMax; ++g) s[g] = 0.f;
        long long page_base = 0;
        int slot = 0;
        if (valid) {
            const int page = table[key / page_size];
            slot = key % page_size;
            page_base = static_cast<long long>(page) * static_cast<long long>(page_elems);
            const T* krow = cache + page_base + k_off + static_cast<size_t>(slot) * head_dim;
            // four loads of the key's row are asked for before the first is used
            for (int d0 = 0; d0 < head_dim; d0 += 16) {
                Vec4<T> kv[4];
#pragma unroll
                for (int u = 0; u < 4; ++u)
                    kv[u].v = *reinterpret_cast<const decltype(kv[u].v)*>(krow + min(d0 + 4 * u, head_dim - 4));
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    const int d = d0 + 4 * u;
                    if (d < head_dim) {
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            const float kf = kv[u].get(e);
#pragma unroll
                            for (int g = 0; g < kGroupMax; ++g)
                                if (g < g_count) s[g] = fmaf(q_s[g * head_dim + d + e], kf, s[g]);
                        }
                    }
                }
            }
        }
        koff_s[lane] = page_base;
        slot_s[lane] = slot;
        // online softmax over the tile, per head
        float alpha[kGroupMax];
#pragma unroll
        for (int g = 0; g < kGroupMax; ++g) {
            if (g < g_count) {
                const float sc = valid ? s[g] * scale : -INFINITY;
                const float m_new = fmaxf(m[g], wave_max(sc));
                const float p = valid ? expf(sc - m_new) : 0.f;
                alpha[g] = expf(m[g] - m_new);      // exp(-inf) = 0 on the first tile
                l[g] = l[g] * alpha[g] + wave_sum(p);
                m[g] = m_new;
                p_s[g * kWave + lane] = p;
            }
        }
        __builtin_amdgcn_wave_barrier();
        // weighted sum: lane = element of the head
        const int keys_here = min(kWave, pos - (lo + tile * kWave) + 1);
#pragma unroll
        for (int k = 0; k < DPL; ++k) {
            const int d = lane + k * kWave;
            if (d < head_dim) {
                float a[kGroupMax];
#pragma unroll
                for (int g = 0; g < kGroupMax; ++g) a[g] = acc[g][k] * (g < g_count ? alpha[g] : 0.f);
                // eight keys' values are asked for before the first is used; beyond the tile's last
                // key the last one is read again and meets a probability of zero
                for (int j0 = 0; j0 < keys_here; j0 += 8) {
                    float vf[8];
#pragma unroll
                    for (int u = 0; u < 8; ++u) {
                        const int j = min(j0 + u, keys_here - 1);
                        vf[u] = to_float(cache[koff_s[j] + v_off + static_cast<size_t>(d) * page_size + slot_s[j]]);
                    }
#pragma unroll
                    for (int u = 0; u < 8; ++u)
#pragma unroll
                        for (int g = 0; g < kGroupMax; ++g)
                            if (g < g_count) a[g] = fmaf(p_s[g * kWave + j0 + u], vf[u], a[g]);
                }
#pragma unroll
                for (int g = 0; g < kGroupMax; ++g) acc[g][k] = a[g];
            }
        }
        __builtin_amdgcn_wave_barrier();
    }

    // merge the wavefronts, in their order: (m, l) of all heads at once, the accumulators head by
    // head through one buffer of [waves][head_dim]
    __syncthreads();
    float* ml_s = smem;                                              // [waves][g][2]
    float* acc_s = smem + kWaves * kGroupMax * 2;                    // [waves][head_dim]
    if (lane == 0) {
#pragma unroll
        for (int g = 0; g < kGroupMax; ++g) {
            ml_s[(wave * kGroupMax + g) * 2] = m[g];
            ml_s[(wave * kGroupMax + g) * 2 + 1] = l[g];
        }
    }
    T* orow = out + static_cast<size_t>(token) * num_heads * head_dim + static_cast<size_t>(kvh * group + group_begin) * head_dim;
#pragma unroll
    for (int g = 0; g < kGroupMax; ++g) {
        if (g >= g_count) break;
#pragma unroll
        for (int k = 0; k < DPL; ++k) {
            const int d = lane + k * kWave;
            if (d < head_dim) acc_s[wave * head_dim + d] = acc[g][k];
        }
        __syncthreads();
        for (int d = threadIdx.x; d < head_dim; d += blockDim.x) {
            float mm = -INFINITY;
            for (int w = 0; w < kWaves; ++w) mm = fmaxf(mm, ml_s[(w * kGroupMax + g) * 2]);
            float num = 0.f, den = 0.f;
            for (int w = 0; w < kWaves; ++w) {
                const float mw = ml_s[(w * kGroupMax + g) * 2];
                const float f = mw == -INFINITY ? 0.f : expf(mw - mm);
                num = fmaf(acc_s[w * head_dim + d], f, num);
                den = fmaf(ml_s[(w * kGroupMax + g) * 2 + 1], f, den);
            }
            orow[g * head_dim + d] = from_float<T>(num / den);
        }
        __syncthreads();
    }
}

static size_t generic_smem_bytes(int head_dim) {
    const size_t main_loop = sizeof(float) * (kGroupMax * head_dim + kWaves * kGroupMax * kWave) +
                             sizeof(long long) * kWaves * kWave + sizeof(int) * kWaves * kWave;
    const size_t merge = sizeof(float) * (kWaves * kGroupMax * 2 + kWaves * head_dim);
    return main_loop > merge ? main_loop : merge;
}

// Returns 0, a HIP error code, or -1 for a size the kernel does not take.
WLLM_API int wllm_paged_attention_generic(const void* qkv, const void* cache, int is_bf16, const int* block_tables,
                                          const int* token_segment, const int* seg_q_start, const int* seg_q_len,
                                          const int* seg_ctx_len, void* out, int n, int num_heads, int num_kv_heads,
                                          int head_dim, int page_size, int max_pages, float scale, int window,
                                          hipStream_t stream) {
    if (head_dim <= 0 || head_dim % 4 != 0 || head_dim > kMaxHeadDim || num_heads % num_kv_heads != 0) return -1;
    const int group = num_heads / num_kv_heads;
    const dim3 grid(n, num_kv_heads);
    const size_t smem = generic_smem_bytes(head_dim);
    const int dpl = (head_dim + kWave - 1) / kWave;
    for (int gb = 0; gb < group; gb += kGroupMax) {
#define LAUNCH(T, D)                                                                                               \
    paged_attention_generic_kernel<T, D><<<grid, kWave * kWaves, smem, stream>>>(                                   \
        static_cast<const T*>(qkv), static_cast<const T*>(cache), block_tables, token_segment, seg_q_start,        \
        seg_q_len, seg_ctx_len, static_cast<T*>(out), num_heads, num_kv_heads, head_dim, page_size, max_pages, scale, \
        window, gb)
        if (is_bf16) {
            if (dpl == 1) LAUNCH(bf16, 1);
            else if (dpl == 2) LAUNCH(bf16, 2);
            else LAUNCH(bf16, 4);
        } else {
            if (dpl == 1) LAUNCH(float, 1);
            else if (dpl == 2) LAUNCH(float, 2);
            else LAUNCH(float, 4);
        }
#undef LAUNCH
        const int err = launch_status();
        if (err) return err;
    }
    return 0;
}
