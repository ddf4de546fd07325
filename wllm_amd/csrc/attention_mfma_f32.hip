// Paged attention on the matrix cores in float32: the true 32-bit path's kernel for tiles of 16 query
// rows (decoded tokens, and prompts cut into such tiles), head sizes 32..256 in steps of 32, pages of a
// multiple of 4 tokens, any number of heads and groups, optional window.  Keys, values, queries, scores,
// probabilities and sums are IEEE float32 from end to end: v_mfma_f32_16x16x4_f32 multiplies and
// accumulates float32, nothing is rounded to a narrower format.
//
// Work items, rows and the partial results of items that share a tile of rows are those of the bfloat16
// kernel (`attention_mfma.hip`): one workgroup of four wavefronts per (tile of 16 rows, chunk of at most
// 128 keys within an aligned group of 128), a wavefront per block of 32 keys, merged through shared
// memory in the order of the wavefronts; tiles with several chunks leave (maximum, sum, accumulator)
// for the reduce kernel below.  The order of every sum depends on the key's index and the element's
// index only.
//
// Matrix products (64 lanes: i = lane % 16, g = lane / 16; an instruction sums over 4 values of k, one
// per lane group):
//   scores^T[key, row] = sum over the head's elements.  Lane group g takes the quarter
//       [g HD/4, (g+1) HD/4) of the head: step s multiplies A = K[key_i][g HD/4 + s] by
//       B = Q[row_i][g HD/4 + s], so a lane reads one contiguous quarter of its key's row from the
//       cache (16-byte loads) and nothing is staged.  The queries of the tile lie in shared memory
//       (all four wavefronts use the same 16 rows).
//       C: lane (i, g) holds the keys 4g..4g+3 of the tile of 16, row_i.
//   out^T[d, row] = sum over keys: step v takes, in lane group g, the key 4g + v of the tile:
//       B = the lane's own probability v (the registers the scores were made in), A = V^T[16t + i][key],
//       which the cache holds transposed ([head_dim, page_size]): a lane's four keys are one 16-byte load.
#include "common.h"

typedef float float4_t __attribute__((ext_vector_type(4)));

namespace {

constexpr int kItemInts = 8;
constexpr int kRowsPerTile = 16;
constexpr int kKeysPerBlock = 32;

template <int HD>
__global__ void __launch_bounds__(256, 2)
paged_attention_f32_kernel(const float* __restrict__ qkv, const float* __restrict__ cache,
                           const int* __restrict__ block_tables, const int* __restrict__ items,
                           const int* __restrict__ live_items, float* __restrict__ out,
                           float* __restrict__ partial_o, float* __restrict__ partial_ml, int num_heads,
                           int num_kv_heads, int page_size, int max_pages, float scale_log2e, int window) {
    constexpr int DQ = HD / 4;                  // elements of a lane group's quarter of the head
    constexpr int DT = HD / 16;                 // 16-row tiles of out^T
    constexpr int kQStride = HD + 4;            // floats; rows 4 banks apart: 16 lanes' 16-byte reads meet no conflict
    constexpr int kMergeStride = HD / 2 + 4;
    __shared__ __align__(16) float q_s[kRowsPerTile * kQStride];
    __shared__ __align__(16) float merge_s[4][kRowsPerTile * kMergeStride];
    __shared__ float row_max_s[4][kRowsPerTile], row_sum_s[4][kRowsPerTile];

    const int* item = items + static_cast<size_t>(blockIdx.x) * kItemInts;
    const int seg = item[0], kvh = item[1] & 0xffff, q_len = item[2], q_start = item[3];
    const int key_begin = item[4], key_end = item[5], partial_slot = item[6], ctx = item[7];
    const int live = live_items != nullptr ? live_items[0] : 0x7fffffff;
    if (static_cast<int>(blockIdx.x) >= live) return;
    const int row_begin = (item[1] >> 16) * kRowsPerTile;     // the tile's number is in the item's high 16 bits
    if (seg < 0) return;    // padding item
    const int lane = threadIdx.x % kWave;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    const int i = lane % 16, g = lane / 16;

    const int group = num_heads / num_kv_heads;
    const int width = (num_heads + 2 * num_kv_heads) * HD;
    const int total_rows = q_len * group;
    const int first_pos = ctx - q_len;
    const int seg_lo = window > 0 ? max(0, first_pos - window + 1) : 0;   // keys below may be given back
    const int row = row_begin + i;
    const bool row_valid = row < total_rows;
    const int tok = row_valid ? row / group : 0;
    const int head = kvh * group + (row_valid ? row % group : 0);
    const int pos = first_pos + tok;
    const int lo = window > 0 ? max(0, pos - window + 1) : 0;
    const int blk_first = key_begin / kKeysPerBlock;
    const int blk_end = (key_end + kKeysPerBlock - 1) / kKeysPerBlock;
    const int blk = blk_first + wave;
    const bool has_block = blk < blk_end;
    const int kbase = blk * kKeysPerBlock;

    const size_t page_elems = static_cast<size_t>(2) * num_kv_heads * page_size * HD;
    const size_t k_off = static_cast<size_t>(kvh) * page_size * HD;
    const size_t v_off = (static_cast<size_t>(num_kv_heads) + kvh) * page_size * HD;
    const int* table = block_tables + static_cast<size_t>(seg) * max_pages;

    // ---- the keys of the wavefront's block are asked for first: a lane's quarter of the rows of the keys
    //      16 t2 + i.  A key beyond the table's width (it is masked) reads the last page the table names. ----
    float4_t kf[2][DQ / 4];
    if (has_block) {
#pragma unroll
        for (int t2 = 0; t2 < 2; ++t2) {
            const int key = kbase + 16 * t2 + i;
            const int page_index = key / page_size, slot = key - page_index * page_size;
            const float* krow = cache + static_cast<size_t>(table[min(page_index, max_pages - 1)]) * page_elems + k_off +
                                static_cast<size_t>(slot) * HD + g * DQ;
#pragma unroll
            for (int j = 0; j < DQ / 4; ++j) kf[t2][j] = *reinterpret_cast<const float4_t*>(krow + 4 * j);
        }
    }
    // ---- the tile's queries into shared memory, rows beyond the segment as zeros ----
    for (int idx = threadIdx.x; idx < kRowsPerTile * (HD / 4); idx += 256) {
        const int r = idx / (HD / 4), c4 = idx % (HD / 4);
        const int rr = row_begin + r;
        float4_t v = float4_t{0.f, 0.f, 0.f, 0.f};
        if (rr < total_rows)
            v = *reinterpret_cast<const float4_t*>(qkv + static_cast<size_t>(q_start + rr / group) * width +
                                                   static_cast<size_t>(kvh * group + rr % group) * HD + 4 * c4);
        *reinterpret_cast<float4_t*>(q_s + r * kQStride + 4 * c4) = v;
    }
    __syncthreads();

    float4_t acc[DT];
#pragma unroll
    for (int t = 0; t < DT; ++t) acc[t] = float4_t{0.f, 0.f, 0.f, 0.f};
    float m_run = -INFINITY, l_run = 0.f;
    if (has_block) {
        // ---- scores: two tiles of 16 keys ----
        float4_t s[2];
#pragma unroll
        for (int t2 = 0; t2 < 2; ++t2) {
            float4_t sc = float4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int j = 0; j < DQ / 4; ++j) {
                const float4_t q = *reinterpret_cast<const float4_t*>(q_s + i * kQStride + g * DQ + 4 * j);
#pragma unroll
                for (int e = 0; e < 4; ++e) sc = __builtin_amdgcn_mfma_f32_16x16x4f32(kf[t2][j][e], q[e], sc, 0, 0, 0);
            }
            s[t2] = sc;
        }
        // ---- the values' fragments: lane (i, g) takes, of row 16 t + i of the transposed values, the
        //      keys 16 t2 + 4 g .. + 3 (one page: pages are multiples of 4 keys and so is the first key) ----
        float4_t vf[2][DT];
#pragma unroll
        for (int t2 = 0; t2 < 2; ++t2) {
            const int key = kbase + 16 * t2 + 4 * g;
            const int page_index = key / page_size, slot = key - page_index * page_size;
            const float* vrow = cache + static_cast<size_t>(table[min(page_index, max_pages - 1)]) * page_elems + v_off + slot;
#pragma unroll
            for (int t = 0; t < DT; ++t)
                vf[t2][t] = *reinterpret_cast<const float4_t*>(vrow + static_cast<size_t>(16 * t + i) * page_size);
        }
        // ---- mask, maximum, probabilities: the lane's keys are 16 t2 + 4 g + v ----
        float pe[8];
        bool ok[8];
        float tile_max = -INFINITY;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const int key = kbase + 16 * (e / 4) + 4 * g + e % 4;
            ok[e] = row_valid && key <= pos && key >= lo && key >= key_begin && key < key_end;
            pe[e] = s[e / 4][e % 4];
            if (ok[e]) tile_max = fmaxf(tile_max, pe[e]);
        }
        tile_max = max_across(max_across(tile_max, 16), 32);
        m_run = tile_max;
        const float mc = (tile_max == -INFINITY ? 0.f : tile_max) * scale_log2e;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            pe[e] = ok[e] ? exp2f(fmaf(pe[e], scale_log2e, -mc)) : 0.f;
            l_run += pe[e];
        }
        l_run = sum_across(sum_across(l_run, 16), 32);
        // ---- out^T += V^T . P^T.  Keys outside the request (stale slots, pages given back) may hold
        //      anything, NaN included; 0 * NaN would poison the sum, so their values are cleared. ----
        const bool edge = kbase < seg_lo || kbase + kKeysPerBlock > ctx;
#pragma unroll
        for (int t2 = 0; t2 < 2; ++t2) {
#pragma unroll
            for (int t = 0; t < DT; ++t) {
                float4_t a = vf[t2][t];
                if (edge) {
#pragma unroll
                    for (int v = 0; v < 4; ++v) {
                        const int key = kbase + 16 * t2 + 4 * g + v;
                        if (key >= ctx || key < seg_lo) a[v] = 0.f;
                    }
                }
#pragma unroll
                for (int v = 0; v < 4; ++v) acc[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[v], pe[4 * t2 + v], acc[t], 0, 0, 0);
            }
        }
    }

    // ---- merge: every wavefront leaves its sums in its part of shared memory, one half of the head after
    //      the other; of each half every wavefront takes every fourth tile of 16 elements and combines the
    //      four wavefronts' sums of that tile, always in the order 0, 1, 2, 3.
    //      lane (i, g) holds out^T[16t + 4g + v][row i]: elements d = 16t + 4g + v of row i ----
    float* mine = merge_s[wave];
    if (g == 0) {
        row_max_s[wave][i] = m_run;
        row_sum_s[wave][i] = l_run;
    }
    float f_of[4] = {0.f, 0.f, 0.f, 0.f};
    float m_all = -INFINITY, l_all = 0.f, inv = 0.f;
    float* orow = out + (static_cast<size_t>(q_start + tok) * num_heads + head) * HD;
    const size_t prow = static_cast<size_t>(max(partial_slot, 0)) * kRowsPerTile + (row - row_begin);
    float* po = partial_o + prow * HD;
#pragma unroll
    for (int half = 0; half < 2; ++half) {
        if (half) __syncthreads();          // the first half has been read
#pragma unroll
        for (int t = 0; t < DT / 2; ++t)
            *reinterpret_cast<float4_t*>(mine + i * kMergeStride + t * 16 + 4 * g) = acc[half * (DT / 2) + t];
        __syncthreads();
        if (!half) {
            float m_of[4], l_of[4];
#pragma unroll
            for (int w = 0; w < 4; ++w) {
                m_of[w] = row_max_s[w][i];
                l_of[w] = row_sum_s[w][i];
                m_all = fmaxf(m_all, m_of[w]);
            }
            const float m_use = m_all == -INFINITY ? 0.f : m_all;
#pragma unroll
            for (int w = 0; w < 4; ++w) {
                f_of[w] = exp2f((m_of[w] - m_use) * scale_log2e);       // 0 for a wavefront without keys
                l_all = fmaf(l_of[w], f_of[w], l_all);
            }
            inv = 1.f / l_all;
        }
        if (row_valid) {
#pragma unroll
            for (int t0 = 0; t0 < DT / 2; t0 += 4) {
                const int t = t0 + wave;
                if (t < DT / 2) {
                    float4_t sum = float4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                    for (int w = 0; w < 4; ++w) {
                        const float4_t v = *reinterpret_cast<const float4_t*>(merge_s[w] + i * kMergeStride + t * 16 + 4 * g);
#pragma unroll
                        for (int e = 0; e < 4; ++e) sum[e] = fmaf(v[e], f_of[w], sum[e]);
                    }
                    const int d = (half * (DT / 2) + t) * 16 + 4 * g;
                    if (partial_slot < 0) {
                        *reinterpret_cast<float4_t*>(orow + d) = float4_t{sum[0] * inv, sum[1] * inv, sum[2] * inv, sum[3] * inv};
                    } else {
                        *reinterpret_cast<float4_t*>(po + d) = sum;
                    }
                }
            }
        }
    }
    if (row_valid && partial_slot >= 0 && wave == 0 && g == 0) {
        partial_ml[prow * 2] = m_all;
        partial_ml[prow * 2 + 1] = l_all;
    }
}

// Combines the partial results of a tile of rows whose keys were split over workgroups, in the order of
// the splits.  reduce items: seg, kvh, first partial slot, number of splits, first row, slots between
// splits, the segment's number of new tokens, the place of its first token among the step's tokens.
// One workgroup a (tile, four rows); a thread four consecutive elements of a row.
template <int HD>
__global__ void __launch_bounds__(HD)
attention_reduce_f32_kernel(const int* __restrict__ reduce_items, const float* __restrict__ partial_o,
                            const float* __restrict__ partial_ml, const int* __restrict__ seg_q_start,
                            const int* __restrict__ seg_q_len, float* __restrict__ out, int num_heads,
                            int num_kv_heads, float scale_log2e) {
    constexpr int kQuads = HD / 4;
    const int* item = reduce_items + static_cast<size_t>(blockIdx.x) * kItemInts;
    const int seg = item[0], kvh = item[1], first = item[2], splits = item[3], row0 = item[4];
    if (seg < 0) return;
    const size_t stride = static_cast<size_t>(item[5]) * kRowsPerTile;     // rows between two splits
    const int group = num_heads / num_kv_heads;
    const int r = blockIdx.y * 4 + threadIdx.x / kQuads, d = (threadIdx.x % kQuads) * 4;
    const int q_start = seg_q_start[seg];
    if (row0 + r >= seg_q_len[seg] * group) return;
    const float* ml = partial_ml + (static_cast<size_t>(first) * kRowsPerTile + r) * 2;
    const float* po = partial_o + (static_cast<size_t>(first) * kRowsPerTile + r) * HD + d;
    float m = -INFINITY, den = 0.f;
    float4_t num = float4_t{0.f, 0.f, 0.f, 0.f};
    for (int s0 = 0; s0 < splits; s0 += 8) {
        float ms[8], ls[8];
        float4_t ps[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const bool ok = s0 + u < splits;
            const size_t at = static_cast<size_t>(ok ? s0 + u : splits - 1) * stride;
            const float2 pair = *reinterpret_cast<const float2*>(ml + at * 2);
            ms[u] = ok ? pair.x : -INFINITY;
            ls[u] = pair.y;
            ps[u] = *reinterpret_cast<const float4_t*>(po + at * HD);
        }
        float m_new = m;
#pragma unroll
        for (int u = 0; u < 8; ++u) m_new = fmaxf(m_new, ms[u]);
        if (m_new == -INFINITY) continue;       // nothing seen yet
        const float keep = m == -INFINITY ? 0.f : exp2f((m - m_new) * scale_log2e);
        num *= keep;
        den *= keep;
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const float f = ms[u] == -INFINITY ? 0.f : exp2f((ms[u] - m_new) * scale_log2e);
#pragma unroll
            for (int v = 0; v < 4; ++v) num[v] = fmaf(ps[u][v], f, num[v]);
            den = fmaf(ls[u], f, den);
        }
        m = m_new;
    }
    const int row = row0 + r;
    const int tok = row / group, head = kvh * group + row % group;
    *reinterpret_cast<float4_t*>(out + (static_cast<size_t>(q_start + tok) * num_heads + head) * HD + d) =
        float4_t{num[0] / den, num[1] / den, num[2] / den, num[3] / den};
}

// Prompt portions: a workgroup takes 64 rows (a wavefront a tile of 16) and walks their keys in blocks of 32,
// which it stages once for all four wavefronts: the keys as rows of HD + 4 floats, the values transposed as rows of
// 32 + 4 (16 lanes' 16-byte fragment reads fall into different banks).  The products are those of the kernel above
// (lane group g takes the quarter g of the head in the scores, the keys 4g..4g+3 of a tile of 16 in the second
// product); the maximum and the sums are carried from block to block.  (The next block's pieces asked for into
// registers while this one is multiplied: 256 registers and spills, 216 to 231 us for 2,048 tokens where this form
// takes 205 to 217.)  Work items are the bfloat16 prompt kernel's
// (`attention_prefill.hip`): segment, key/value head, first row, first key, end key, partial slot (-1: final).
constexpr int kBlockKeys = 32;

template <int HD>
__global__ void __launch_bounds__(256, 2)
paged_attention_prefill_f32_kernel(const float* __restrict__ qkv, const float* __restrict__ cache,
                                   const int* __restrict__ block_tables, const int* __restrict__ items,
                                   const int* __restrict__ seg_q_start, const int* __restrict__ seg_q_len,
                                   const int* __restrict__ seg_ctx_len, float* __restrict__ out,
                                   float* __restrict__ partial_o, float* __restrict__ partial_ml, int num_heads,
                                   int num_kv_heads, int page_size, int max_pages, float scale_log2e, int window) {
    constexpr int DQ = HD / 4, DT = HD / 16;
    constexpr int SK = HD + 4, SV = kBlockKeys + 4;
    __shared__ __align__(16) float k_s[kBlockKeys * SK];
    __shared__ __align__(16) float v_s[HD * SV];

    const int* item = items + static_cast<size_t>(blockIdx.x) * kItemInts;
    const int seg = item[0], kvh = item[1], row_begin = item[2];
    const int key_begin = item[3], key_end = item[4], partial_slot = item[5];
    if (seg < 0) return;
    const int tid = threadIdx.x, lane = tid % kWave, wave = tid / kWave;
    const int i = lane % 16, g = lane / 16;
    const int group = num_heads / num_kv_heads;
    const int q_start = seg_q_start[seg], q_len = seg_q_len[seg], ctx = seg_ctx_len[seg];
    const int total_rows = q_len * group;
    const int first_pos = ctx - q_len;
    const int seg_lo = window > 0 ? max(0, first_pos - window + 1) : 0;
    const int width = (num_heads + 2 * num_kv_heads) * HD;
    const size_t page_elems = static_cast<size_t>(2) * num_kv_heads * page_size * HD;
    const size_t k_off = static_cast<size_t>(kvh) * page_size * HD;
    const size_t v_off = (static_cast<size_t>(num_kv_heads) + kvh) * page_size * HD;
    const int* table = block_tables + static_cast<size_t>(seg) * max_pages;

    const int wr0 = row_begin + wave * 16;
    const int row = wr0 + i;
    const bool row_valid = row < total_rows;
    const int tok = row_valid ? row / group : 0;
    const int head = kvh * group + (row_valid ? row % group : 0);
    const int pos = first_pos + tok;
    const int lo = window > 0 ? max(0, pos - window + 1) : 0;
    // a block that lies wholly inside every row's range needs no mask (a wavefront-wide decision)
    const int w_last_row = min(total_rows - 1, wr0 + 15);
    const bool wave_active = wr0 < total_rows;
    const int t_pos_min = (wave_active && w_last_row == wr0 + 15) ? first_pos + wr0 / group : -1;
    const int t_lo_max = window > 0 ? max(0, first_pos + max(w_last_row, 0) / group - window + 1) : 0;
    const int w_hi = wave_active ? first_pos + w_last_row / group + 1 : 0;                       // exclusive
    const int w_lo = window > 0 ? max(0, first_pos + wr0 / group - window + 1) : 0;
    const int b_last_row = min(total_rows - 1, row_begin + 63);
    const int b_hi = first_pos + b_last_row / group + 1;
    const int b_lo = window > 0 ? max(0, first_pos + row_begin / group - window + 1) : 0;
    const int blk_first = max(b_lo, key_begin) / kBlockKeys;
    const int blk_end = (min(b_hi, key_end) + kBlockKeys - 1) / kBlockKeys;

    // the lane's quarter of its row of queries
    float4_t qv[DQ / 4];
    {
        const float* qrow = qkv + static_cast<size_t>(q_start + tok) * width + static_cast<size_t>(head) * HD + g * DQ;
#pragma unroll
        for (int j = 0; j < DQ / 4; ++j)
            qv[j] = row_valid ? *reinterpret_cast<const float4_t*>(qrow + 4 * j) : float4_t{0.f, 0.f, 0.f, 0.f};
    }
    float4_t acc[DT];
#pragma unroll
    for (int t = 0; t < DT; ++t) acc[t] = float4_t{0.f, 0.f, 0.f, 0.f};
    float m_run = -INFINITY, l_run = 0.f;

    for (int blk = blk_first; blk < blk_end; ++blk) {
        const int kbase = blk * kBlockKeys;
        __syncthreads();        // everyone is done with the block before
        // ---- the block's keys, rows of the cache as they lie; a key beyond the table's width (it is masked) reads
        //      the last page the table names ----
#pragma unroll
        for (int u = 0; u < kBlockKeys * (HD / 4) / 256; ++u) {
            const int p = tid + 256 * u;
            const int key = p / (HD / 4), c4 = p % (HD / 4);
            const int kk = kbase + key;
            const int page_index = kk / page_size, slot = kk - page_index * page_size;
            const float* src = cache + static_cast<size_t>(table[min(page_index, max_pages - 1)]) * page_elems + k_off +
                               static_cast<size_t>(slot) * HD + 4 * c4;
            *reinterpret_cast<float4_t*>(k_s + key * SK + 4 * c4) = *reinterpret_cast<const float4_t*>(src);
        }
        // ---- its values, four keys of a transposed row a piece (one page: pages are multiples of 4 keys); what is
        //      not the request's (stale slots, pages given back) may hold anything and is cleared ----
        const bool edge = kbase < seg_lo || kbase + kBlockKeys > ctx;
#pragma unroll
        for (int u = 0; u < HD * (kBlockKeys / 4) / 256; ++u) {
            const int p = tid + 256 * u;
            const int d = p / (kBlockKeys / 4), q4 = p % (kBlockKeys / 4);
            const int kk = kbase + 4 * q4;
            const int page_index = kk / page_size, slot = kk - page_index * page_size;
            const float* src = cache + static_cast<size_t>(table[min(page_index, max_pages - 1)]) * page_elems + v_off +
                               static_cast<size_t>(d) * page_size + slot;
            float4_t v = *reinterpret_cast<const float4_t*>(src);
            if (edge) {
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    if (kk + e >= ctx || kk + e < seg_lo) v[e] = 0.f;
            }
            *reinterpret_cast<float4_t*>(v_s + d * SV + 4 * q4) = v;
        }
        __syncthreads();
        if (!wave_active || kbase >= w_hi || kbase + kBlockKeys <= w_lo) continue;
        // ---- scores: two tiles of 16 keys; the lane's keys are 16 t2 + 4 g + v ----
        float sv[8];
#pragma unroll
        for (int t2 = 0; t2 < 2; ++t2) {
            float4_t sc = float4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int j = 0; j < DQ / 4; ++j) {
                const float4_t kf = *reinterpret_cast<const float4_t*>(k_s + (16 * t2 + i) * SK + g * DQ + 4 * j);
#pragma unroll
                for (int e = 0; e < 4; ++e) sc = __builtin_amdgcn_mfma_f32_16x16x4f32(kf[e], qv[j][e], sc, 0, 0, 0);
            }
#pragma unroll
            for (int v = 0; v < 4; ++v) sv[4 * t2 + v] = sc[v];
        }
        const bool inside = kbase + kBlockKeys - 1 <= t_pos_min && kbase >= t_lo_max;
        if (!inside) {
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const int key = kbase + 16 * (e / 4) + 4 * g + e % 4;
                if (!(row_valid && key <= pos && key >= lo)) sv[e] = -INFINITY;
            }
        }
        float tile_max = fmaxf(fmaxf(fmaxf(sv[0], sv[1]), fmaxf(sv[2], sv[3])), fmaxf(fmaxf(sv[4], sv[5]), fmaxf(sv[6], sv[7])));
        tile_max = max_across(max_across(tile_max, 16), 32);
        const float m_new = fmaxf(m_run, tile_max);
        const float mc = (m_new == -INFINITY ? 0.f : m_new) * scale_log2e;
        const float alpha = exp2f(fmaf(m_run, scale_log2e, -mc));        // exp2(-inf) = 0: nothing was summed yet
        float pe[8], psum = 0.f;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            pe[e] = exp2f(fmaf(sv[e], scale_log2e, -mc));                   // 0 for masked keys
            psum += pe[e];
        }
        l_run = l_run * alpha + psum;
        m_run = m_new;
        if (__builtin_amdgcn_readfirstlane(__any(alpha != 1.f))) {
#pragma unroll
            for (int t = 0; t < DT; ++t) acc[t] *= alpha;
        }
        // ---- out^T += V^T . P^T ----
#pragma unroll
        for (int t = 0; t < DT; ++t) {
#pragma unroll
            for (int t2 = 0; t2 < 2; ++t2) {
                const float4_t vf = *reinterpret_cast<const float4_t*>(v_s + (16 * t + i) * SV + 16 * t2 + 4 * g);
#pragma unroll
                for (int v = 0; v < 4; ++v) acc[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(vf[v], pe[4 * t2 + v], acc[t], 0, 0, 0);
            }
        }
    }
    float l = sum_across(sum_across(l_run, 16), 32);
    if (!row_valid) return;
    if (partial_slot >= 0) {
        // one slot per tile of 16 rows: [16][HD] accumulators and [16][2] (maximum, sum)
        const size_t slot = static_cast<size_t>(partial_slot) + wave;
        float* po = partial_o + (slot * 16 + i) * HD;
#pragma unroll
        for (int t = 0; t < DT; ++t) *reinterpret_cast<float4_t*>(po + t * 16 + 4 * g) = acc[t];
        if (g == 0) *reinterpret_cast<float2*>(partial_ml + (slot * 16 + i) * 2) = make_float2(m_run, l);
        return;
    }
    const float inv = 1.f / l;
    float* orow = out + (static_cast<size_t>(q_start + tok) * num_heads + head) * HD;
#pragma unroll
    for (int t = 0; t < DT; ++t)
        *reinterpret_cast<float4_t*>(orow + t * 16 + 4 * g) = float4_t{acc[t][0] * inv, acc[t][1] * inv, acc[t][2] * inv, acc[t][3] * inv};
}

template <int HD>
int launch_f32(const float* qkv, const float* cache, const int* block_tables, const int* items, const int* live_items,
               int num_items, const int* reduce_items, int num_reduce_items, const int* seg_q_start, const int* seg_q_len,
               float* out, float* partial_o, float* partial_ml, int num_heads, int num_kv_heads, int page_size,
               int max_pages, float scale_log2e, int window, hipStream_t stream) {
    if (num_items > 0)
        paged_attention_f32_kernel<HD><<<num_items, 256, 0, stream>>>(qkv, cache, block_tables, items, live_items, out,
                                                                      partial_o, partial_ml, num_heads, num_kv_heads,
                                                                      page_size, max_pages, scale_log2e, window);
    if (num_reduce_items > 0)
        attention_reduce_f32_kernel<HD><<<dim3(num_reduce_items, kRowsPerTile / 4), HD, 0, stream>>>(
            reduce_items, partial_o, partial_ml, seg_q_start, seg_q_len, out, num_heads, num_kv_heads, scale_log2e);
    return launch_status();
}

}  // namespace

// Returns 0, a HIP error code, or -1 for sizes these kernels do not take.  `live_items`: null, or a
// device int that says how many of the `num_items` items count (a captured graph's plan).
WLLM_API int wllm_paged_attention_mfma_f32(const float* qkv, const float* cache, const int* block_tables, const int* items,
                                           const int* live_items, int num_items, const int* reduce_items,
                                           int num_reduce_items, const int* seg_q_start, const int* seg_q_len, float* out,
                                           float* partial_o, float* partial_ml, int num_heads, int num_kv_heads,
                                           int head_dim, int page_size, int max_pages, float scale, int window,
                                           hipStream_t stream) {
    if (head_dim % 32 != 0 || head_dim < 32 || head_dim > 256 || page_size % 4 != 0 || num_heads % num_kv_heads != 0 ||
        num_heads >= (1 << 16))       // an item holds a key/value head and a tile's first row in 16 bits each
        return -1;
    const float scale_log2e = scale * 1.4426950408889634f;
#define LAUNCH(HD)                                                                                                       \
    return launch_f32<HD>(qkv, cache, block_tables, items, live_items, num_items, reduce_items, num_reduce_items,         \
                          seg_q_start, seg_q_len, out, partial_o, partial_ml, num_heads, num_kv_heads, page_size, max_pages, \
                          scale_log2e, window, stream)
    switch (head_dim) {
        case 32: LAUNCH(32);
        case 64: LAUNCH(64);
        case 96: LAUNCH(96);
        case 128: LAUNCH(128);
        case 160: LAUNCH(160);
        case 192: LAUNCH(192);
        case 224: LAUNCH(224);
        case 256: LAUNCH(256);
        default: return -1;
    }
#undef LAUNCH
}

// The prompt portions of a float32 step: `items` are prefill items of 64 rows (`rows_per_item` says what the plan was
// made for).  Blocks whose keys were cut into pieces leave partial results for the reduce kernel, which
// `wllm_paged_attention_mfma_f32` runs with the step's reduce items.  Returns 0, a HIP error code, or -1.
WLLM_API int wllm_paged_attention_prefill_f32(const float* qkv, const float* cache, const int* block_tables, const int* items,
                                              int num_items, int rows_per_item, const int* seg_q_start, const int* seg_q_len,
                                              const int* seg_ctx_len, float* out, float* partial_o, float* partial_ml,
                                              int num_heads, int num_kv_heads, int head_dim, int page_size, int max_pages,
                                              float scale, int window, hipStream_t stream) {
    if (head_dim % 32 != 0 || head_dim < 32 || head_dim > 256 || page_size % 4 != 0 || num_heads % num_kv_heads != 0 ||
        rows_per_item != 64)
        return -1;
    if (num_items <= 0) return 0;
    const float scale_log2e = scale * 1.4426950408889634f;
#define LAUNCH(HD)                                                                                                    \
    paged_attention_prefill_f32_kernel<HD><<<num_items, 256, 0, stream>>>(qkv, cache, block_tables, items, seg_q_start, \
                                                                          seg_q_len, seg_ctx_len, out, partial_o,        \
                                                                          partial_ml, num_heads, num_kv_heads, page_size, \
                                                                          max_pages, scale_log2e, window);               \
    break
    switch (head_dim) {
        case 32: LAUNCH(32);
        case 64: LAUNCH(64);
        case 96: LAUNCH(96);
        case 128: LAUNCH(128);
        case 160: LAUNCH(160);
        case 192: LAUNCH(192);
        case 224: LAUNCH(224);
        case 256: LAUNCH(256);
        default: return -1;
    }
#undef LAUNCH
    return launch_status();
}

