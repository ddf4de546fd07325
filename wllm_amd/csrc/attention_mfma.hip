// Paged attention on the matrix cores for bfloat16, for segments of at most 16 query rows (decoded
// tokens, and portions short enough): head sizes 32..256 in steps of 32, pages of a multiple of 4
// tokens, any number of heads and groups, optional window.  Longer segments take the kernel of
// `attention_prefill.hip`, which shares the products' layout described here.
//
// Rows.  For one request (segment) and one key/value head, the query rows are the pairs (token,
// query head of the group): row r = token * G + head.  All rows of a tile read the same keys and
// values, so under multi-query attention the G heads of a token share one pass over the cache
// (the reference's kernel runs one workgroup per query head and reads the cache G times,
// src/wllm/kernels/csrc/paged_attention.cu:44-45,185).
//
// Work items.  The host cuts every (segment, key/value head) into work items, one workgroup of 4
// wavefronts each: a tile of 16 of the segment's rows (it has one, unless more than 16 query heads
// share a key/value head) and a chunk of keys that lies within one
// aligned group of 128 keys, cut to what the rows can need.  Each wavefront takes one of the
// chunk's four blocks of 32 keys; its loads of keys and values wait for the item and the block
// table only (the request's lengths and the queries are read while they are in flight), and the
// four are merged through shared memory.  A segment with more keys than a chunk is split over
// workgroups; those write partial results (maximum, sum, unnormalised accumulator) that
// `attention_reduce_kernel` combines.  Chunk boundaries depend on the key index only, never on
// the batch.  A captured graph launches a workgroup for every item its plan has room for and reads
// the number of live items, which come first, from device memory.
//
// Matrix products (v_mfma_f32_16x16x32_bf16, 64 lanes: i = lane % 16, g = lane / 16):
//   scores^T[key, row] = K[key, :] . Q[row, :]     A = K: lane (i, g) holds K[key_i][32c + 8g ..+8]
//                                                  B = Q: lane (i, g) holds Q[row_i][32c + 8g ..+8]
//                                                  C: lane (i, g) holds rows (keys) 4g..4g+3, column row_i
//   out^T[d, row] = V^T[d, keys] . P^T[keys, row]  A = V^T: lane (i, g) holds V^T[16t + i][8 keys of g]
//                                                  B = P^T: the lane's own 8 probabilities of row_i
// so every value a lane holds belongs to one query row, softmax needs two shuffles per tile, and the
// probabilities feed the second product from the registers they were computed in.  The cache holds
// keys as [page_size, head_dim] rows and values transposed as [head_dim, page_size] rows.  Values are
// loaded as fragments (16-byte loads when the page size is a multiple of 8: per instruction two runs
// of 512 bytes).  Keys are loaded as whole rows, 16 bytes a lane in the order they lie in the page,
// and become fragments in the wavefront's part of shared memory: a fragment load straight from the
// cache asks for 64-byte pieces of 16 rows, a pattern the memory system serves more slowly.
// Scores, maxima, sums and accumulators are float32.
#include "common.h"

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float float4_t __attribute__((ext_vector_type(4)));
typedef uint32_t uint4_t __attribute__((ext_vector_type(4)));     // 16 bytes as one value (no aggregate copy)

constexpr int kItemInts = 8;
constexpr int kRowsPerTile = 16;
constexpr int kKeysPerBlock = 32;

union Pack16 {
    uint4 u;
    bf16x8_t v;
    uint2 half[2];
    uint16_t s[8];
};

__device__ __forceinline__ uint16_t bf16_bits(float f) { return from_float<bf16>(f).bits; }

// Three workgroups a compute unit (168 registers a lane) where the kernel fits them without spilling;
// two for the head sizes and page sizes whose staging needs more.
template <int HD, bool V16>
__global__ void __launch_bounds__(256, (HD <= 160 || (HD == 256 && V16)) ? 3 : 2)
paged_attention_mfma_kernel(const bf16* __restrict__ qkv, const bf16* __restrict__ cache,
                            const int* __restrict__ block_tables, const int* __restrict__ items,
                            const int* __restrict__ live_items, const int* __restrict__ seg_q_start, const int* __restrict__ seg_q_len,
                            const int* __restrict__ seg_ctx_len, bf16* __restrict__ out,
                            float* __restrict__ partial_o, float* __restrict__ partial_ml, int num_heads,
                            int num_kv_heads, int page_size, int max_pages, float scale_log2e, int window) {
    constexpr int DC = HD / 32;   // 32-wide chunks of the head for the score product
    constexpr int DT = HD / 16;   // 16-row tiles of out^T
    // Shared memory, a part for each wavefront, used four times: three workgroups share a compute
    // unit's 160 KB.  The wavefront turns its block of keys, which it reads from the cache row by row
    // (whole key rows: contiguous runs the memory system streams much faster than the 64-byte pieces
    // a fragment load straight from the cache would ask for), into fragments, the 16 keys of the
    // first score tile and then the 16 of the second: [16 keys][HD + 8] bfloat16, rows padded so that
    // the fragment reads spread over the banks.  Then it leaves its sums there for the merge, one
    // half of the head after the other: [16 rows][HD / 2 + 4] floats.
    constexpr int kKeyStride = HD + 8;                                      // elements
    constexpr int kPartBytes = 16 * kKeyStride * 2;
    constexpr int kMergeStride = HD / 2 + 4;                                // floats
    static_assert(kRowsPerTile * kMergeStride * 4 <= kPartBytes, "half of the sums fits a wavefront's part");
    __shared__ __align__(16) unsigned char shared_raw[4 * kPartBytes];
    __shared__ float row_max_s[4][kRowsPerTile], row_sum_s[4][kRowsPerTile];

    // A captured graph launches as many workgroups as its plan has room for items; the live ones come
    // first.  The item is asked for together with their number, not after it (there is an item, live
    // or stale, for every workgroup of the launch), and brings the segment's lengths with it: one trip
    // to memory for all of them.
    const int* item = items + static_cast<size_t>(blockIdx.x) * kItemInts;
    const int seg = item[0], kvh = item[1] & 0xffff, q_len = item[2], q_start = item[3];
    const int key_begin = item[4], key_end = item[5], partial_slot = item[6], ctx = item[7];
    const int live = live_items != nullptr ? live_items[0] : 0x7fffffff;
    if (static_cast<int>(blockIdx.x) >= live) return;
    const int row_begin = (item[1] >> 16) * kRowsPerTile;      // the tile's first row: 0 unless a token has more than 16 heads a group
    if (seg < 0) return;    // padding item
    const int lane = threadIdx.x % kWave;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    const int i = lane % 16, g = lane / 16;

    // ---- This lane's queries are asked for first: they arrive while the addresses of the keys and
    //      values are worked out. ----
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
    // An item's keys lie within one aligned group of 128 (the host's chunk), so each of the four
    // wavefronts has at most one block of 32 keys and nothing is carried from block to block.
    const int blk_first = key_begin / kKeysPerBlock;
    const int blk_end = (key_end + kKeysPerBlock - 1) / kKeysPerBlock;
    const int blk = blk_first + wave;
    const bool has_block = blk < blk_end;
    bf16x8_t qreg[DC];
    if (has_block) {
        const bf16* qrow = qkv + static_cast<size_t>(q_start + tok) * width + static_cast<size_t>(head) * HD;
#pragma unroll
        for (int c = 0; c < DC; ++c) {
            Pack16 p;
            p.u = row_valid ? *reinterpret_cast<const uint4*>(qrow + c * 32 + 8 * g) : make_uint4(0, 0, 0, 0);
            qreg[c] = p.v;
        }
    }

    const size_t page_elems = static_cast<size_t>(2) * num_kv_heads * page_size * HD;
    const size_t k_off = static_cast<size_t>(kvh) * page_size * HD;
    const size_t v_off = (static_cast<size_t>(num_kv_heads) + kvh) * page_size * HD;
    const int* table = block_tables + static_cast<size_t>(seg) * max_pages;
    // a block's keys as the cache holds them: 32 rows of HD, 16 bytes a lane and load
    constexpr int kPieces = HD / 8;                 // 16-byte pieces of a key row
    uint4_t kraw[DT];                               // 32 * kPieces / 64 = HD / 16 loads a lane
    Pack16 va_[DT];
    const int kbase = blk * kKeysPerBlock;
    float4_t acc[DT];
    float m_run = -INFINITY, l_run = 0.f;
    uint16_t* stage = reinterpret_cast<uint16_t*>(shared_raw + wave * kPartBytes);
    if (has_block) {
        // All loads of the block are issued before the first product needs one, so a block costs
        // one trip to memory after the block table's.  Keys beyond the request are masked later;
        // their table entry is clamped to the table's width (entries beyond a request's pages name
        // a valid page), not to the length.  A key's page and slot come from its place within the
        // block and one division a wavefront: the quotient by the page size as a float product,
        // exact for the few hundred values it is asked for here.
        const int base_page = kbase / page_size, base_slot = kbase % page_size;     // the same for all lanes
        const float inv_page = 1.f / static_cast<float>(page_size);
        auto place = [&](int within, int& page_index, int& slot) {
            const int x = base_slot + within;                                  // < page_size + 32
            const int q = static_cast<int>((static_cast<float>(x) + 0.5f) * inv_page);
            page_index = min(base_page + q, max_pages - 1);
            slot = x - q * page_size;
        };
        const bf16* kpiece[DT];
#pragma unroll
        for (int j = 0; j < DT; ++j) {
            // piece f of the block: key f / kPieces, its 8 elements f % kPieces; a wavefront's load
            // covers whole consecutive rows
            const int f = j * kWave + lane;
            int page_index, slot;
            place(f / kPieces, page_index, slot);
            kpiece[j] = cache + static_cast<size_t>(table[page_index]) * page_elems + k_off +
                        static_cast<size_t>(slot) * HD + (f % kPieces) * 8;
        }
        int vpage0, vslot0, vpage1 = 0, vslot1 = 0;
        place(V16 ? 8 * g : 4 * g, vpage0, vslot0);
        if (!V16) place(16 + 4 * g, vpage1, vslot1);
        const bf16* vbase0 = cache + static_cast<size_t>(table[vpage0]) * page_elems + v_off + vslot0;
        const bf16* vbase1 = cache + static_cast<size_t>(V16 ? 0 : table[vpage1]) * page_elems + v_off + vslot1;
#pragma unroll
        for (int j = 0; j < DT; ++j) kraw[j] = __builtin_nontemporal_load(reinterpret_cast<const uint4_t*>(kpiece[j]));
#pragma unroll
        for (int t = 0; t < DT; ++t) {
            const size_t drow = static_cast<size_t>(t * 16 + i) * page_size;
            if (V16) {
                va_[t].u = load_streamed(vbase0 + drow);
            } else {
                va_[t].half[0] = load_streamed8(vbase0 + drow);
                va_[t].half[1] = load_streamed8(vbase1 + drow);
            }
        }
        const bool edge = kbase < seg_lo || kbase + kKeysPerBlock > ctx;
        // ---- the keys through this wavefront's part of shared memory, then the scores: one tile
        //      of 16 keys after the other.  Which keys row i of a tile's first operand is: see the
        //      header for why. ----
        float4_t s[2];
#pragma unroll
        for (int t2 = 0; t2 < 2; ++t2) {
#pragma unroll
            for (int j = 0; j < DT; ++j) {
                const int f = lane + j * kWave;
                const int key = f / kPieces;
                const int tile = V16 ? (key / 4) % 2 : key / 16;
                const int at = V16 ? 4 * (key / 8) + key % 4 : key % 16;
                if (tile == t2)
                    *reinterpret_cast<uint4_t*>(stage + at * kKeyStride + (f % kPieces) * 8) = kraw[j];
            }
            // Lanes read what other lanes of the wavefront wrote, with no barrier between (a
            // wavefront's accesses to shared memory run in order): the compiler has to be told
            // that the memory changed, or a lane that wrote nothing keeps what it read before.
            asm volatile("" ::: "memory");
            float4_t sc = float4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int c = 0; c < DC; ++c) {
                Pack16 a;
                a.u = *reinterpret_cast<const uint4*>(stage + i * kKeyStride + c * 32 + 8 * g);
                sc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a.v, qreg[c], sc, 0, 0, 0);
            }
            s[t2] = sc;
        }
        // ---- mask, maximum, probabilities ----
        float sv[8];
        bool ok[8];
        float tile_max = -INFINITY;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const int t2 = e / 4, v = e % 4;
            const int key = kbase + (V16 ? 8 * g + 4 * t2 + v : 16 * t2 + 4 * g + v);
            ok[e] = row_valid && key <= pos && key >= lo && key >= key_begin && key < key_end;
            sv[e] = s[t2][v];
            if (ok[e]) tile_max = fmaxf(tile_max, sv[e]);
        }
        tile_max = max_across(max_across(tile_max, 16), 32);
        m_run = tile_max;
        const float mc = (tile_max == -INFINITY ? 0.f : tile_max) * scale_log2e;
        Pack16 pv;
        float pe[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            pe[e] = ok[e] ? exp2_probability(fmaf(sv[e], scale_log2e, -mc)) : 0.f;
            l_run += pe[e];
        }
        pv.u = make_uint4(pack2_bf16(pe[0], pe[1]), pack2_bf16(pe[2], pe[3]), pack2_bf16(pe[4], pe[5]),
                          pack2_bf16(pe[6], pe[7]));
        // the row's sum over its four lanes
        l_run = sum_across(sum_across(l_run, 16), 32);
        // ---- out^T = V^T . P^T ----
#pragma unroll
        for (int t = 0; t < DT; ++t) {
            Pack16 a = va_[t];
            if (edge) {
                // keys outside the request (stale slots, pages given back) may hold anything,
                // NaN included; 0 * NaN would poison the sum, so they are cleared
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    const int key = kbase + (V16 ? 8 * g + e : (e < 4 ? 4 * g + e : 16 + 4 * g + e - 4));
                    if (key >= ctx || key < seg_lo) a.s[e] = 0;
                }
            }
            acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a.v, pv.v, float4_t{0.f, 0.f, 0.f, 0.f}, 0, 0, 0);
        }
    } else {
#pragma unroll
        for (int t = 0; t < DT; ++t) acc[t] = float4_t{0.f, 0.f, 0.f, 0.f};
    }

    // ---- merge: every wavefront leaves its sums in its own part of shared memory (it has read its
    //      keys from there already), one half of the head after the other; of each half every
    //      wavefront takes every fourth tile of 16 elements and combines the four wavefronts' sums of
    //      that tile, always in the order 0, 1, 2, 3.
    //      lane (i, g) holds out^T[16t + 4g + v][row i]: elements d = 16t + 4g + v of row i ----
    float* mine = reinterpret_cast<float*>(stage);
    if (g == 0) {
        row_max_s[wave][i] = m_run;
        row_sum_s[wave][i] = l_run;
    }
    float f_of[4] = {0.f, 0.f, 0.f, 0.f};
    float m_all = -INFINITY, l_all = 0.f, inv = 0.f;
    bf16* orow = out + (static_cast<size_t>(q_start + tok) * num_heads + head) * HD;
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
                        const float* part = reinterpret_cast<const float*>(shared_raw + w * kPartBytes);
                        const float4_t v = *reinterpret_cast<const float4_t*>(part + i * kMergeStride + t * 16 + 4 * g);
#pragma unroll
                        for (int e = 0; e < 4; ++e) sum[e] = fmaf(v[e], f_of[w], sum[e]);
                    }
                    const int d = (half * (DT / 2) + t) * 16 + 4 * g;
                    if (partial_slot < 0) {
                        uint2 w2;
                        w2.x = pack2_bf16(sum[0] * inv, sum[1] * inv);
                        w2.y = pack2_bf16(sum[2] * inv, sum[3] * inv);
                        *reinterpret_cast<uint2*>(orow + d) = w2;
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

// Combines the partial results of a (segment, key/value head) whose keys were split over workgroups.
// reduce items: seg, kvh, first partial slot, number of splits, first row, slots between splits, 2 unused.
template <int HD>
__global__ void __launch_bounds__(HD)
attention_reduce_kernel(const int* __restrict__ reduce_items, const float* __restrict__ partial_o,
                        const float* __restrict__ partial_ml, const int* __restrict__ seg_q_start,
                        const int* __restrict__ seg_q_len, bf16* __restrict__ out, int num_heads, int num_kv_heads,
                        float scale_log2e) {
    // one workgroup per (item, row); one thread per element of the head; the loads of the
    // splits do not depend on each other.  Reduce items are 8 int32: segment, key/value head, first
    // slot, number of splits, first row of the tile within the segment, slots between two splits.
    const int* item = reduce_items + static_cast<size_t>(blockIdx.x) * kItemInts;
    const int seg = item[0], kvh = item[1], first = item[2], splits = item[3], row0 = item[4];
    if (seg < 0) return;
    const size_t stride = static_cast<size_t>(item[5]) * kRowsPerTile;     // rows between two splits
    const int group = num_heads / num_kv_heads;
    const int r = blockIdx.y, d = threadIdx.x;
    const int q_start = seg_q_start[seg];       // asked for with the length: the store at the end does not wait for it
    if (row0 + r >= seg_q_len[seg] * group) return;
    const float* ml = partial_ml + (static_cast<size_t>(first) * kRowsPerTile + r) * 2;
    const float* po = partial_o + (static_cast<size_t>(first) * kRowsPerTile + r) * HD + d;
    // One pass in groups of eight splits: all loads of a group are issued together, and the sums are
    // rescaled when a group raises the maximum, so the kernel makes one trip to memory per group.
    float m = -INFINITY, num = 0.f, den = 0.f;
    for (int s0 = 0; s0 < splits; s0 += 8) {
        float ms[8], ls[8], ps[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            // a split beyond the last reads the last one again (the same addresses) and does not count
            const bool ok = s0 + u < splits;
            const size_t at = static_cast<size_t>(ok ? s0 + u : splits - 1) * stride;
            const float m_at = ml[at * 2];
            ms[u] = ok ? m_at : -INFINITY;
            ls[u] = ml[at * 2 + 1];
            ps[u] = po[at * HD];
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
            num = fmaf(ps[u], f, num);
            den = fmaf(ls[u], f, den);
        }
        m = m_new;
    }
    const int row = row0 + r;
    const int tok = row / group, head = kvh * group + row % group;
    out[(static_cast<size_t>(q_start + tok) * num_heads + head) * HD + d] = from_float<bf16>(num / den);
}

// The same sums for steps with many tiles to combine (the pieces of a long prompt): a thread takes
// four consecutive elements of a row (16-byte loads), a workgroup of HD threads four rows.  Every
// element goes through the operations of the kernel above in the same order, so which of the two
// runs changes no bit of the result.
template <int HD>
__global__ void __launch_bounds__(HD)
attention_reduce_wide_kernel(const int* __restrict__ reduce_items, const float* __restrict__ partial_o,
                             const float* __restrict__ partial_ml, const int* __restrict__ seg_q_start,
                             const int* __restrict__ seg_q_len, bf16* __restrict__ out, int num_heads,
                             int num_kv_heads, float scale_log2e) {
    const int* item = reduce_items + static_cast<size_t>(blockIdx.x) * kItemInts;
    const int seg = item[0], kvh = item[1], first = item[2], splits = item[3], row0 = item[4];
    if (seg < 0) return;
    const size_t stride = static_cast<size_t>(item[5]) * kRowsPerTile;     // rows between two splits
    const int group = num_heads / num_kv_heads;
    constexpr int kQuads = HD / 4;
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
    uint2 w;
    w.x = pack2_bf16(num[0] / den, num[1] / den);
    w.y = pack2_bf16(num[2] / den, num[3] / den);
    *reinterpret_cast<uint2*>(out + (static_cast<size_t>(q_start + tok) * num_heads + head) * HD + d) = w;
}

namespace {

struct AttentionArguments {
    const bf16* qkv;
    const bf16* cache;
    const int* block_tables;
    const int* items;
    const int* live_items;
    int num_items;
    const int* reduce_items;
    int num_reduce_items;
    const int* seg_q_start;
    const int* seg_q_len;
    const int* seg_ctx_len;
    bf16* out;
    float* partial_o;
    float* partial_ml;
    int num_heads, num_kv_heads, page_size, max_pages;
    float scale_log2e;
    int window;
    hipStream_t stream;
};

template <int HD, bool V16>
int launch_items(const AttentionArguments& a) {
    paged_attention_mfma_kernel<HD, V16><<<a.num_items, 256, 0, a.stream>>>(
        a.qkv, a.cache, a.block_tables, a.items, a.live_items, a.seg_q_start, a.seg_q_len, a.seg_ctx_len, a.out,
        a.partial_o, a.partial_ml, a.num_heads, a.num_kv_heads, a.page_size, a.max_pages, a.scale_log2e, a.window);
    return 0;
}

template <int HD>
int launch_all(const AttentionArguments& a) {
    if (a.num_items > 0) {
        const int status = a.page_size % 8 == 0 ? launch_items<HD, true>(a) : launch_items<HD, false>(a);
        if (status != 0) return status;
    }
    if (a.num_reduce_items >= 64) {
        attention_reduce_wide_kernel<HD><<<dim3(a.num_reduce_items, kRowsPerTile / 4), HD, 0, a.stream>>>(
            a.reduce_items, a.partial_o, a.partial_ml, a.seg_q_start, a.seg_q_len, a.out, a.num_heads, a.num_kv_heads,
            a.scale_log2e);
    } else if (a.num_reduce_items > 0) {
        attention_reduce_kernel<HD><<<dim3(a.num_reduce_items, kRowsPerTile), HD, 0, a.stream>>>(
            a.reduce_items, a.partial_o, a.partial_ml, a.seg_q_start, a.seg_q_len, a.out, a.num_heads, a.num_kv_heads,
            a.scale_log2e);
    }
    return launch_status();
}

}  // namespace

// Returns 0, a HIP error code, or -1 for sizes these kernels do not take.  `live_items`: null, or a
// device int that says how many of the `num_items` items count (a captured graph's plan).
WLLM_API int wllm_paged_attention_mfma(const void* qkv, const void* cache, const int* block_tables, const int* items,
                                       const int* live_items, int num_items, const int* reduce_items,
                                       int num_reduce_items, const int* seg_q_start, const int* seg_q_len,
                                       const int* seg_ctx_len, void* out, float* partial_o, float* partial_ml,
                                       int num_heads, int num_kv_heads, int head_dim, int page_size, int max_pages,
                                       float scale, int window, hipStream_t stream) {
    if (head_dim % 32 != 0 || head_dim < 32 || head_dim > 256 || page_size % 4 != 0 || num_heads % num_kv_heads != 0 ||
        num_heads >= (1 << 16))       // an item holds a key/value head and a tile's first row in 16 bits each
        return -1;
    const AttentionArguments a = {static_cast<const bf16*>(qkv), static_cast<const bf16*>(cache), block_tables, items,
                                  live_items, num_items, reduce_items, num_reduce_items, seg_q_start, seg_q_len,
                                  seg_ctx_len, static_cast<bf16*>(out), partial_o, partial_ml, num_heads, num_kv_heads,
                                  page_size, max_pages, scale * 1.4426950408889634f, window, stream};
    switch (head_dim) {
        case 32: return launch_all<32>(a);
        case 64: return launch_all<64>(a);
        case 96: return launch_all<96>(a);
        case 128: return launch_all<128>(a);
        case 160: return launch_all<160>(a);
        case 192: return launch_all<192>(a);
        case 224: return launch_all<224>(a);
        case 256: return launch_all<256>(a);
        default: return -1;
    }
}
