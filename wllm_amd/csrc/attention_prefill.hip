// Paged attention for long segments (prompt portions) on the matrix cores, bfloat16: the keys
// and values of a block of 32 keys are staged through shared memory once per workgroup and read
// by all four wavefronts; a wavefront owns one tile of 16 query rows.  A workgroup is 64 rows of one
// (segment, key/value head): rows are (token, query head of the group) pairs, row r = token * G +
// head.  (With two tiles a wavefront, every fragment read from shared memory would feed two
// products, but the registers of 128 rows leave room for one workgroup a compute unit; with 64
// rows two workgroups share it and hide each other's waits, which measured a quarter faster.)
//
// The products are those of `attention_mfma.hip` (v_mfma_f32_16x16x32_bf16, scores transposed so
// that a lane's values all belong to one query row, probabilities fed to the second product from
// the registers they were computed in).  Staging: while the products of block b run from shared
// memory, the global loads of block b+1 are in flight into registers; they are written to shared
// memory after a barrier.  Keys land as [32][HD] rows (padded), values as [HD][32] rows whose 32
// keys are permuted so that the 8 keys a lane needs are contiguous.  Keys outside the request
// (stale slots of the last page, pages a window gave back) are cleared while staging, so that a
// NaN there cannot meet a zero probability.
#include "common.h"

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float float4_t __attribute__((ext_vector_type(4)));

constexpr int kPrefillWaves = 4;       // wavefronts per workgroup
constexpr int kPrefillThreads = kPrefillWaves * 64;
constexpr int kBlockKeys = 32;
constexpr int kMaxTablePages = 1024;     // pages one work item's keys may span (the host cuts items to fit)
constexpr int kPrefillItemInts = 8;

union PPack {
    uint4 u;
    bf16x8_t v;
    uint2 half[2];
    uint16_t s[8];
};

template <int HD>
struct PrefillSmem {
    static constexpr int kStrideK = HD + 8;            // elements; the pad spreads rows over banks
    static constexpr int kStrideV = kBlockKeys + 8;
    static constexpr int kBytes = (kBlockKeys * kStrideK + HD * kStrideV) * 2;
};

// prefill items: seg, kvh, first row, first key, end key, partial slot (-1: the workgroup walks all
// the keys of its rows and writes the result itself), 2 unused.  Items that split the keys of a
// block of rows write, per tile of 16 rows, an unnormalised accumulator and (maximum, sum) into
// slot `partial slot + tile`, which `attention_reduce_kernel` combines.
template <int HD, int RTW>      // RTW: tiles of 16 rows per wavefront (1 or 2)
__global__ void __launch_bounds__(kPrefillThreads, RTW == 1 ? 2 : 1)
paged_attention_prefill_kernel(const bf16* __restrict__ qkv, const bf16* __restrict__ cache,
                               const int* __restrict__ block_tables, const int* __restrict__ items,
                               const int* __restrict__ seg_q_start, const int* __restrict__ seg_q_len,
                               const int* __restrict__ seg_ctx_len, bf16* __restrict__ out,
                               float* __restrict__ partial_o, float* __restrict__ partial_ml, int num_heads,
                               int num_kv_heads, int page_size, int max_pages, float scale_log2e, int window) {
    constexpr int DC = HD / 32, DT = HD / 16;
    constexpr int SK = PrefillSmem<HD>::kStrideK, SV = PrefillSmem<HD>::kStrideV;
    __shared__ __align__(16) uint16_t k_s[kBlockKeys * SK];
    __shared__ __align__(16) uint16_t v_s[HD * SV];
    __shared__ int table_s[kMaxTablePages];     // the pages of this item's keys: lookups never leave the CU

    const int* item = items + static_cast<size_t>(blockIdx.x) * kPrefillItemInts;
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

    // this wavefront's two tiles of rows
    constexpr int kWaveRows = 16 * RTW, kPrefillRows = kPrefillWaves * kWaveRows;
    const int wr0 = row_begin + wave * kWaveRows;
    int row[RTW], tok[RTW], head[RTW], pos[RTW], lo[RTW];
    bool row_valid[RTW];
    bf16x8_t qreg[RTW][DC];
#pragma unroll
    for (int rt = 0; rt < RTW; ++rt) {
        row[rt] = wr0 + rt * 16 + i;
        row_valid[rt] = row[rt] < total_rows;
        tok[rt] = row_valid[rt] ? row[rt] / group : 0;
        head[rt] = kvh * group + (row_valid[rt] ? row[rt] % group : 0);
        pos[rt] = first_pos + tok[rt];
        lo[rt] = window > 0 ? max(0, pos[rt] - window + 1) : 0;
        const bf16* qrow = qkv + static_cast<size_t>(q_start + tok[rt]) * width + static_cast<size_t>(head[rt]) * HD;
#pragma unroll
        for (int c = 0; c < DC; ++c) {
            PPack p;
            p.u = row_valid[rt] ? *reinterpret_cast<const uint4*>(qrow + c * 32 + 8 * g) : make_uint4(0, 0, 0, 0);
            qreg[rt][c] = p.v;
        }
    }
    // per row tile: the lowest position and the highest window start of its rows (wavefront-wide)
    int t_pos_min[RTW], t_lo_max[RTW];
#pragma unroll
    for (int rt = 0; rt < RTW; ++rt) {
        const int first = wr0 + rt * 16, last = min(total_rows - 1, first + 15);
        t_pos_min[rt] = first < total_rows ? first_pos + first / group : -1;
        const int pmax = first_pos + max(last, 0) / group;
        t_lo_max[rt] = window > 0 ? max(0, pmax - window + 1) : 0;
        if (last < first + 15) t_pos_min[rt] = -1;      // a tile with rows beyond the segment always masks
    }
    // keys the wavefront's rows can need
    const bool wave_active = wr0 < total_rows;
    const int w_last_row = min(total_rows - 1, wr0 + kWaveRows - 1);
    const int w_hi = wave_active ? first_pos + w_last_row / group + 1 : 0;                       // exclusive
    const int w_lo = window > 0 ? max(0, first_pos + wr0 / group - window + 1) : 0;
    // keys the workgroup stages: from the first wavefront's lowest to the last row's highest
    const int b_last_row = min(total_rows - 1, row_begin + kPrefillRows - 1);
    const int b_hi = first_pos + b_last_row / group + 1;
    const int b_lo = window > 0 ? max(0, first_pos + row_begin / group - window + 1) : 0;
    const int blk_first = max(b_lo, key_begin) / kBlockKeys;
    const int blk_end = (min(b_hi, key_end) + kBlockKeys - 1) / kBlockKeys;
    // the pages of keys blk_first * 32 .. blk_end * 32 (clamped to the request's keys)
    const int page_base = blk_first * kBlockKeys / page_size;
    if (blk_first < blk_end) {
        const int* table_g = block_tables + static_cast<size_t>(seg) * max_pages + page_base;
        const int page_last = (min(blk_end * kBlockKeys, ctx) - 1) / page_size;
        const int count = min(min(max_pages - 1, page_last) - page_base + 1, kMaxTablePages);
        for (int p = tid; p < count; p += kPrefillThreads) table_s[p] = table_g[p];
    }

    float4_t acc[RTW][DT];
    float m_run[RTW], l_run[RTW];
#pragma unroll
    for (int rt = 0; rt < RTW; ++rt) {
        m_run[rt] = -INFINITY;
        l_run[rt] = 0.f;
#pragma unroll
        for (int t = 0; t < DT; ++t) acc[rt][t] = float4_t{0.f, 0.f, 0.f, 0.f};
    }

    // ---- staging.  Keys: kTPK threads share a key row and take its 16-byte chunks in turn, so a
    //      thread looks up one page per block.  Values: a thread keeps one group of 4 keys (j) and
    //      walks the rows d of the transposed page, again one page lookup per block. ----
    constexpr int kTPK = kPrefillThreads / kBlockKeys;              // threads per key row
    constexpr int KCH = (HD / 8 + kTPK - 1) / kTPK;
    constexpr int kRowsPerPass = kPrefillThreads / 8;               // value rows staged per pass
    constexpr int VCH = (HD + kRowsPerPass - 1) / kRowsPerPass;
    const int k_key = tid / kTPK, k_lane = tid % kTPK;
    const int v_j = tid % 8, v_d0 = tid / 8;
    uint4 kreg_a[KCH];
    uint2 vreg_a[VCH];
    const int page_shift = (page_size & (page_size - 1)) == 0 ? __builtin_ctz(page_size) : -1;
    auto page_of = [&](int key, int& slot) -> int {
        if (page_shift >= 0) {
            slot = key & (page_size - 1);
            return table_s[(key >> page_shift) - page_base];
        }
        slot = key % page_size;
        return table_s[key / page_size - page_base];
    };
    auto fetch = [&](uint4* kreg, uint2* vreg, int kbase) {
        {
            const int key = kbase + k_key;
            const bool ok = key < ctx && key >= seg_lo;
            const int kk = min(key, ctx - 1);
            int slot;
            const int page = page_of(kk, slot);
            const bf16* src = cache + static_cast<size_t>(page) * page_elems + k_off + static_cast<size_t>(slot) * HD;
#pragma unroll
            for (int u = 0; u < KCH; ++u) {
                const int chunk = k_lane + u * kTPK;
                kreg[u] = (ok && chunk < HD / 8) ? *reinterpret_cast<const uint4*>(src + chunk * 8)
                                                 : make_uint4(0, 0, 0, 0);
            }
        }
        {
            const int key = kbase + 4 * v_j;                 // group v_j: keys key .. key + 3
            const int kk = min(key, ctx - 1) & ~3;
            int slot;
            const int page = page_of(kk, slot);
            const bf16* src = cache + static_cast<size_t>(page) * page_elems + v_off + slot;
            // keys of the group that are not the request's are cleared
            uint2 keep = make_uint2(0xffffffffu, 0xffffffffu);
            if (key + 3 >= ctx || key < seg_lo) {
                const bool k0 = key < ctx && key >= seg_lo, k1 = key + 1 < ctx && key + 1 >= seg_lo;
                const bool k2 = key + 2 < ctx && key + 2 >= seg_lo, k3 = key + 3 < ctx && key + 3 >= seg_lo;
                keep.x = (k0 ? 0x0000ffffu : 0u) | (k1 ? 0xffff0000u : 0u);
                keep.y = (k2 ? 0x0000ffffu : 0u) | (k3 ? 0xffff0000u : 0u);
            }
#pragma unroll
            for (int u = 0; u < VCH; ++u) {
                const int d = min(v_d0 + u * kRowsPerPass, HD - 1);
                uint2 v = *reinterpret_cast<const uint2*>(src + static_cast<size_t>(d) * page_size);
                v.x &= keep.x;
                v.y &= keep.y;
                vreg[u] = v;
            }
        }
    };
    auto stage = [&](const uint4* kreg, const uint2* vreg) {
#pragma unroll
        for (int u = 0; u < KCH; ++u) {
            const int chunk = k_lane + u * kTPK;
            if (chunk < HD / 8) *reinterpret_cast<uint4*>(&k_s[k_key * SK + chunk * 8]) = kreg[u];
        }
#pragma unroll
        for (int u = 0; u < VCH; ++u) {
            const int d = v_d0 + u * kRowsPerPass;
            // keys 4j..4j+3 go to positions 8*(j%4) + 4*(j/4): a lane's keys {4g..4g+3, 16+4g..} become contiguous
            if (d < HD) *reinterpret_cast<uint2*>(&v_s[d * SV + 8 * (v_j % 4) + 4 * (v_j / 4)]) = vreg[u];
        }
    };

    __syncthreads();      // the block table is in shared memory
    // the loads of the next block are in flight while the products of this one run
    if (blk_first < blk_end) fetch(kreg_a, vreg_a, blk_first * kBlockKeys);
    for (int blk = blk_first; blk < blk_end; ++blk) {
        const int kbase = blk * kBlockKeys;
        __syncthreads();                 // everyone is done with the previous block's tiles
        stage(kreg_a, vreg_a);
        __syncthreads();
        if (blk + 1 < blk_end) fetch(kreg_a, vreg_a, kbase + kBlockKeys);
        if (!wave_active || kbase >= w_hi || kbase + kBlockKeys <= w_lo) continue;
        // ---- scores: tile t2 holds keys kbase + 16*t2 + (0..15); lane (i, g) gets keys 16*t2 + 4g + v ----
        float4_t s[RTW][2];
#pragma unroll
        for (int t2 = 0; t2 < 2; ++t2) {
            float4_t sc[RTW];
#pragma unroll
            for (int rt = 0; rt < RTW; ++rt) sc[rt] = float4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int c = 0; c < DC; ++c) {
                PPack a;
                a.u = *reinterpret_cast<const uint4*>(&k_s[(16 * t2 + i) * SK + c * 32 + 8 * g]);
#pragma unroll
                for (int rt = 0; rt < RTW; ++rt)
                    sc[rt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a.v, qreg[rt][c], sc[rt], 0, 0, 0);
            }
#pragma unroll
            for (int rt = 0; rt < RTW; ++rt) s[rt][t2] = sc[rt];
        }
        // ---- softmax bookkeeping per row tile ----
        PPack pv[RTW];
        float alpha[RTW];
        bool rescale[RTW];
#pragma unroll
        for (int rt = 0; rt < RTW; ++rt) {
            float sv[8];
#pragma unroll
            for (int e = 0; e < 8; ++e) sv[e] = s[rt][e / 4][e % 4];
            // blocks that lie wholly inside every row's range need no mask (a wavefront-wide decision)
            const bool inside = kbase + kBlockKeys - 1 <= t_pos_min[rt] && kbase >= t_lo_max[rt];
            if (!inside) {
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    const int key = kbase + 16 * (e / 4) + 4 * g + (e % 4);
                    if (!(row_valid[rt] && key <= pos[rt] && key >= lo[rt])) sv[e] = -INFINITY;
                }
            }
            float tile_max = fmaxf(fmaxf(fmaxf(sv[0], sv[1]), fmaxf(sv[2], sv[3])),
                                   fmaxf(fmaxf(sv[4], sv[5]), fmaxf(sv[6], sv[7])));
            tile_max = max_across(max_across(tile_max, 16), 32);
            const float m_new = fmaxf(m_run[rt], tile_max);
            const float m_use = m_new == -INFINITY ? 0.f : m_new;
            const float mc = m_use * scale_log2e;
            alpha[rt] = exp2_probability(fmaf(m_run[rt], scale_log2e, -mc));
            float pe[8], psum = 0.f;
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                pe[e] = exp2_probability(fmaf(sv[e], scale_log2e, -mc));       // exp2(-inf) = 0 for masked keys
                psum += pe[e];
            }
            pv[rt].u = make_uint4(pack2_bf16(pe[0], pe[1]), pack2_bf16(pe[2], pe[3]), pack2_bf16(pe[4], pe[5]),
                                  pack2_bf16(pe[6], pe[7]));
            l_run[rt] = l_run[rt] * alpha[rt] + psum;
            m_run[rt] = m_new;
            rescale[rt] = __any(alpha[rt] != 1.f);
        }
        // ---- out^T += V^T . P^T; the accumulators are rescaled only when some row's maximum moved ----
#pragma unroll
        for (int rt = 0; rt < RTW; ++rt) {
            if (__builtin_amdgcn_readfirstlane(rescale[rt])) {      // one branch for the wavefront, not a select per number
#pragma unroll
                for (int t = 0; t < DT; ++t) acc[rt][t] *= alpha[rt];
            }
        }
#pragma unroll
        for (int t = 0; t < DT; ++t) {
            PPack a;
            a.u = *reinterpret_cast<const uint4*>(&v_s[(16 * t + i) * SV + 8 * g]);
#pragma unroll
            for (int rt = 0; rt < RTW; ++rt)
                acc[rt][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a.v, pv[rt].v, acc[rt][t], 0, 0, 0);
        }
    }
#pragma unroll
    for (int rt = 0; rt < RTW; ++rt) {
        float l = l_run[rt];
        l = sum_across(sum_across(l, 16), 32);
        if (!row_valid[rt]) continue;
        if (partial_slot >= 0) {
            // one slot per tile of 16 rows: [16][HD] accumulators and [16][2] (maximum, sum)
            const size_t slot = static_cast<size_t>(partial_slot) + wave * RTW + rt;
            float* po = partial_o + (slot * 16 + i) * HD;
#pragma unroll
            for (int t = 0; t < DT; ++t)
                *reinterpret_cast<float4*>(po + t * 16 + 4 * g) =
                    make_float4(acc[rt][t][0], acc[rt][t][1], acc[rt][t][2], acc[rt][t][3]);
            if (g == 0) *reinterpret_cast<float2*>(partial_ml + (slot * 16 + i) * 2) = make_float2(m_run[rt], l);
            continue;
        }
        const float inv = 1.f / l;
        bf16* orow = out + (static_cast<size_t>(q_start + tok[rt]) * num_heads + head[rt]) * HD;
#pragma unroll
        for (int t = 0; t < DT; ++t) {
            uint2 w;
            w.x = pack2_bf16(acc[rt][t][0] * inv, acc[rt][t][1] * inv);
            w.y = pack2_bf16(acc[rt][t][2] * inv, acc[rt][t][3] * inv);
            *reinterpret_cast<uint2*>(orow + t * 16 + 4 * g) = w;
        }
    }
}

// ---- the same kernel with the tiles moved into shared memory by the memory pipeline itself -------
// For head sizes 64, 128 and 256 and pages of 8, 16, 32, ... keys (a power of two, so that a key's
// place is a shift and a mask and most of a load's address is fixed for a lane: with divisions and a
// table look-up per load the address arithmetic was a third of the kernel's time; other page sizes
// take the kernel above).  A lane's 16-byte load goes
// straight to shared memory (lane l of a wavefront to base + 16 l), so staging costs no registers,
// no writes to shared memory and no second barrier; two tiles of keys and values are held, and
// the loads of block b+1 run while block b is multiplied.  Since a lane chooses its address, the
// 16-byte chunks of a tile are placed so that fragment reads are free of bank conflicts: the 16
// lanes that read together (one chunk each of 16 rows) have to hit 16 different chunks of the 256
// bytes that the banks span.  Chunk c of key row r lies at position c ^ (r % 16) of the row (heads
// of 64, whose rows are 8 chunks and lie two to the 256 bytes: c ^ ((r / 2) % 8)), chunk q (8 keys)
// of value row d at q ^ ((d / 2) % 4).  Measured with a loop of such reads alone, eight wavefronts a
// compute unit: 4.0 clocks a read (256 bytes a clock), and 6.4 with c ^ (r % 8), where rows r and
// r + 8 meet in the same banks.  The keys of a block are staged in the order the second product wants them: row
// 16 t + 4 g + v of the tile holds key 8 g + 4 t + v, so that after the first product a lane's eight
// scores are the keys 8 g .. 8 g + 7 of its row, the same eight keys that chunk g of a value row holds.
// Nothing is cleared in flight: in the blocks at the edges of a request the stale keys' values are
// cleared in shared memory after they have landed (their scores are masked in any case).
// 16 bytes per lane from global memory to shared memory without passing through registers: lane l's
// bytes land at dst + 16 l; dst is the same for the whole wavefront (its address goes through M0).
// Written as assembly on purpose.  Given the intrinsic, the compiler cannot tell which tile a later
// read of shared memory touches and makes every such read wait for all loads in flight, the next
// block's included, which is the overlap this kernel exists for.  So the compiler does not see
// these loads; the kernel waits for them itself (s_waitcnt vmcnt(0) and a barrier before a tile
// is read).  Loads the compiler does not know of can only make its own waits longer, never too short:
// loads return in order, and it waits for one of its own by counting the loads issued after it.
__device__ __forceinline__ void load_to_shared(const void* src, void* dst) {
    const uint32_t lds_address = __builtin_amdgcn_readfirstlane(
        static_cast<uint32_t>(reinterpret_cast<uintptr_t>((__attribute__((address_space(3))) void*)dst)));
    // M0 is put back as it was: naming it as clobbered instead makes the compiler wait for every load in
    // flight before the next read of shared memory
    uint32_t saved_m0;
    asm volatile("s_mov_b32 %0, m0\n\ts_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off\n\ts_mov_b32 m0, %0"
                 : "=&s"(saved_m0) : "v"(src), "s"(lds_address) : "memory");
}

// The same with the destination as a shared-memory address that is the same in all lanes (a scalar).
__device__ __forceinline__ void load_to_shared_at(const void* src, uint32_t lds_address) {
    uint32_t saved_m0;
    asm volatile("s_mov_b32 %0, m0\n\ts_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off\n\ts_mov_b32 m0, %0"
                 : "=&s"(saved_m0) : "v"(src), "s"(__builtin_amdgcn_readfirstlane(lds_address)) : "memory");
}
__device__ __forceinline__ uint32_t shared_address(const void* p) {
    return __builtin_amdgcn_readfirstlane(
        static_cast<uint32_t>(reinterpret_cast<uintptr_t>((__attribute__((address_space(3))) const void*)p)));
}

template <int HD>
__global__ void __launch_bounds__(kPrefillThreads, 2)
paged_attention_prefill_dma_kernel(const bf16* __restrict__ qkv, const bf16* __restrict__ cache,
                                   const int* __restrict__ block_tables, const int* __restrict__ items,
                                   const int* __restrict__ seg_q_start, const int* __restrict__ seg_q_len,
                                   const int* __restrict__ seg_ctx_len, bf16* __restrict__ out,
                                   float* __restrict__ partial_o, float* __restrict__ partial_ml, int num_heads,
                                   int num_kv_heads, int page_size, int max_pages, float scale_log2e, int window) {
    constexpr int DC = HD / 32, DT = HD / 16, CPR = HD / 8;       // CPR: 16-byte chunks of a key row
    constexpr int kKeyInstr = kBlockKeys * CPR / 64, kValInstr = HD * 4 / 64;    // wavefront loads per tile
    __shared__ __align__(16) uint16_t k_s0[kBlockKeys * HD], k_s1[kBlockKeys * HD];
    __shared__ __align__(16) uint16_t v_s0[HD * kBlockKeys], v_s1[HD * kBlockKeys];
    __shared__ int table_s[kMaxTablePages];

    const int* item = items + static_cast<size_t>(blockIdx.x) * kPrefillItemInts;
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

    constexpr int kPrefillRows = kPrefillWaves * 16;
    const int wr0 = row_begin + wave * 16;
    const int row = wr0 + i;
    const bool row_valid = row < total_rows;
    const int tok = row_valid ? row / group : 0;
    const int head = kvh * group + (row_valid ? row % group : 0);
    const int pos = first_pos + tok;
    const int lo = window > 0 ? max(0, pos - window + 1) : 0;
    bf16x8_t qreg[DC];
    {
        const bf16* qrow = qkv + static_cast<size_t>(q_start + tok) * width + static_cast<size_t>(head) * HD;
#pragma unroll
        for (int c = 0; c < DC; ++c) {
            PPack p;
            p.u = row_valid ? *reinterpret_cast<const uint4*>(qrow + c * 32 + 8 * g) : make_uint4(0, 0, 0, 0);
            qreg[c] = p.v;
        }
    }
    // the lowest position and the highest window start of the wavefront's rows
    int t_pos_min, t_lo_max;
    {
        const int last = min(total_rows - 1, wr0 + 15);
        t_pos_min = wr0 < total_rows ? first_pos + wr0 / group : -1;
        const int pmax = first_pos + max(last, 0) / group;
        t_lo_max = window > 0 ? max(0, pmax - window + 1) : 0;
        if (last < wr0 + 15) t_pos_min = -1;      // a tile with rows beyond the segment always masks
    }
    const bool wave_active = wr0 < total_rows;
    const int w_last_row = min(total_rows - 1, wr0 + 15);
    const int w_hi = wave_active ? first_pos + w_last_row / group + 1 : 0;                       // exclusive
    const int w_lo = window > 0 ? max(0, first_pos + wr0 / group - window + 1) : 0;
    const int b_last_row = min(total_rows - 1, row_begin + kPrefillRows - 1);
    const int b_hi = first_pos + b_last_row / group + 1;
    const int b_lo = window > 0 ? max(0, first_pos + row_begin / group - window + 1) : 0;
    const int blk_first = max(b_lo, key_begin) / kBlockKeys;
    const int blk_end = (min(b_hi, key_end) + kBlockKeys - 1) / kBlockKeys;
    const int page_base = blk_first * kBlockKeys / page_size;
    if (blk_first < blk_end) {
        const int* table_g = block_tables + static_cast<size_t>(seg) * max_pages + page_base;
        const int page_last = (min(blk_end * kBlockKeys, ctx) - 1) / page_size;
        const int count = min(min(max_pages - 1, page_last) - page_base + 1, kMaxTablePages);
        for (int p = tid; p < count; p += kPrefillThreads) table_s[p] = table_g[p];
    }

    float4_t acc[DT];
    float m_run = -INFINITY, l_run = 0.f;
#pragma unroll
    for (int t = 0; t < DT; ++t) acc[t] = float4_t{0.f, 0.f, 0.f, 0.f};

    // ---- the loads of a block.  The page size is a power of two here and a block begins at a multiple
    //      of 32 keys, so the place of a lane's key kbase + rel splits into a part all lanes share and the
    //      lane's own, which is worked out once: page (kbase >> shift) + (rel >> shift) of the request,
    //      slot (kbase & mask) + (rel & mask).  Per block and load that leaves one look-up in the table
    //      and one multiply-add for the address.  A page index beyond the request's last page (the keys
    //      after the end of the last block) is clamped: whatever lies there is masked and cleared. ----
    const int shift = __builtin_ctz(page_size), mask = page_size - 1;
    static_assert(kKeyInstr % kPrefillWaves == 0 && kValInstr % kPrefillWaves == 0, "whole loads per wavefront");
    constexpr int KU = kKeyInstr / kPrefillWaves, VU = kValInstr / kPrefillWaves;
    const uint32_t page_bytes = static_cast<uint32_t>(page_elems * 2);
    // keys: wavefront load q = wave + 4 u of the tile carries the chunks 64 q .. 64 q + 63 of the tile in
    // shared-memory order
    auto k_swizzle = [](int r) { return CPR >= 16 ? r % 16 : (r / 2) % 8; };      // what row r exchanges its chunks by
    int k_page[KU];
    const char* k_src[KU];
#pragma unroll
    for (int u = 0; u < KU; ++u) {
        const int chunk_index = (wave + u * kPrefillWaves) * 64 + lane;       // position in the tile, in chunks
        const int r = chunk_index / CPR;                                      // row of the tile
        const int chunk = (chunk_index % CPR) ^ k_swizzle(r);                 // the chunk of the key's row that lies there
        const int rel = 8 * ((r % 16) / 4) + 4 * (r / 16) + r % 4;            // the key of the block that row r holds
        k_page[u] = rel >> shift;
        k_src[u] = reinterpret_cast<const char*>(cache + k_off + static_cast<size_t>(rel & mask) * HD + chunk * 8);
    }
    // values: a lane moves the same chunk of 8 keys in every load, of the rows d = 16 q + lane / 4
    const int v_rel = 8 * ((lane % 4) ^ ((lane / 8) % 4));
    const int v_page = v_rel >> shift;
    const char* v_src[VU];
#pragma unroll
    for (int u = 0; u < VU; ++u) {
        const int d = (wave + u * kPrefillWaves) * 16 + lane / 4;
        v_src[u] = reinterpret_cast<const char*>(cache + v_off + static_cast<size_t>(d) * page_size + (v_rel & mask));
    }
    const int table_last = blk_first < blk_end
                               ? min(min(max_pages - 1, (min(blk_end * kBlockKeys, ctx) - 1) / page_size) - page_base + 1,
                                     kMaxTablePages) - 1
                               : 0;
    // where this wavefront's loads land: tile + 1 KiB * (wave + 4 u)
    const uint32_t k_lds[2] = {shared_address(k_s0) + wave * 1024u, shared_address(k_s1) + wave * 1024u};
    const uint32_t v_lds[2] = {shared_address(v_s0) + wave * 1024u, shared_address(v_s1) + wave * 1024u};
    auto issue = [&](int which, int kbase) {
        const int pb = (kbase >> shift) - page_base;
        const uint32_t k_slot_bytes = static_cast<uint32_t>(kbase & mask) * HD * 2, v_slot_bytes = static_cast<uint32_t>(kbase & mask) * 2;
        int kp[KU];
#pragma unroll
        for (int u = 0; u < KU; ++u) kp[u] = table_s[min(pb + k_page[u], table_last)];
        const int vp = table_s[min(pb + v_page, table_last)];
#pragma unroll
        for (int u = 0; u < KU; ++u)
            load_to_shared_at(k_src[u] + (static_cast<uint64_t>(static_cast<uint32_t>(kp[u])) * page_bytes + k_slot_bytes),
                              k_lds[which] + u * (kPrefillWaves * 1024u));
        const uint64_t v_page_bytes = static_cast<uint64_t>(static_cast<uint32_t>(vp)) * page_bytes + v_slot_bytes;
#pragma unroll
        for (int u = 0; u < VU; ++u) load_to_shared_at(v_src[u] + v_page_bytes, v_lds[which] + u * (kPrefillWaves * 1024u));
    };

    __syncthreads();      // the block table is in shared memory
    if (blk_first < blk_end) issue(0, blk_first * kBlockKeys);
    // One block: its tiles are k_s and v_s, the next block's loads go to k_next and v_next.  The loop below
    // names the two pairs of tiles in turn, so every address in shared memory is a constant plus a lane's
    // fixed offset.
    // a lane's fragment reads: every address is the tile, the lane's offset and a constant.  With x what row i
    // exchanges by, chunk (4 c + g) ^ x of a key row is 4 (c ^ (x >> 2)) + (g ^ (x & 3)), and x >> 2 touches the
    // two low bits of c only: one offset for each c % 4.
    const int k_x = k_swizzle(i);
    int k_lane[4];
#pragma unroll
    for (int c = 0; c < 4; ++c) k_lane[c] = (i * CPR + 4 * ((c ^ (k_x >> 2)) % DC) + (g ^ (k_x & 3))) * 8;
    const int v_lane = (i * 4 + (g ^ ((i / 2) % 4))) * 8;
    auto block = [&](int blk, const uint16_t* k_s, uint16_t* v_s, int next) {
        const int kbase = blk * kBlockKeys;
        __builtin_amdgcn_s_waitcnt(0);   // this lane's loads of the block have landed
        __syncthreads();                 // everyone's have, and everyone is done with the block before
        if (kbase + kBlockKeys > ctx || kbase < seg_lo) {
            // a block at the edge of the request: the values of keys that are not the request's are cleared
            if (tid < HD) {
                for (int kib = 0; kib < kBlockKeys; ++kib) {
                    const int key = kbase + kib;
                    if (key >= ctx || key < seg_lo) v_s[(tid * 4 + ((kib / 8) ^ ((tid / 2) % 4))) * 8 + kib % 8] = 0;
                }
            }
            __syncthreads();
        }
        // The order below is kept as written (nothing moves across a sched_barrier): all fragments of the keys
        // are asked for before the next block's loads are, the values' fragments before the softmax, so that
        // a product waits for no read that was asked for just before it.  Left to itself the compiler keeps two
        // reads in flight and every product waits a trip to shared memory.
        const bool active = wave_active && kbase < w_hi && kbase + kBlockKeys > w_lo;
        PPack kf[2 * DC], vf[DT];
        if (active) {
#pragma unroll
            for (int t2 = 0; t2 < 2; ++t2)
#pragma unroll
                for (int c = 0; c < DC; ++c)
                    kf[t2 * DC + c].u = *reinterpret_cast<const uint4*>(&k_s[k_lane[c % 4] + (16 * t2 * CPR + 4 * (c & ~3)) * 8]);
        }
        __builtin_amdgcn_sched_barrier(0);
        if (blk + 1 < blk_end) issue(next, kbase + kBlockKeys);
        if (!active) return;
        __builtin_amdgcn_sched_barrier(0);
        // ---- scores: tile t2, lane (i, g) gets the keys 8 g + 4 t2 + v of the block ----
        float sv[8];
#pragma unroll
        for (int t2 = 0; t2 < 2; ++t2) {
            float4_t sc = float4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int c = 0; c < DC; ++c) sc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[t2 * DC + c].v, qreg[c], sc, 0, 0, 0);
#pragma unroll
            for (int v = 0; v < 4; ++v) sv[4 * t2 + v] = sc[v];
        }
#pragma unroll
        for (int t = 0; t < DT; ++t) vf[t].u = *reinterpret_cast<const uint4*>(&v_s[v_lane + 16 * t * 4 * 8]);
        __builtin_amdgcn_sched_barrier(0);
        // ---- softmax bookkeeping ----
        const bool inside = kbase + kBlockKeys - 1 <= t_pos_min && kbase >= t_lo_max;
        if (!inside) {
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const int key = kbase + 8 * g + e;
                if (!(row_valid && key <= pos && key >= lo)) sv[e] = -INFINITY;
            }
        }
        float tile_max = fmaxf(fmaxf(fmaxf(sv[0], sv[1]), fmaxf(sv[2], sv[3])), fmaxf(fmaxf(sv[4], sv[5]), fmaxf(sv[6], sv[7])));
        tile_max = max_across(max_across(tile_max, 16), 32);
        const float m_new = fmaxf(m_run, tile_max);
        const float m_use = m_new == -INFINITY ? 0.f : m_new;
        const float mc = m_use * scale_log2e;
        const float alpha = exp2_probability(fmaf(m_run, scale_log2e, -mc));
        float pe[8], psum = 0.f;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            pe[e] = exp2_probability(fmaf(sv[e], scale_log2e, -mc));       // exp2(-inf) = 0 for masked keys
            psum += pe[e];
        }
        PPack pv;
        pv.u = make_uint4(pack2_bf16(pe[0], pe[1]), pack2_bf16(pe[2], pe[3]), pack2_bf16(pe[4], pe[5]), pack2_bf16(pe[6], pe[7]));
        l_run = l_run * alpha + psum;
        m_run = m_new;
        // ---- out^T += V^T . P^T; the accumulators are rescaled only when some row's maximum moved: one
        // branch for the whole wavefront around all of them (a test per accumulator becomes a multiply and a
        // select for each of its 64 numbers, whether or not anything moved) ----
        if (__builtin_amdgcn_readfirstlane(__any(alpha != 1.f))) {
#pragma unroll
            for (int t = 0; t < DT; ++t) acc[t] *= alpha;
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int t = 0; t < DT; ++t) acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf[t].v, pv.v, acc[t], 0, 0, 0);
    };
    for (int blk = blk_first; blk < blk_end; blk += 2) {
        block(blk, k_s0, v_s0, 1);
        if (blk + 1 < blk_end) block(blk + 1, k_s1, v_s1, 0);
    }
    float l = l_run;
    l = sum_across(sum_across(l, 16), 32);
    if (!row_valid) return;
    if (partial_slot >= 0) {
        const size_t slot = static_cast<size_t>(partial_slot) + wave;
        float* po = partial_o + (slot * 16 + i) * HD;
#pragma unroll
        for (int t = 0; t < DT; ++t)
            *reinterpret_cast<float4*>(po + t * 16 + 4 * g) = make_float4(acc[t][0], acc[t][1], acc[t][2], acc[t][3]);
        if (g == 0) *reinterpret_cast<float2*>(partial_ml + (slot * 16 + i) * 2) = make_float2(m_run, l);
        return;
    }
    const float inv = 1.f / l;
    bf16* orow = out + (static_cast<size_t>(q_start + tok) * num_heads + head) * HD;
#pragma unroll
    for (int t = 0; t < DT; ++t) {
        uint2 w;
        w.x = pack2_bf16(acc[t][0] * inv, acc[t][1] * inv);
        w.y = pack2_bf16(acc[t][2] * inv, acc[t][3] * inv);
        *reinterpret_cast<uint2*>(orow + t * 16 + 4 * g) = w;
    }
}

// Returns 0, a HIP error code, or -1 for sizes this kernel does not take.
WLLM_API int wllm_paged_attention_prefill(const void* qkv, const void* cache, const int* block_tables,
                                          const int* items, int num_items, int rows_per_item, const int* seg_q_start,
                                          const int* seg_q_len, const int* seg_ctx_len, void* out, float* partial_o,
                                          float* partial_ml, int num_heads,
                                          int num_kv_heads, int head_dim, int page_size, int max_pages, float scale,
                                          int window, hipStream_t stream) {
    if (head_dim % 32 != 0 || head_dim < 32 || head_dim > 256 || page_size % 4 != 0 || num_heads % num_kv_heads != 0)
        return -1;
    if (rows_per_item != 64) return -1;
    if (num_items <= 0) return 0;
    const float scale_log2e = scale * 1.4426950408889634f;
    if (page_size >= 8 && (page_size & (page_size - 1)) == 0 && (head_dim == 64 || head_dim == 128 || head_dim == 256)) {
#define LAUNCH_DMA(HD)                                                                                              \
    paged_attention_prefill_dma_kernel<HD><<<num_items, kPrefillThreads, 0, stream>>>(                              \
        static_cast<const bf16*>(qkv), static_cast<const bf16*>(cache), block_tables, items, seg_q_start, seg_q_len, \
        seg_ctx_len, static_cast<bf16*>(out), partial_o, partial_ml, num_heads, num_kv_heads, page_size, max_pages, \
        scale_log2e, window)
        if (head_dim == 64) LAUNCH_DMA(64);
        else if (head_dim == 128) LAUNCH_DMA(128);
        else LAUNCH_DMA(256);
#undef LAUNCH_DMA
        return launch_status();
    }
#define LAUNCH_RTW(HD, RTW)                                                                                         \
    paged_attention_prefill_kernel<HD, RTW><<<num_items, kPrefillThreads, 0, stream>>>(                             \
        static_cast<const bf16*>(qkv), static_cast<const bf16*>(cache), block_tables, items, seg_q_start, seg_q_len, \
        seg_ctx_len, static_cast<bf16*>(out), partial_o, partial_ml, num_heads, num_kv_heads, page_size, max_pages, \
        scale_log2e, window)
#define LAUNCH(HD) LAUNCH_RTW(HD, 1)
    switch (head_dim) {
        case 32: LAUNCH(32); break;
        case 64: LAUNCH(64); break;
        case 96: LAUNCH(96); break;
        case 128: LAUNCH(128); break;
        case 160: LAUNCH(160); break;
        case 192: LAUNCH(192); break;
        case 224: LAUNCH(224); break;
        case 256: LAUNCH(256); break;
        default: return -1;
    }
#undef LAUNCH
#undef LAUNCH_RTW
    return launch_status();
}
