// The query/key/value projection of a decode step, its bias, the rotation of queries and keys and
// the write of keys and values into their pages, in one kernel: for at most 32 tokens, bfloat16,
// heads whose size is a multiple of 32 and that are rotated whole.
//
// out[m, :] = x[m, :] . w^T as in `gemm_skinny.hip` (weights as the A operand of
// v_mfma_f32_16x16x32_bf16, read row by row or from the tile-major copy).  A workgroup owns two
// bands of 16 columns of one head that the rotation pairs: columns 16p .. 16p+15 and the same
// HD/2 further on.  Its eight wavefronts split the K axis, issue all their loads before the first
// product (a register is refilled as soon as its product is issued), and add their sums through
// shared memory in the order of the pieces.  The first wavefront then holds, per lane, four
// columns of both bands for one token: element j of the head and its partner j + HD/2, so the
// pair is turned in registers by position * inv_freq[j] (angle, sine, cosine in float32), written
// to the row of queries, keys and values, and keys go to the cache as [page_size, HD], values
// transposed as [HD, page_size].  Heads of values take the same path without the rotation.
// 17 to 32 tokens are two tiles of 16: every fragment of the weights then feeds two products.  (Three
// and four tiles were measured too: with fewer steps in flight to fit the registers they are no faster
// than the product and the rotation as two kernels.)
#include "common.h"

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float float4_t __attribute__((ext_vector_type(4)));

union QFrag {
    uint4 u;
    bf16x8_t v;
};

constexpr int kQkvWaves = 8;

// What the first wavefront does with one token's sums of a pair of bands: bias, the rotation of the
// pair (element j of the head with j + HD/2), the row of queries, keys and values, and the cache.
__device__ __forceinline__ void finish_row(float4_t acc_lo, float4_t acc_hi, const float* __restrict__ bias, int col, int half,
                                           bool rotated, float pos, const float* fr, bf16* __restrict__ qkv, int m, int width,
                                           bf16* __restrict__ cache, int head, int num_heads, int num_kv_heads, int slot,
                                           int page_size, long long num_pages, size_t page_elems, int HD, int j0) {
    if (bias) {
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            acc_lo[v] += bias[col + v];
            acc_hi[v] += bias[col + half + v];
        }
    }
    if (rotated) {
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            float s, c;
            sincosf(pos * fr[v], &s, &c);
            const float a = acc_lo[v], b = acc_hi[v];
            float ra, rb;
            rotate_pair(a, b, s, c, ra, rb);
            acc_lo[v] = ra;
            acc_hi[v] = rb;
        }
    }
    uint2 plo, phi;
    plo.x = pack2_bf16(acc_lo[0], acc_lo[1]);
    plo.y = pack2_bf16(acc_lo[2], acc_lo[3]);
    phi.x = pack2_bf16(acc_hi[0], acc_hi[1]);
    phi.y = pack2_bf16(acc_hi[2], acc_hi[3]);
    bf16* row = qkv + static_cast<size_t>(m) * width + col;
    *reinterpret_cast<uint2*>(row) = plo;
    *reinterpret_cast<uint2*>(row + half) = phi;
    if (!cache || head < num_heads) return;
    const long long page = slot / page_size;
    const int off = slot % page_size;
    if (slot < 0 || page >= num_pages) return;
    bf16* kpage = cache + page * page_elems;
    if (head < num_heads + num_kv_heads) {
        bf16* dst = kpage + (static_cast<size_t>(head - num_heads) * page_size + off) * HD + j0;
        *reinterpret_cast<uint2*>(dst) = plo;
        *reinterpret_cast<uint2*>(dst + half) = phi;
    } else {
        bf16* vpage = kpage + static_cast<size_t>(num_kv_heads) * page_size * HD;
        const int vh = head - num_heads - num_kv_heads;
        const uint16_t el[4] = {static_cast<uint16_t>(plo.x & 0xffff), static_cast<uint16_t>(plo.x >> 16),
                                static_cast<uint16_t>(plo.y & 0xffff), static_cast<uint16_t>(plo.y >> 16)};
        const uint16_t eh[4] = {static_cast<uint16_t>(phi.x & 0xffff), static_cast<uint16_t>(phi.x >> 16),
                                static_cast<uint16_t>(phi.y & 0xffff), static_cast<uint16_t>(phi.y >> 16)};
        uint16_t* vp = reinterpret_cast<uint16_t*>(vpage);
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            vp[(static_cast<size_t>(vh) * HD + j0 + v) * page_size + off] = el[v];
            vp[(static_cast<size_t>(vh) * HD + j0 + half + v) * page_size + off] = eh[v];
        }
    }
}

template <bool TILED, int MT>
__global__ void __launch_bounds__(kQkvWaves * 64)
qkv_rope_kernel(const bf16* __restrict__ x, const bf16* __restrict__ w, const float* __restrict__ bias,
                const int* __restrict__ positions, const float* __restrict__ inv_freq, const int* __restrict__ slots,
                bf16* __restrict__ qkv, bf16* __restrict__ cache, int M, int K, int num_heads, int num_kv_heads, int HD,
                int page_size, long long num_pages) {
    __shared__ float4_t red[(kQkvWaves - 1) * kWave * 2 * MT];
    const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
    const int i = lane % 16, g = lane / 16;
    const int pairs = HD / 32;                          // pairs of bands in a head
    const int head = blockIdx.x / pairs, p = blockIdx.x % pairs;
    const int band_lo = head * (HD / 16) + p, band_hi = band_lo + pairs;
    const int steps = K / 32;
    const int per = (steps + kQkvWaves - 1) / kQkvWaves;
    const int s0 = wave * per, s1 = min(steps, s0 + per);
    constexpr int kStep = TILED ? 512 : 32;             // elements from one step of 32 keys to the next
    const bf16* lo = TILED ? w + static_cast<size_t>(band_lo) * steps * 512 + lane * 8
                           : w + (static_cast<size_t>(band_lo) * 16 + i) * K + 8 * g;
    const bf16* hi = TILED ? w + static_cast<size_t>(band_hi) * steps * 512 + lane * 8
                           : w + (static_cast<size_t>(band_hi) * 16 + i) * K + 8 * g;
    const bf16* xp[MT];
    bool x_row[MT];
#pragma unroll
    for (int t = 0; t < MT; ++t) {
        xp[t] = x + static_cast<size_t>(min(16 * t + i, M - 1)) * K + 8 * g;
        x_row[t] = 16 * t + i < M;
    }
    // what the first wavefront needs after the sums, asked for now so that it has arrived by then
    const int j0 = p * 16 + 4 * g, half = HD / 2;
    const bool rotated = head < num_heads + num_kv_heads && inv_freq != nullptr;
    float pos[MT];
    float4 freq = make_float4(0.f, 0.f, 0.f, 0.f);
    int slot[MT];
#pragma unroll
    for (int t = 0; t < MT; ++t) {
        pos[t] = 0.f;
        slot[t] = -1;
        if (wave == 0 && x_row[t]) {
            if (rotated) pos[t] = static_cast<float>(positions[16 * t + i]);
            if (cache && head >= num_heads) slot[t] = slots[16 * t + i];
        }
    }
    if (wave == 0 && rotated) freq = *reinterpret_cast<const float4*>(inv_freq + j0);
    constexpr int U = 8;        // steps of 32 keys whose loads a wavefront keeps in flight, per band
    QFrag cl[U], ch[U], cx[U][MT];
    auto load_step = [&](int u, int at) {
        const bool ok = at < s1;
        cl[u].u = ok ? load_streamed(lo + static_cast<size_t>(at) * kStep) : make_uint4(0, 0, 0, 0);
        ch[u].u = ok ? load_streamed(hi + static_cast<size_t>(at) * kStep) : make_uint4(0, 0, 0, 0);
#pragma unroll
        for (int t = 0; t < MT; ++t)
            cx[u][t].u = ok && x_row[t] ? *reinterpret_cast<const uint4*>(xp[t] + static_cast<size_t>(at) * 32) : make_uint4(0, 0, 0, 0);
    };
#pragma unroll
    for (int u = 0; u < U; ++u) load_step(u, s0 + u);
    float4_t acc_lo[MT], acc_hi[MT];
#pragma unroll
    for (int t = 0; t < MT; ++t) {
        acc_lo[t] = float4_t{0.f, 0.f, 0.f, 0.f};
        acc_hi[t] = float4_t{0.f, 0.f, 0.f, 0.f};
    }
    for (int s = s0; s < s1; s += U) {
#pragma unroll
        for (int u = 0; u < U; ++u) {
#pragma unroll
            for (int t = 0; t < MT; ++t) {
                acc_lo[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(cl[u].v, cx[u][t].v, acc_lo[t], 0, 0, 0);
                acc_hi[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ch[u].v, cx[u][t].v, acc_hi[t], 0, 0, 0);
            }
            load_step(u, s + U + u);
        }
    }
    if (wave > 0) {
#pragma unroll
        for (int t = 0; t < MT; ++t) {
            red[(((wave - 1) * kWave + lane) * MT + t) * 2] = acc_lo[t];
            red[(((wave - 1) * kWave + lane) * MT + t) * 2 + 1] = acc_hi[t];
        }
    }
    __syncthreads();
    if (wave > 0) return;
#pragma unroll
    for (int q = 0; q < kQkvWaves - 1; ++q)
#pragma unroll
        for (int t = 0; t < MT; ++t) {
            acc_lo[t] += red[((q * kWave + lane) * MT + t) * 2];
            acc_hi[t] += red[((q * kWave + lane) * MT + t) * 2 + 1];
        }
    const int width = (num_heads + 2 * num_kv_heads) * HD;
    const int col = head * HD + j0;
    const float fr[4] = {freq.x, freq.y, freq.z, freq.w};
    const size_t page_elems = static_cast<size_t>(2) * num_kv_heads * page_size * HD;
    // lane (i, g): token m = 16 t + i, elements j .. j + 3 of the head and their partners
#pragma unroll
    for (int t = 0; t < MT; ++t) {
        const int m = 16 * t + i;
        if (m >= M) continue;
        finish_row(acc_lo[t], acc_hi[t], bias, col, half, rotated, pos[t], fr, qkv, m, width, cache, head, num_heads,
                   num_kv_heads, slot[t], page_size, num_pages, page_elems, HD, j0);
    }
}
// Returns 0, a HIP error code, or -1 for sizes this kernel does not take (the caller then runs the
// product and the rotation as two kernels).  `w` is the stacked [q; k; v] weight, row by row or
// (`tiled`) its tile-major copy.  inv_freq has HD/2 entries or is null (no rotation).
WLLM_API int wllm_qkv_rope(const void* x, const void* w, int tiled, const float* bias, const int* positions,
                           const float* inv_freq, const int* slots, void* qkv, void* cache, long long num_pages, int M,
                           int K, int num_heads, int num_kv_heads, int head_dim, int page_size, hipStream_t stream) {
    if (M < 1 || M > 32 || K < 32 || K % 32 != 0 || head_dim < 32 || head_dim % 32 != 0 || num_heads < 1 || num_kv_heads < 1 ||
        page_size < 1)
        return -1;
    const int grid = (num_heads + 2 * num_kv_heads) * (head_dim / 32);
#define LAUNCH(T, MT)                                                                                                  \
    qkv_rope_kernel<T, MT><<<grid, kQkvWaves * 64, 0, stream>>>(                                                       \
        static_cast<const bf16*>(x), static_cast<const bf16*>(w), bias, positions, inv_freq, slots, static_cast<bf16*>(qkv), \
        static_cast<bf16*>(cache), M, K, num_heads, num_kv_heads, head_dim, page_size, num_pages)
    if (tiled) {
        if (M <= 16) LAUNCH(true, 1);
        else LAUNCH(true, 2);
    } else {
        if (M <= 16) LAUNCH(false, 1);
        else LAUNCH(false, 2);
    }
#undef LAUNCH
    return launch_status();
}
