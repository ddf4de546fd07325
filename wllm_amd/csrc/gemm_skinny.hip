// out[M, N] = x[M, K] * w[N, K]^T for bfloat16 with few rows (M <= 64): the product of a decode
// step, bound by reading w once from HBM.
//
// v_mfma_f32_16x16x32_bf16 with the weights as the A operand: a wavefront owns 16 rows of w (16
// columns of the result) and streams them with 16-byte loads, lane (i, g) reading
// w[n0 + i][k + 8g .. +8]; the rows of x are the B operand, staged through shared memory once per
// workgroup and chunk of K and read back as 16-byte fragments; each 16-row tile of x costs one more
// MFMA per 32 k, which is free beside the weight stream.  The result tile lands as C[n = 4g + v][m = i],
// four consecutive columns of one output row per lane.  A workgroup is 4 wavefronts = 64 rows of w.
// When N is small the K axis is split over workgroups (grid.y) so that enough wavefronts stream at
// once; the partial sums are float32 and a second kernel adds them in split order.  The split
// depends on N and K only, and every output element is summed over k in ascending order, so a
// row's result does not depend on how many other rows the batch has.
#include "common.h"

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float float4_t __attribute__((ext_vector_type(4)));

union Frag {
    uint4 u;
    bf16x8_t v;
};

// ---- the tile-major copy of a weight that the few-row kernels stream --------------------------
// dst holds, for each band of 16 rows (the last one padded with zero rows) and each step of 32
// keys, the tile's 1 KiB: lane l = 16g + i holds w[16 * band + i][32 * step + 8g .. +8].  A
// wavefront's load of a tile is then one contiguous KiB and its walk along K one contiguous run,
// which the memory system serves faster than 16 pieces of 64 bytes a row apart.
__global__ void tile_weight_kernel(const bf16* __restrict__ src, bf16* __restrict__ dst, int N, int K, long long pieces) {
    const long long p = static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (p >= pieces) return;
    const int lane = static_cast<int>(p % 64);
    const long long tile = p / 64;
    const int steps = K / 32;
    const int step = static_cast<int>(tile % steps);
    const long long band = tile / steps;
    const long long row = band * 16 + lane % 16;
    uint4 v = make_uint4(0, 0, 0, 0);
    if (row < N) v = *reinterpret_cast<const uint4*>(src + row * K + step * 32 + 8 * (lane / 16));
    *reinterpret_cast<uint4*>(dst + p * 8) = v;
}

// dst must hold ceil(N / 16) * 16 * K elements.  Returns 0, a HIP error code, or -1 for sizes it does not take.
WLLM_API int wllm_tile_weight(const void* src, void* dst, int N, int K, hipStream_t stream) {
    if (N < 1 || K < 32 || K % 32 != 0) return -1;
    const long long pieces = static_cast<long long>((N + 15) / 16) * (K / 32) * 64;
    const long long blocks = (pieces + 255) / 256;
    if (blocks > 0x7fffffffLL) return -1;
    tile_weight_kernel<<<static_cast<unsigned>(blocks), 256, 0, stream>>>(static_cast<const bf16*>(src), static_cast<bf16*>(dst), N, K,
                                                                        pieces);
    return launch_status();
}

template <typename TO> __device__ __forceinline__ void store4(TO* p, float4_t v);
template <> __device__ __forceinline__ void store4<float>(float* p, float4_t v) { *reinterpret_cast<float4_t*>(p) = v; }
template <> __device__ __forceinline__ void store4<bf16>(bf16* p, float4_t v) {
    uint2 w;
    w.x = pack2_bf16(v[0], v[1]);
    w.y = pack2_bf16(v[2], v[3]);
    *reinterpret_cast<uint2*>(p) = w;
}

// NT: tiles of 16 weight rows per wavefront.  With many rows of x (MT > 1) every fragment of x read
// from shared memory then feeds NT products, and a workgroup stages x once for 64*NT weight rows.
// TILED: w is stored tile by tile (see `wllm_tile_weight`): a tile of 16 rows and 32 keys as the 16
// bytes of each of the 64 lanes in lane order, the tiles of a band of 16 rows one after the other along
// K, so a wavefront streams one contiguous run.
//
// More than 64 rows (row_groups > 1, unsplit products only): groups of 64 rows are made by workgroups of
// their own that read the same weights.  The workgroups of a tile's row groups get indices that are 8
// apart, so they are dispatched one after the other to the same XCD (workgroup index modulo 8) and the
// later ones find the weights in that XCD's L2 instead of asking HBM for them again.
template <int MT, int NT, typename TO, bool TILED>
__global__ void __launch_bounds__(256)
gemm_skinny_kernel(const bf16* __restrict__ x, const bf16* __restrict__ w, TO* __restrict__ out,
                   float* __restrict__ partial, int M, int N, int K, int k_per_split, int chunk, int row_groups, int splits) {
    extern __shared__ uint4 xs[];                 // [MT*16][chunk/8 + 1]
    const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
    const int i = lane % 16, g = lane / 16;
    int tile_group = blockIdx.x;                  // which 64 * NT weight rows
    int split = 0;                                // which piece of the K axis
    if (splits > 1) {
        // The workgroups of one piece of the K axis read the same part of x: they get indices that are
        // equal modulo 8, so they run on one XCD and all but the first find that part in its L2.  (The
        // XCDs' caches are separate: a part of x that all eight of them read crosses the fabric eight
        // times, which at 64 rows and a long K axis is a quarter of what the weights take.)
        const int xcd = blockIdx.x % 8, j = blockIdx.x / 8;
        if (splits >= 8) {
            const int per = splits / 8;           // splits is a power of two
            split = xcd * per + j % per;
            tile_group = j / per;
        } else {
            split = xcd % splits;
            tile_group = xcd / splits + (8 / splits) * j;
            if (tile_group * 64 * NT >= N) return;     // the grid is padded to whole rounds of 8
        }
    }
    if (row_groups > 1) {
        const int xcd = blockIdx.x % 8, j = blockIdx.x / 8;
        const int rg = j % row_groups;
        tile_group = (j / row_groups) * 8 + xcd;
        x += static_cast<size_t>(rg) * 64 * K;
        out += static_cast<size_t>(rg) * 64 * N;
        M = min(64, M - rg * 64);
    }
    const int n0 = (tile_group * 4 + wave) * 16 * NT;
    const int k_begin = split * k_per_split, k_end = min(K, k_begin + k_per_split);
    const int stride = chunk / 8 + 1;             // in uint4; the odd stride spreads rows over the banks
    constexpr int kStep = TILED ? 512 : 32;       // elements from one step of 32 keys to the next
    const bf16* wp[NT];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
        if (TILED) {
            const int band = min(n0 / 16 + nt, (N + 15) / 16 - 1);
            wp[nt] = w + (static_cast<size_t>(band) * (K / 32) + k_begin / 32) * 512 + lane * 8;
        } else {
            wp[nt] = w + static_cast<size_t>(min(n0 + nt * 16 + i, N - 1)) * K + k_begin + 8 * g;
        }
    }
    float4_t acc[NT][MT];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int t = 0; t < MT; ++t) acc[nt][t] = float4_t{0.f, 0.f, 0.f, 0.f};

    // The weight stream: kBatch 16-byte loads per lane and tile are in flight, the first before x is
    // staged at all; a register is refilled with the step kBatch further on as soon as its products
    // have been issued.
    constexpr int kBatch = 16 / NT;
    const bool live = n0 < N;
    const int steps = (k_end - k_begin) / 32;
    Frag cur[NT][kBatch];
    auto load_step = [&](int u, int at) {
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
            cur[nt][u].u = (live && at < steps) ? (row_groups > 1 ? *reinterpret_cast<const uint4*>(wp[nt] + at * kStep)
                                                                  : load_streamed(wp[nt] + at * kStep))
                                                : make_uint4(0, 0, 0, 0);
    };
#pragma unroll
    for (int u = 0; u < kBatch; ++u) load_step(u, u);
    // x is staged chunk by chunk; the loads of the next chunk are in flight during the products
    constexpr int kXRegs = 8;                     // 16-byte pieces of a chunk per thread (MT*16*chunk/8 <= 2048)
    uint4 xreg[kXRegs];
    // A thread's pieces are (row, 8 keys) pairs of the whole chunk's shape, piece number threadIdx.x +
    // 256 u; their places are worked out once, not per chunk (a division by a run-time number costs
    // some forty instructions), and a shorter last chunk only leaves pieces out.
    const int vecs_full = chunk / 8;
    int x_col[kXRegs], x_row[kXRegs];
    {
        const int dq = 256 / vecs_full, dr = 256 % vecs_full;
        int m = threadIdx.x / vecs_full, c = threadIdx.x % vecs_full;
#pragma unroll
        for (int u = 0; u < kXRegs; ++u) {
            x_row[u] = m < MT * 16 ? m : -1;
            x_col[u] = c;
            m += dq;
            c += dr;
            if (c >= vecs_full) { c -= vecs_full; ++m; }
        }
    }
    auto fetch_x = [&](int kc) {
        const int vecs = min(chunk, k_end - kc) / 8;
#pragma unroll
        for (int u = 0; u < kXRegs; ++u) {
            const int m = x_row[u], c = x_col[u];
            xreg[u] = (m >= 0 && m < M && c < vecs) ? *reinterpret_cast<const uint4*>(x + static_cast<size_t>(m) * K + kc + c * 8)
                                                    : make_uint4(0, 0, 0, 0);
        }
    };
    fetch_x(k_begin);
    int step = 0;
    for (int kc = k_begin; kc < k_end; kc += chunk) {
        const int len = min(chunk, k_end - kc);   // a multiple of 32 * kBatch, except the last
        const int vecs = len / 8;
        __syncthreads();
#pragma unroll
        for (int u = 0; u < kXRegs; ++u)
            if (x_row[u] >= 0 && x_col[u] < vecs) xs[x_row[u] * stride + x_col[u]] = xreg[u];
        __syncthreads();
        if (kc + chunk < k_end) fetch_x(kc + chunk);
        for (int k = 0; k < len; k += 32 * kBatch) {
#pragma unroll
            for (int u = 0; u < kBatch; ++u) {
                if (k + 32 * u < len) {
                    Frag b[MT];
#pragma unroll
                    for (int t = 0; t < MT; ++t) b[t].u = xs[(t * 16 + i) * stride + k / 8 + 4 * u + g];
#pragma unroll
                    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
                        for (int t = 0; t < MT; ++t)
                            acc[nt][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(cur[nt][u].v, b[t].v, acc[nt][t], 0, 0, 0);
                    load_step(u, step + u + kBatch);
                }
            }
            step += kBatch;
        }
    }
    if (!live) return;
    // lane (i, g) holds columns n .. n + 3 of row m = 16t + i
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
        const int n = n0 + nt * 16 + 4 * g;
        if (n >= N) continue;
#pragma unroll
        for (int t = 0; t < MT; ++t) {
            const int m = t * 16 + i;
            if (m >= M) continue;
            if (splits == 1) {
                TO* o = out + static_cast<size_t>(m) * N + n;
                if (n + 3 < N && (N % 4 == 0)) {
                    store4<TO>(o, acc[nt][t]);
                } else {
#pragma unroll
                    for (int v = 0; v < 4; ++v)
                        if (n + v < N) o[v] = from_float<TO>(acc[nt][t][v]);
                }
            } else {
                float* o = partial + (static_cast<size_t>(split) * M + m) * N + n;
                if (n + 3 < N && (N % 4 == 0)) {
                    *reinterpret_cast<float4_t*>(o) = acc[nt][t];
                } else {
#pragma unroll
                    for (int v = 0; v < 4; ++v)
                        if (n + v < N) o[v] = acc[nt][t][v];
                }
            }
        }
    }
}

template <typename TO>
__global__ void split_sum_kernel(const float* __restrict__ partial, TO* __restrict__ out, long long total, int splits) {
    const long long stride = static_cast<long long>(gridDim.x) * blockDim.x;
    for (long long idx = static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x; idx < total; idx += stride) {
        float s = 0.f;
        for (int p = 0; p < splits; ++p) s += partial[p * total + idx];
        out[idx] = from_float<TO>(s);
    }
}

// out[i] = the sum in order of partial[p * total + i], p < splits.
WLLM_API int wllm_split_sum(const float* partial, void* out, int out_bf16, long long total, int splits, hipStream_t stream) {
    if (total < 1 || splits < 1) return -1;
    const long long want = (total + 255) / 256;
    const int blocks = static_cast<int>(want < 4096 ? want : 4096);
    if (out_bf16) split_sum_kernel<bf16><<<blocks, 256, 0, stream>>>(partial, static_cast<bf16*>(out), total, splits);
    else split_sum_kernel<float><<<blocks, 256, 0, stream>>>(partial, static_cast<float*>(out), total, splits);
    return launch_status();
}

// Returns 0, a HIP error code, or -1 for sizes this kernel does not take.
// `partial` must hold splits * M * N floats when splits > 1; with `out` null the partial sums
// are the result and nothing adds them.
WLLM_API int wllm_gemm_skinny(const void* x, const void* w, int tiled, void* out, int out_bf16, float* partial, int M,
                              int N, int K, int splits, int chunk, hipStream_t stream) {
    if (M < 1 || K % 32 != 0 || splits < 1 || K % splits != 0 || (K / splits) % 32 != 0 || chunk % 32 != 0)
        return -1;
    // every result needs somewhere to go: a split product its partial sums, an unsplit one its output
    if ((splits > 1 && partial == nullptr) || (splits == 1 && out == nullptr)) return -1;
    // more than 64 rows: groups of 64 rows by workgroups of their own, for unsplit products
    const int row_groups = (M + 63) / 64;
    if (row_groups > 1 && splits != 1) return -1;
    const int mt = row_groups > 1 ? 4 : (M + 15) / 16;
    const int k_per_split = K / splits;
    if (chunk > k_per_split) chunk = k_per_split;
    const size_t smem = static_cast<size_t>(mt) * 16 * (chunk / 8 + 1) * sizeof(uint4);
    if (smem > 65536 || mt * 16 * (chunk / 8) > 2048) return -1;     // 8 pieces of x per thread at most
    // weight rows per wavefront: more when x has many rows, as long as about a thousand wavefronts remain
    const long long tiles = (N + 15) / 16;
    int nt = 1;
    if (mt >= 2) {
        if (tiles / 4 * splits >= 1024) nt = 4;
        else if (tiles / 2 * splits >= 1024) nt = 2;
    }
    // a wavefront reads its weights in batches of 16 / nt steps of 32 keys; a chunk of x that is not the
    // last must be whole batches
    if (chunk < k_per_split) {
        while (nt < 4 && chunk % ((16 / nt) * 32) != 0) nt *= 2;
        if (chunk % ((16 / nt) * 32) != 0) return -1;     // a register's step is fixed by its place in the batch
    }
    // with row groups the tile groups are padded to a multiple of 8, one stripe per XCD (tile groups beyond
    // the last hold no live weight rows and write nothing)
    const int tile_groups = (N + 64 * nt - 1) / (64 * nt);
    long long blocks = row_groups > 1 ? static_cast<long long>((tile_groups + 7) / 8 * 8) * row_groups : tile_groups;
    if (splits > 1) {
        // one index for pieces of K and tile groups, the pieces spread over the XCDs (see the kernel)
        if ((splits & (splits - 1)) != 0) return -1;
        const int q = splits >= 8 ? 1 : 8 / splits;
        blocks = splits >= 8 ? static_cast<long long>(splits) * tile_groups
                             : static_cast<long long>((tile_groups + q - 1) / q) * 8;
    }
    if (blocks > 0x7fffffffLL) return -1;
    const dim3 grid(static_cast<unsigned>(blocks));
#define LAUNCH_T(MT, NT, TO, T)                                                                                  \
    gemm_skinny_kernel<MT, NT, TO, T><<<grid, 256, smem, stream>>>(static_cast<const bf16*>(x), static_cast<const bf16*>(w), \
                                                                   static_cast<TO*>(out), partial, M, N, K, k_per_split, chunk, \
                                                                   row_groups, splits)
#define LAUNCH(MT, NT, TO)                  \
    if (tiled) LAUNCH_T(MT, NT, TO, true);  \
    else LAUNCH_T(MT, NT, TO, false)
#define BY_NT(MT, TO)                    \
    if (nt == 4) LAUNCH(MT, 4, TO);      \
    else if (nt == 2) LAUNCH(MT, 2, TO); \
    else LAUNCH(MT, 1, TO)
#define BY_MT(TO)                         \
    switch (mt) {                         \
        case 1: BY_NT(1, TO); break;      \
        case 2: BY_NT(2, TO); break;      \
        case 3: BY_NT(3, TO); break;      \
        default: BY_NT(4, TO); break;     \
    }
    if (out_bf16) { BY_MT(bf16) } else { BY_MT(float) }
#undef BY_MT
#undef BY_NT
#undef LAUNCH
#undef LAUNCH_T
    int err = launch_status();
    if (err) return err;
    if (splits > 1 && out != nullptr) {
        const long long total = static_cast<long long>(M) * N;
        const long long want = (total + 255) / 256;
        const int blocks = static_cast<int>(want < 4096 ? want : 4096);
        if (out_bf16) split_sum_kernel<bf16><<<blocks, 256, 0, stream>>>(partial, static_cast<bf16*>(out), total, splits);
        else split_sum_kernel<float><<<blocks, 256, 0, stream>>>(partial, static_cast<float*>(out), total, splits);
        err = launch_status();
    }
    return err;
}

// ---- gated feed-forward input: out[M, I] = act(x . Wg^T) * (x . Wu^T), w = [Wg; Wu] of 2I rows -----
// A wavefront streams 16 gate rows and the 16 up rows that belong to them; both results land
// in the same lanes, so the activation and the product are made in registers and only [M, I]
// is written.

// A workgroup is TPW tiles of 16 gate rows (with their up rows) times 2 halves of the K axis; the
// halves are added through shared memory in a fixed order before the activation.  A workgroup is 2
// tiles (4 wavefronts); with few rows of x (MT <= 2) the kernel needs few registers and four
// workgroups share a compute unit, 16 wavefronts with 16 loads each in flight, with three or four
// tiles of rows two workgroups do.  (Workgroups of 4 tiles, which stage x half as often, are slower
// at 48 and 64 rows, 34 against 30 and 38 against 35 us at the 2B sizes: a barrier then holds eight
// wavefronts to the slowest one's loads.)
//
// NORM (at most 16 rows, chunks of 256 keys): x is not given; the kernel reads the float32 residual
// stream and applies the RMS norm as it stages a chunk: x = residual * rsqrt(mean square + eps) *
// (offset + norm weight), rounded to bfloat16 as the norm kernel would round it.  A row's mean square
// comes from `sumsq` ([M, sumsq_cols], whose row sums are the rows' sums of squares: see
// `gemm_residual.hip`), so no kernel has to pass over the stream between the product that wrote it
// and this one.  XR is the number of 16-byte pieces of x a thread stages per chunk (rows beyond M are
// not staged: they only feed results that are not written).
struct NormOnLoad {
    const float* residual;      // [M, K]
    const float* sumsq;         // [M, sumsq_cols]
    const float* weight;        // [K]
    int sumsq_cols;
    float eps, offset;
};

template <int MT, int ACT, bool TILED, int TPW, bool NORM, int XR>
__global__ void __launch_bounds__(TPW * 128, MT == 1 ? (NORM && XR > 2 ? 3 : 4) : (MT == 2 ? 3 : 2))
gemm_skinny_gated_kernel(const bf16* __restrict__ x, NormOnLoad norm, const bf16* __restrict__ w, bf16* __restrict__ out,
                         int M, int inter, int K, int chunk) {
    extern __shared__ uint4 xs[];                 // two halves of [MT*16][chunk/8 + 1]
    __shared__ float inv_s[16];                   // NORM: a row's rsqrt(mean square + eps)
    const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
    const int i = lane % 16, g = lane / 16;
    const int tile = wave % TPW, half = wave / TPW;
    const int n0 = (blockIdx.x * TPW + tile) * 16;
    const int stride = chunk / 8 + 1;
    const int half_k = K / 2;                     // a multiple of 32
    const int k_begin = half * half_k;
    uint4* xh = xs + half * (MT * 16 * stride);
    // TILED: the gate rows' bands of 16 rows first, then the up rows' bands
    constexpr int kStep = TILED ? 512 : 32;
    const int nrow = min(n0 + i, inter - 1);
    const int bands = (inter + 15) / 16, band = min(n0 / 16, bands - 1);
    const bf16* gp = TILED ? w + (static_cast<size_t>(band) * (K / 32) + k_begin / 32) * 512 + lane * 8
                           : w + static_cast<size_t>(nrow) * K + k_begin + 8 * g;
    const bf16* up = TILED ? w + (static_cast<size_t>(bands + band) * (K / 32) + k_begin / 32) * 512 + lane * 8
                           : w + static_cast<size_t>(inter + nrow) * K + k_begin + 8 * g;
    float4_t accg[MT], accu[MT];
#pragma unroll
    for (int t = 0; t < MT; ++t) {
        accg[t] = float4_t{0.f, 0.f, 0.f, 0.f};
        accu[t] = float4_t{0.f, 0.f, 0.f, 0.f};
    }
    // The weight stream: kBatch 16-byte loads per lane and stream are in flight; a register is
    // refilled with the step kBatch further on as soon as its product has been issued, so the loads
    // in flight take 16 registers a stream and not twice that, and two workgroups fit a compute unit.
    constexpr int kBatch = 8;       // per stream; two streams
    const bool live = n0 < inter;
    const int steps = half_k / 32;
    Frag curg[kBatch], curu[kBatch];
    auto load_step = [&](int u, int at) {
        const bool ok = live && at < steps;
        curg[u].u = ok ? load_streamed(gp + at * kStep) : make_uint4(0, 0, 0, 0);
        curu[u].u = ok ? load_streamed(up + at * kStep) : make_uint4(0, 0, 0, 0);
    };
#pragma unroll
    for (int u = 0; u < kBatch; ++u) load_step(u, u);
    int step = 0;
    constexpr int kHalfThreads = TPW * 64;        // the threads that stage one half's x
    const int tid_half = threadIdx.x % kHalfThreads;
    if (NORM) {
        // 16 threads a row add the row of `sumsq` in a fixed order
        const int t = threadIdx.x;
        if (t < 256) {
            const int r = t / 16, part = t % 16;
            float total = 0.f;
            if (r < M)
                for (int b = part; b < norm.sumsq_cols; b += 16) total += norm.sumsq[static_cast<size_t>(r) * norm.sumsq_cols + b];
            total += __shfl_xor(total, 8, kWave);
            total += __shfl_xor(total, 4, kWave);
            total += __shfl_xor(total, 2, kWave);
            total += __shfl_xor(total, 1, kWave);
            if (part == 0) inv_s[r] = rsqrtf(total / static_cast<float>(K) + norm.eps);
        }
    }
    // x is staged chunk by chunk (per half of K); the next chunk's loads are in flight during the products
    constexpr int kXRegs = NORM ? XR : (MT == 1 ? 4 : (MT >= 3 && TPW == 2 ? 16 : 8));       // pieces of a chunk per thread
    uint4 xreg[NORM ? 1 : kXRegs];
    float4 xraw[NORM ? kXRegs : 1][2], wraw[2];
    // a thread's pieces of a chunk as (row, 8 keys) pairs of the whole chunk's shape, worked out once: a
    // division by a run-time number per piece and chunk would cost more than the products
    int x_col[NORM ? 1 : kXRegs], x_row[NORM ? 1 : kXRegs];
    if (!NORM) {
        const int vecs_full = chunk / 8;
        const int dq = kHalfThreads / vecs_full, dr = kHalfThreads % vecs_full;
        int m = tid_half / vecs_full, c = tid_half % vecs_full;
#pragma unroll
        for (int u = 0; u < (NORM ? 1 : kXRegs); ++u) {
            x_row[u] = m < MT * 16 ? m : -1;
            x_col[u] = c;
            m += dq;
            c += dr;
            if (c >= vecs_full) { c -= vecs_full; ++m; }
        }
    }
    auto fetch_x = [&](int kc) {
        if (NORM) {
            // chunks of 256 keys: a thread's pieces are rows tid_half / 32 + (kHalfThreads / 32) * u at the
            // same 8 keys, so it needs 8 norm weights a chunk
            const int c = tid_half % 32;
            const float* wsrc = norm.weight + k_begin + kc + c * 8;
            wraw[0] = *reinterpret_cast<const float4*>(wsrc);
            wraw[1] = *reinterpret_cast<const float4*>(wsrc + 4);
#pragma unroll
            for (int u = 0; u < kXRegs; ++u) {
                const int m = tid_half / 32 + (kHalfThreads / 32) * u;
                const float* src = norm.residual + static_cast<size_t>(min(m, M - 1)) * K + k_begin + kc + c * 8;
                xraw[u][0] = *reinterpret_cast<const float4*>(src);
                xraw[u][1] = *reinterpret_cast<const float4*>(src + 4);
            }
            return;
        }
        const int vecs = min(chunk, half_k - kc) / 8;
#pragma unroll
        for (int u = 0; u < (NORM ? 1 : kXRegs); ++u) {
            const int m = x_row[u], c = x_col[u];
            xreg[u] = (m >= 0 && m < M && c < vecs)
                          ? *reinterpret_cast<const uint4*>(x + static_cast<size_t>(m) * K + k_begin + kc + c * 8)
                          : make_uint4(0, 0, 0, 0);
        }
    };
    auto stage_x = [&](int vecs) {
        if (NORM) {
            const int c = tid_half % 32;
#pragma unroll
            for (int u = 0; u < kXRegs; ++u) {
                const int m = tid_half / 32 + (kHalfThreads / 32) * u;
                if (m >= 16) continue;
                const float inv = inv_s[m];
                const float4 a = xraw[u][0], b = xraw[u][1];
                uint4 v;
                v.x = pack2_bf16(a.x * inv * (norm.offset + wraw[0].x), a.y * inv * (norm.offset + wraw[0].y));
                v.y = pack2_bf16(a.z * inv * (norm.offset + wraw[0].z), a.w * inv * (norm.offset + wraw[0].w));
                v.z = pack2_bf16(b.x * inv * (norm.offset + wraw[1].x), b.y * inv * (norm.offset + wraw[1].y));
                v.w = pack2_bf16(b.z * inv * (norm.offset + wraw[1].z), b.w * inv * (norm.offset + wraw[1].w));
                xh[m * stride + c] = v;
            }
            return;
        }
#pragma unroll
        for (int u = 0; u < (NORM ? 1 : kXRegs); ++u)
            if (x_row[u] >= 0 && x_col[u] < vecs) xh[x_row[u] * stride + x_col[u]] = xreg[u];
    };
    fetch_x(0);
    for (int kc = 0; kc < half_k; kc += chunk) {
        const int len = min(chunk, half_k - kc);      // a multiple of 32 * kBatch, except the last
        __syncthreads();
        stage_x(len / 8);
        __syncthreads();
        if (kc + chunk < half_k) fetch_x(kc + chunk);
        for (int k = 0; k < len; k += 32 * kBatch) {
#pragma unroll
            for (int u = 0; u < kBatch; ++u) {
                if (k + 32 * u < len) {
#pragma unroll
                    for (int t = 0; t < MT; ++t) {
                        Frag b;
                        b.u = xh[(t * 16 + i) * stride + k / 8 + 4 * u + g];
                        accg[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(curg[u].v, b.v, accg[t], 0, 0, 0);
                        accu[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(curu[u].v, b.v, accu[t], 0, 0, 0);
                    }
                    load_step(u, step + u + kBatch);
                }
            }
            step += kBatch;
        }
    }
    // the second half hands its sums to the first through shared memory
    __syncthreads();
    float* red = reinterpret_cast<float*>(xs) + (tile * kWave + lane) * (MT * 8);
    if (half == 1) {
#pragma unroll
        for (int t = 0; t < MT; ++t)
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                red[t * 8 + v] = accg[t][v];
                red[t * 8 + 4 + v] = accu[t][v];
            }
    }
    __syncthreads();
    if (half == 1 || n0 >= inter) return;
    const int n = n0 + 4 * g;
#pragma unroll
    for (int t = 0; t < MT; ++t) {
        const int m = t * 16 + i;
        if (m >= M) continue;
        float4_t r;
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            const float gate = accg[t][v] + red[t * 8 + v], upv = accu[t][v] + red[t * 8 + 4 + v];
            r[v] = activate<ACT>(gate) * upv;
        }
        bf16* o = out + static_cast<size_t>(m) * inter + n;
        if (n + 3 < inter && (inter % 4 == 0)) {
            store4<bf16>(o, r);
        } else {
#pragma unroll
            for (int v = 0; v < 4; ++v)
                if (n + v < inter) o[v] = from_float<bf16>(r[v]);
        }
    }
}

static int gated_launch(const void* x, NormOnLoad norm, bool with_norm, const void* w, int tiled, void* out, int M,
                        int inter, int K, int activation, int chunk, hipStream_t stream) {
    if (M < 1 || M > 64 || K % 64 != 0 || chunk % 32 != 0 || activation < 0 || activation >= kActivations) return -1;
    const int mt = (M + 15) / 16;
    if (chunk > K / 2) chunk = K / 2;
    // the norm on load: at most 16 rows, whole chunks of 256 keys
    if (with_norm && (mt != 1 || chunk != 256 || (K / 2) % 256 != 0)) return -1;
    const int tpw = 2;                               // tiles of 16 gate rows per workgroup
    size_t smem = static_cast<size_t>(2) * mt * 16 * (chunk / 8 + 1) * sizeof(uint4);
    const size_t red = static_cast<size_t>(tpw) * kWave * mt * 8 * sizeof(float);
    if (red > smem) smem = red;
    // the pieces of x a thread stages (4 up to 16 rows, else 8); a chunk that is not the last must be
    // whole batches of 8 steps, because a register's step is fixed by its place
    const int x_regs = mt == 1 ? 4 : (mt >= 3 && tpw == 2 ? 16 : 8);
    if (smem > 160 * 1024 - 4096 || mt * 16 * (chunk / 8) > tpw * 64 * x_regs || (chunk % 256 != 0 && chunk < K / 2))
        return -1;
    const dim3 grid((inter + 16 * tpw - 1) / (16 * tpw));
#define LAUNCH_K(MT, A, T, TPW, NORM, XR)                                                                            \
    do {                                                                                                              \
        static bool roomy = false;     /* more than 64 KiB of shared memory must be asked for once */                \
        if (smem > 65536 && !roomy) {                                                                                 \
            if (hipFuncSetAttribute(reinterpret_cast<const void*>(&gemm_skinny_gated_kernel<MT, A, T, TPW, NORM, XR>), \
                                    hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024 - 4096) != hipSuccess)    \
                return launch_status();                                                                               \
            roomy = true;                                                                                             \
        }                                                                                                             \
        gemm_skinny_gated_kernel<MT, A, T, TPW, NORM, XR><<<grid, TPW * 128, smem, stream>>>(                        \
            static_cast<const bf16*>(x), norm, static_cast<const bf16*>(w), static_cast<bf16*>(out), M, inter, K, chunk); \
    } while (0)
#define LAUNCH_T(MT, A, T, TPW) LAUNCH_K(MT, A, T, TPW, false, 4)
#define LAUNCH(MT, A)                        \
    if (tiled) LAUNCH_T(MT, A, true, 2);      \
    else LAUNCH_T(MT, A, false, 2)
#define LAUNCH_N(A)                                           \
    if (tiled) {                                              \
        if (M <= 8) LAUNCH_K(1, A, true, 2, true, 2);         \
        else LAUNCH_K(1, A, true, 2, true, 4);                \
    } else {                                                  \
        if (M <= 8) LAUNCH_K(1, A, false, 2, true, 2);        \
        else LAUNCH_K(1, A, false, 2, true, 4);               \
    }
#define BY_MT(A)                     \
    switch (mt) {                    \
        case 1: LAUNCH(1, A); break; \
        case 2: LAUNCH(2, A); break; \
        case 3: LAUNCH(3, A); break; \
        default: LAUNCH(4, A); break; \
    }
    if (with_norm) {
        WLLM_BY_ACTIVATION(activation, LAUNCH_N(ACT))
    } else {
        WLLM_BY_ACTIVATION(activation, BY_MT(ACT))
    }
#undef BY_MT
#undef LAUNCH_N
#undef LAUNCH
#undef LAUNCH_T
#undef LAUNCH_K
    return launch_status();
}

WLLM_API int wllm_gemm_skinny_gated(const void* x, const void* w, int tiled, void* out, int M, int inter, int K,
                                    int activation, int chunk, hipStream_t stream) {
    return gated_launch(x, NormOnLoad{nullptr, nullptr, nullptr, 0, 0.f, 0.f}, false, w, tiled, out, M, inter, K, activation,
                        chunk, stream);
}

// The same product with the RMS norm of the residual stream folded into the load of x: at most 16
// rows, K a multiple of 512.  sumsq float32 [M, sumsq_cols]: a row's entries add up to the sum of
// squares of the row of `residual`.  Returns -1 for sizes it does not take.
WLLM_API int wllm_gemm_skinny_gated_norm(const float* residual, const float* sumsq, int sumsq_cols, const float* norm_weight,
                                         float eps, float offset, const void* w, int tiled, void* out, int M, int inter,
                                         int K, int activation, hipStream_t stream) {
    if (M > 16 || sumsq_cols < 1) return -1;
    return gated_launch(nullptr, NormOnLoad{residual, sumsq, norm_weight, sumsq_cols, eps, offset}, true, w, tiled, out, M,
                        inter, K, activation, 256, stream);
}
