// out[M, N] = x[M, K] * w[N, K]^T for float32 and bfloat16 operands, accumulated in float32.  It is
// the product of the float32 path, and the product of last resort for bfloat16 (shapes the
// bfloat16 matrix-core kernels do not take, float32 results from bfloat16 operands).  No
// reduced-precision mode is involved anywhere: float32 operands are multiplied and added as float32,
// on the matrix cores' float32 instruction where the K axis is a multiple of 4 (below), with fused
// multiply-adds on the vector units otherwise (this kernel).
//
// A workgroup of 256 threads makes a 64x64 tile of the result; the K axis is walked in steps of
// 16 through shared memory; a thread holds a 4x4 block.  The K axis is cut into segments of kSegment
// keys counted from 0, a segment is summed over k in ascending order of fused multiply-adds from
// zero, and the segments' sums are added in ascending order: an order fixed by K alone, so a row's
// result does not depend on the other rows of the batch.
#include "common.h"

constexpr int kTile = 64;
constexpr int kStep = 16;
constexpr int kSegment = 2048;

template <typename TI, typename TO>
__global__ void __launch_bounds__(256)
gemm_nt_kernel(const TI* __restrict__ x, const TI* __restrict__ w, TO* __restrict__ out, int M, int N, int K) {
    __shared__ float xs[kStep][kTile + 4];
    __shared__ float ws[kStep][kTile + 4];
    const int tid = threadIdx.x;
    const int row0 = blockIdx.y * kTile, col0 = blockIdx.x * kTile;
    const int tr = (tid / 16) * 4, tc = (tid % 16) * 4;
    float acc[4][4], total[4][4];
    // each thread stages 4 elements of x and 4 of w per step: row = tid / 4, k = (tid % 4) * 4 ..
    const int lr = tid / 4, lk = (tid % 4) * 4;
    for (int seg0 = 0; seg0 < K; seg0 += kSegment) {
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;
    for (int k0 = seg0; k0 < min(K, seg0 + kSegment); k0 += kStep) {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int k = k0 + lk + e;
            const int xr = row0 + lr, wr = col0 + lr;
            xs[lk + e][lr] = (xr < M && k < K) ? to_float(x[static_cast<size_t>(xr) * K + k]) : 0.f;
            ws[lk + e][lr] = (wr < N && k < K) ? to_float(w[static_cast<size_t>(wr) * K + k]) : 0.f;
        }
        __syncthreads();
#pragma unroll
        for (int k = 0; k < kStep; ++k) {
            float a[4], b[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) a[i] = xs[k][tr + i];
#pragma unroll
            for (int j = 0; j < 4; ++j) b[j] = ws[k][tc + j];
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
        }
        __syncthreads();
    }
    // the segment's sum joins the sums of the segments before it
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) total[i][j] = seg0 == 0 ? acc[i][j] : total[i][j] + acc[i][j];
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int r = row0 + tr + i;
        if (r >= M) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int c = col0 + tc + j;
            if (c < N) out[static_cast<size_t>(r) * N + c] = from_float<TO>(total[i][j]);
        }
    }
}

// ---- float32 on the matrix cores ----------------------------------------------------------------
// v_mfma_f32_16x16x4_f32 multiplies and accumulates IEEE float32 (no narrower format is involved), at
// twice the rate that unpacked vector multiply-adds reach.  Both kernels below make an element of the
// result by the same instructions on the same numbers in the same order, whatever the rows and columns
// beside it, so a token's projection has the same bits in a decode step as inside a prompt:
//   the K axis is cut into segments of kF32Segment keys counted from 0; within a segment the keys go
//   in chunks of 16; a chunk is four instructions, the t-th of which takes the keys 16 q + 4 g + t
//   (g = 0..3, the lane's group) and accumulates into the segment's sum, which starts at zero; the
//   segments' sums are added in ascending order.
// A lane (i, g) of a wavefront holds, of a chunk, w[n0 + i][16 q + 4 g .. + 3] and x[m0 + i][the same
// keys]: one 16-byte load each, whose t-th element goes to the t-th instruction.  The first operand is
// w, so a lane's four results are four consecutive columns of one row of out.
typedef float f32x4 __attribute__((ext_vector_type(4)));
constexpr int kF32Segment = 512;
constexpr int kF32Chunk = 16;

__device__ __forceinline__ f32x4 mfma_chunk(const f32x4 a, const f32x4 b, f32x4 acc) {
    acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a[0], b[0], acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a[1], b[1], acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a[2], b[2], acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a[3], b[3], acc, 0, 0, 0);
    return acc;
}

// At most 64 rows (the decode steps of the float32 path): the weights stream from memory straight
// into the lanes that multiply them, a wavefront a band of 16 columns, `U` chunks of it in flight at a
// time; x comes through the caches (all wavefronts read the same few rows).  MT tiles of 16 rows: a
// fragment of the weights feeds MT products, each row's sums in the one order (the tiled kernel below
// took 300 us for the gate and up projections of 64 rows at the 2B sizes, this one streams them).  SPLIT: a wavefront takes
// one segment of the K axis (blockIdx.y) and leaves its sum in partial[segment]; a second kernel adds
// the segments in ascending order.  Otherwise it walks all segments and adds as it goes.
// TILED: w is the weight's tile-major copy (`tile_weight_f32_kernel`): per band of 16 rows and chunk
// of 16 keys one KiB in lane order, so that a wavefront's load is one contiguous KiB and its walk along
// K one contiguous run (gate and up at Gemma-2B sizes: 76 us from the row-major weight, whose loads
// touch 16 rows of 64 bytes each, 49 us from the copy).
template <bool SPLIT, bool TILED, int MT>
__global__ void __launch_bounds__(256)
gemm_f32_few_rows_kernel(const float* __restrict__ x, const float* __restrict__ w, float* __restrict__ out, int M, int N,
                         int K) {
    constexpr int U = MT <= 2 ? 8 : 4;
    const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
    const int i = lane % 16, g = lane / 16;
    const int n0 = (blockIdx.x * 4 + wave) * 16;
    if (n0 >= N) return;
    const int chunks_of_row = (K + kF32Chunk - 1) / kF32Chunk;
    const float* wrow = TILED ? w + (static_cast<size_t>(n0 / 16) * chunks_of_row * 64 + lane) * 4
                              : w + static_cast<size_t>(min(n0 + i, N - 1)) * K;
    const float* xrow[MT];
    bool x_live[MT];
#pragma unroll
    for (int t = 0; t < MT; ++t) {
        xrow[t] = x + static_cast<size_t>(min(16 * t + i, M - 1)) * K;
        x_live[t] = 16 * t + i < M;
    }
    const int segments = (K + kF32Segment - 1) / kF32Segment;
    const int seg_first = SPLIT ? blockIdx.y : 0, seg_end = SPLIT ? blockIdx.y + 1 : segments;
    f32x4 total[MT];
#pragma unroll
    for (int t = 0; t < MT; ++t) total[t] = f32x4{0.f, 0.f, 0.f, 0.f};
    for (int seg = seg_first; seg < seg_end; ++seg) {
        const int k_begin = seg * kF32Segment, k_end = min(K, k_begin + kF32Segment);
        f32x4 acc[MT];
#pragma unroll
        for (int t = 0; t < MT; ++t) acc[t] = f32x4{0.f, 0.f, 0.f, 0.f};
        for (int k0 = k_begin; k0 < k_end; k0 += U * kF32Chunk) {
            f32x4 a[U], b[MT][U];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                // every lane loads, from a clamped address; what lies beyond the segment becomes zero
                const int k = k0 + u * kF32Chunk + 4 * g;
                // (a chunk beyond the row's last is clamped to the last: what it holds becomes zero below)
                a[u] = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(
                    TILED ? wrow + static_cast<size_t>(min(k0 / kF32Chunk + u, chunks_of_row - 1)) * 256 : wrow + min(k, K - 4)));
#pragma unroll
                for (int t = 0; t < MT; ++t) b[t][u] = *reinterpret_cast<const f32x4*>(xrow[t] + min(k, K - 4));
            }
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int k = k0 + u * kF32Chunk + 4 * g;
                const bool live = k < k_end;
                const f32x4 zero = f32x4{0.f, 0.f, 0.f, 0.f};
                const f32x4 av = live ? a[u] : zero;
                if (k0 + u * kF32Chunk < k_end) {     // the same for all lanes
#pragma unroll
                    for (int t = 0; t < MT; ++t) acc[t] = mfma_chunk(av, live && x_live[t] ? b[t][u] : zero, acc[t]);
                }
            }
        }
#pragma unroll
        for (int t = 0; t < MT; ++t) total[t] = seg == seg_first ? acc[t] : total[t] + acc[t];
    }
    // lane (i, g) holds out[row 16 t + i][n0 + 4 g .. + 3]
#pragma unroll
    for (int t = 0; t < MT; ++t) {
        if (!x_live[t]) continue;
        float* dst = out + (SPLIT ? static_cast<size_t>(blockIdx.y) * M * N : 0) + static_cast<size_t>(16 * t + i) * N + n0 + 4 * g;
        if (N % 4 == 0 && n0 + 4 * g + 3 < N) {
            *reinterpret_cast<f32x4*>(dst) = total[t];
        } else {
#pragma unroll
            for (int v = 0; v < 4; ++v)
                if (n0 + 4 * g + v < N) dst[v] = total[t][v];
        }
    }
}

// More rows: a workgroup of four wavefronts (2 x 2) makes 32 WM rows by 32 WN columns; the tiles of
// x and w of a chunk go through shared memory, the next chunk's loads in flight while this one is
// multiplied.  Rows of a tile are padded to 20 floats, so that the 16-byte fragment reads of 8 lanes
// fall into different banks.
template <int WM, int WN>
__global__ void __launch_bounds__(256, 2)
gemm_f32_tile_kernel(const float* __restrict__ x, const float* __restrict__ w, float* __restrict__ out, int M, int N, int K) {
    constexpr int TM = 32 * WM, TN = 32 * WN, kStride = kF32Chunk + 4;
    constexpr int XP = TM * 4 / 256, WP = TN * 4 / 256;       // 16-byte pieces of a chunk's tiles per thread
    static_assert(XP * 256 == TM * 4 && WP * 256 == TN * 4, "whole pieces per thread");
    __shared__ __align__(16) float xs[2][TM * kStride];
    __shared__ __align__(16) float ws[2][TN * kStride];
    const int tid = threadIdx.x, lane = tid % kWave, wave = tid / kWave;
    const int i = lane % 16, g = lane / 16;
    const int m0 = blockIdx.y * TM, n0 = blockIdx.x * TN;
    const int wm0 = (wave / 2) * (TM / 2), wn0 = (wave % 2) * (TN / 2);
    // a thread's pieces: row tid / 4 (+ 64 per further piece), keys 4 (tid % 4) ..
    const int p_row = tid / 4, p_k = (tid % 4) * 4;
    const float* xsrc[XP];
    const float* wsrc[WP];
#pragma unroll
    for (int p = 0; p < XP; ++p) xsrc[p] = x + static_cast<size_t>(min(m0 + p_row + 64 * p, M - 1)) * K;
#pragma unroll
    for (int p = 0; p < WP; ++p) wsrc[p] = w + static_cast<size_t>(min(n0 + p_row + 64 * p, N - 1)) * K;
    // two sets of registers for chunks on their way: a chunk is asked for two chunks before it is
    // multiplied, so a trip to memory has two chunks' products to hide behind
    f32x4 xr[2][XP], wr[2][WP];
    auto fetch = [&](f32x4 (&xq)[XP], f32x4 (&wq)[WP], int k0) {
        const int k = k0 + p_k;
        const bool live = k < K;
        const f32x4 zero = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int p = 0; p < XP; ++p) {
            const f32x4 v = *reinterpret_cast<const f32x4*>(xsrc[p] + min(k, K - 4));
            xq[p] = live ? v : zero;
        }
#pragma unroll
        for (int p = 0; p < WP; ++p) {
            const f32x4 v = *reinterpret_cast<const f32x4*>(wsrc[p] + min(k, K - 4));
            wq[p] = live ? v : zero;
        }
    };
    auto stage = [&](int buf, const f32x4 (&xq)[XP], const f32x4 (&wq)[WP]) {
#pragma unroll
        for (int p = 0; p < XP; ++p) *reinterpret_cast<f32x4*>(&xs[buf][(p_row + 64 * p) * kStride + p_k]) = xq[p];
#pragma unroll
        for (int p = 0; p < WP; ++p) *reinterpret_cast<f32x4*>(&ws[buf][(p_row + 64 * p) * kStride + p_k]) = wq[p];
    };
    f32x4 acc[WM][WN], total[WM][WN];
#pragma unroll
    for (int jm = 0; jm < WM; ++jm)
#pragma unroll
        for (int jn = 0; jn < WN; ++jn) acc[jm][jn] = total[jm][jn] = f32x4{0.f, 0.f, 0.f, 0.f};
    const int chunks = (K + kF32Chunk - 1) / kF32Chunk;
    constexpr int kChunksPerSegment = kF32Segment / kF32Chunk;
    // chunk q: multiplied from tile q % 2 of shared memory; chunk q + 1 waits in the registers (q + 1) % 2
    // and goes to the other tile when the products of chunk q are issued; chunk q + 2 is asked for
    auto step = [&](int q, int buf, f32x4 (&x_next)[XP], f32x4 (&w_next)[WP], f32x4 (&x_ask)[XP], f32x4 (&w_ask)[WP]) {
        if (q + 2 < chunks) fetch(x_ask, w_ask, (q + 2) * kF32Chunk);
        f32x4 a[WN], b[WM];
#pragma unroll
        for (int jn = 0; jn < WN; ++jn) a[jn] = *reinterpret_cast<const f32x4*>(&ws[buf][(wn0 + 16 * jn + i) * kStride + 4 * g]);
#pragma unroll
        for (int jm = 0; jm < WM; ++jm) b[jm] = *reinterpret_cast<const f32x4*>(&xs[buf][(wm0 + 16 * jm + i) * kStride + 4 * g]);
#pragma unroll
        for (int t = 0; t < 4; ++t)
#pragma unroll
            for (int jm = 0; jm < WM; ++jm)
#pragma unroll
                for (int jn = 0; jn < WN; ++jn)
                    acc[jm][jn] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[jn][t], b[jm][t], acc[jm][jn], 0, 0, 0);
        if ((q + 1) % kChunksPerSegment == 0 || q + 1 == chunks) {
            // a segment ends: its sum joins the sums of the segments before it
            const bool first = q < kChunksPerSegment;
#pragma unroll
            for (int jm = 0; jm < WM; ++jm)
#pragma unroll
                for (int jn = 0; jn < WN; ++jn) {
                    total[jm][jn] = first ? acc[jm][jn] : total[jm][jn] + acc[jm][jn];
                    acc[jm][jn] = f32x4{0.f, 0.f, 0.f, 0.f};
                }
        }
        if (q + 1 < chunks) stage(buf ^ 1, x_next, w_next);
        __syncthreads();
    };
    fetch(xr[0], wr[0], 0);
    stage(0, xr[0], wr[0]);
    if (chunks > 1) fetch(xr[1], wr[1], kF32Chunk);
    __syncthreads();
    for (int q = 0; q < chunks; q += 2) {
        step(q, 0, xr[1], wr[1], xr[0], wr[0]);
        if (q + 1 < chunks) step(q + 1, 1, xr[0], wr[0], xr[1], wr[1]);
    }
#pragma unroll
    for (int jm = 0; jm < WM; ++jm) {
        const int m = m0 + wm0 + 16 * jm + i;
        if (m >= M) continue;
#pragma unroll
        for (int jn = 0; jn < WN; ++jn) {
            const int n = n0 + wn0 + 16 * jn + 4 * g;
            float* dst = out + static_cast<size_t>(m) * N + n;
            if (N % 4 == 0 && n + 3 < N) {
                *reinterpret_cast<f32x4*>(dst) = total[jm][jn];
            } else {
#pragma unroll
                for (int v = 0; v < 4; ++v)
                    if (n + v < N) dst[v] = total[jm][jn][v];
            }
        }
    }
}

// out[i] = partial[0][i] + partial[1][i] + ... in ascending order of the segments.
__global__ void __launch_bounds__(256)
gemm_segments_sum_kernel(const float* __restrict__ partial, float* __restrict__ out, int count, int segments) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= count) return;
    float total = partial[i];
    for (int s = 1; s < segments; ++s) total = total + partial[static_cast<size_t>(s) * count + i];
    out[i] = total;
}

namespace {
// Whether the few-row kernel gives every segment of the K axis a wavefront of its own: where the bands
// of 16 columns alone are too few wavefronts to keep the memory busy.
bool few_rows_split(int N, int K) { return K > kF32Segment && (N + 15) / 16 < 1024; }
bool f32_by_matrix_cores(int in_bf16, int out_bf16, int K) { return !in_bf16 && !out_bf16 && K % 4 == 0 && K >= 4; }
}  // namespace

// The tile-major copy of a float32 weight [N, K] (K a multiple of 4): for band b of 16 rows and chunk q
// of 16 keys, lane 16 g + i finds w[16 b + i][16 q + 4 g .. + 3] at ((b * chunks + q) * 64 + lane) * 4;
// rows beyond N and keys beyond K are zeros.
__global__ void __launch_bounds__(256)
tile_weight_f32_kernel(const float* __restrict__ w, float* __restrict__ tiles, int N, int K, int chunks, long long pieces) {
    const long long piece = static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (piece >= pieces) return;
    const int lane = piece % 64, i = lane % 16, g = lane / 16;
    const long long tile = piece / 64;
    const int q = tile % chunks;
    const long long row = tile / chunks * 16 + i;
    const int k = 16 * q + 4 * g;
    f32x4 v = f32x4{0.f, 0.f, 0.f, 0.f};
    if (row < N && k < K) v = *reinterpret_cast<const f32x4*>(w + row * K + k);
    *reinterpret_cast<f32x4*>(tiles + piece * 4) = v;
}

// Elements of the tile-major copy of a float32 weight [N, K].
WLLM_API long long wllm_tiled_size_f32(int N, int K) {
    return static_cast<long long>((N + 15) / 16) * 16 * ((K + kF32Chunk - 1) / kF32Chunk) * kF32Chunk;
}

WLLM_API int wllm_tile_weight_f32(const float* w, float* tiles, int N, int K, hipStream_t stream) {
    if (N < 1 || K < 4 || K % 4 != 0) return -1;
    const int chunks = (K + kF32Chunk - 1) / kF32Chunk;
    const long long pieces = static_cast<long long>((N + 15) / 16) * chunks * 64;
    const long long blocks = (pieces + 255) / 256;
    if (blocks > 0x7fffffffLL) return -1;
    tile_weight_f32_kernel<<<static_cast<unsigned>(blocks), 256, 0, stream>>>(w, tiles, N, K, chunks, pieces);
    return launch_status();
}

// Into how many partial sums [segments, M, N] a float32 product of these sizes is split (1: it is not).
// `wllm_gemm_generic` needs `partial` to hold them; with `out` null it leaves them there for a consumer
// that adds them in ascending order.
WLLM_API int wllm_gemm_f32_segments(int M, int N, int K) {
    if (M < 1 || M > 64 || K % 4 != 0 || !few_rows_split(N, K)) return 1;
    return (K + kF32Segment - 1) / kF32Segment;
}

// `tiles`: null, or the tile-major copy of a float32 w (`wllm_tile_weight_f32`), which the few-row kernel
// streams faster; everything else reads w.
WLLM_API int wllm_gemm_generic(const void* x, const void* w, const void* tiles, int in_bf16, void* out, int out_bf16,
                               void* partial, int M, int N, int K, hipStream_t stream) {
    if (M < 1 || N < 1 || K < 1) return -1;
    if (f32_by_matrix_cores(in_bf16, out_bf16, K)) {
        const float* xf = static_cast<const float*>(x);
        const float* wf = static_cast<const float*>(w);
        const float* tf = static_cast<const float*>(tiles);
        float* of = static_cast<float*>(out);
        if (M <= 64) {
            const int bands = (N + 15) / 16, groups = (bands + 3) / 4;
            const int mt = (M + 15) / 16;
#define FEW_ROWS(SPLIT, GRID, DST)                                                                                      \
    do {                                                                                                                \
        if (tf) {                                                                                                       \
            if (mt == 1) gemm_f32_few_rows_kernel<SPLIT, true, 1><<<GRID, 256, 0, stream>>>(xf, tf, DST, M, N, K);       \
            else if (mt == 2) gemm_f32_few_rows_kernel<SPLIT, true, 2><<<GRID, 256, 0, stream>>>(xf, tf, DST, M, N, K);  \
            else if (mt == 3) gemm_f32_few_rows_kernel<SPLIT, true, 3><<<GRID, 256, 0, stream>>>(xf, tf, DST, M, N, K);  \
            else gemm_f32_few_rows_kernel<SPLIT, true, 4><<<GRID, 256, 0, stream>>>(xf, tf, DST, M, N, K);               \
        } else {                                                                                                        \
            if (mt == 1) gemm_f32_few_rows_kernel<SPLIT, false, 1><<<GRID, 256, 0, stream>>>(xf, wf, DST, M, N, K);      \
            else if (mt == 2) gemm_f32_few_rows_kernel<SPLIT, false, 2><<<GRID, 256, 0, stream>>>(xf, wf, DST, M, N, K); \
            else if (mt == 3) gemm_f32_few_rows_kernel<SPLIT, false, 3><<<GRID, 256, 0, stream>>>(xf, wf, DST, M, N, K); \
            else gemm_f32_few_rows_kernel<SPLIT, false, 4><<<GRID, 256, 0, stream>>>(xf, wf, DST, M, N, K);              \
        }                                                                                                               \
    } while (0)
            if (few_rows_split(N, K)) {
                const int segments = (K + kF32Segment - 1) / kF32Segment;
                if (!partial || segments > 65535) return -1;
                float* pf = static_cast<float*>(partial);
                FEW_ROWS(true, dim3(groups, segments), pf);
                if (int err = launch_status()) return err;
                if (of) gemm_segments_sum_kernel<<<(M * N + 255) / 256, 256, 0, stream>>>(pf, of, M * N, segments);
            } else {
                if (!of) return -1;
                FEW_ROWS(false, dim3(groups), of);
            }
#undef FEW_ROWS
            return launch_status();
        }
        if (!of) return -1;
        // tiles of 128 x 128 where they fill the machine, smaller ones where a product has few columns or rows
        const long long rows128 = (M + 127) / 128, cols128 = (N + 127) / 128, cols64 = (N + 63) / 64;
        if (rows128 > 65535 || (M + 63) / 64 > 65535) return -1;
        if (rows128 * cols128 >= 384) {
            gemm_f32_tile_kernel<4, 4><<<dim3(cols128, rows128), 256, 0, stream>>>(xf, wf, of, M, N, K);
        } else if (rows128 * cols64 >= 384) {
            gemm_f32_tile_kernel<4, 2><<<dim3(cols64, rows128), 256, 0, stream>>>(xf, wf, of, M, N, K);
        } else {
            gemm_f32_tile_kernel<2, 2><<<dim3(cols64, (M + 63) / 64), 256, 0, stream>>>(xf, wf, of, M, N, K);
        }
        return launch_status();
    }
    const dim3 grid((N + kTile - 1) / kTile, (M + kTile - 1) / kTile);
    if (grid.y > 65535) return -1;
#define LAUNCH(TI, TO)                                                                                  \
    gemm_nt_kernel<TI, TO><<<grid, 256, 0, stream>>>(static_cast<const TI*>(x), static_cast<const TI*>(w), \
                                                     static_cast<TO*>(out), M, N, K)
    if (in_bf16 && out_bf16) LAUNCH(bf16, bf16);
    else if (in_bf16) LAUNCH(bf16, float);
    else if (!out_bf16) LAUNCH(float, float);
    else return -1;
#undef LAUNCH
    return launch_status();
}
