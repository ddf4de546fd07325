// out[M, N] = x[M, K] * w[N, K]^T for float32 and bfloat16 operands, accumulated in float32 with
// fused multiply-adds on the vector units.  No matrix-core instruction and no reduced-precision
// mode is involved, so with float32 operands this is a true 32-bit product; it is the product
// of the float32 path, and the product of last resort for bfloat16 (shapes the matrix-core
// kernels do not take, float32 results from bfloat16 operands).
//
// A workgroup of 256 threads makes a 64x64 tile of the result; the K axis is walked in steps of
// 16 through shared memory; a thread holds a 4x4 block.
//
// The order of an element's sum is fixed by K alone: the K axis is cut into segments of kSegment
// keys counted from 0, a segment is summed over k in ascending order of fused multiply-adds from
// zero, and the segments' sums are added in ascending order.  Every kernel in this file sums in
// that order, whatever the shape of the batch, so a row's result does not depend on the other rows
// and a token's projection has the same bits in a decode step as inside a prompt.  (With one
// segment, K <= kSegment, that is the plain ascending sum.)  The segments are what lets the
// few-row kernel below spread a long K axis over many workgroups.
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

// The same product for at most 16 rows of float32 (the decode steps of the float32 path).  The big
// tile would leave all but N/64 workgroups idle and seven eighths of each tile empty; here a
// workgroup makes ROWS rows x COLS columns, a thread one element, and the K axis is walked in chunks
// through shared memory.  An element is still the sum over k in ascending order of fused
// multiply-adds from zero within a segment of the K axis, so it has the same bits as the kernel above
// gives it.  A workgroup takes one segment (blockIdx.y); with several segments their sums go to a
// buffer of partial sums [segments, M, N] and a second kernel adds them in ascending order.
//
// What bounds it is how fast shared memory hands out operands (every product needs two), so the
// tile is chosen for as many compute units as possible to share that work: 16 x 16 where there are
// many columns; 8 columns, and 8 rows if the step has no more, for a projection back to the model's
// width, whose N / 16 workgroups would be fewer than compute units.  There the chunks of the next
// STAGES steps are on their way into registers while a chunk is summed: a trip to memory takes
// microseconds, the sums of a chunk a fraction of one, and no other workgroup is there to hide it.
constexpr int kFewRows = 16;

// One chunk of x and of w into a thread's registers, 16 bytes a piece; piece p is row p / (CHUNK / 4),
// 16-byte column p % (CHUNK / 4).  Every lane loads, from a clamped address, and what lies outside the
// operands is replaced by zeros afterwards (beyond K: the last piece again, then zeros): without a
// branch around the loads the compiler counts exactly how many loads are in flight and waits only
// for the stage it needs.
template <int ROWS, int CHUNK, int THREADS>
__device__ __forceinline__ void fetch_rows(float4 (&reg)[ROWS * (CHUNK / 4) / THREADS], const float* __restrict__ src, int tid,
                                           int row0, int rows_end, int stride, int K, int k0) {
#pragma unroll
    for (int j = 0; j < ROWS * (CHUNK / 4) / THREADS; ++j) {
        const int piece = j * THREADS + tid, row = row0 + piece / (CHUNK / 4), k = k0 + (piece % (CHUNK / 4)) * 4;
        const float4 v = *reinterpret_cast<const float4*>(src + static_cast<size_t>(min(row, rows_end - 1)) * stride + min(k, K - 4));
        const bool in = row < rows_end && k < K;       // element by element: a choice between two whole vectors goes through memory
        reg[j] = make_float4(in ? v.x : 0.f, in ? v.y : 0.f, in ? v.z : 0.f, in ? v.w : 0.f);
    }
}

template <int ROWS, int COLS, int CHUNK, int STAGES>
__global__ void __launch_bounds__(ROWS * COLS)
gemm_nt_few_rows_kernel(const float* __restrict__ x, const float* __restrict__ w, float* __restrict__ out, int M,
                        int N, int K_all) {
    constexpr int kThreads = ROWS * COLS;
    // this workgroup's segment of the K axis: x and w begin at its first key, K is its length, and the row
    // stride stays that of the whole operands
    const int seg_begin = blockIdx.y * kSegment;
    const int K = min(kSegment, K_all - seg_begin);
    x += seg_begin;
    w += seg_begin;
    out += static_cast<size_t>(blockIdx.y) * M * N;
    constexpr int kXPieces = ROWS * (CHUNK / 4) / kThreads, kWPieces = COLS * (CHUNK / 4) / kThreads;
    static_assert(kXPieces * kThreads == ROWS * (CHUNK / 4) && kWPieces * kThreads == COLS * (CHUNK / 4), "whole pieces per thread");
    __shared__ float4 xs[ROWS][CHUNK / 4 + 1];
    __shared__ float4 ws[COLS][CHUNK / 4 + 1];
    const int tid = threadIdx.x;
    const int col0 = blockIdx.x * COLS;
    const int r = tid / COLS, c = tid % COLS;
    float4 xreg[STAGES][kXPieces], wreg[STAGES][kWPieces];
    float acc = 0.f;
#pragma unroll
    for (int s = 0; s < STAGES; ++s) {
        fetch_rows<ROWS, CHUNK, kThreads>(xreg[s], x, tid, 0, M, K_all, K, s * CHUNK);
        fetch_rows<COLS, CHUNK, kThreads>(wreg[s], w, tid, col0, N, K_all, K, s * CHUNK);
    }
    for (int k0 = 0; k0 < K; k0 += STAGES * CHUNK) {
#pragma unroll
        for (int s = 0; s < STAGES; ++s) {
            const int kk = k0 + s * CHUNK;
            if (kk >= K) continue;       // the same for all threads (no `break`: the stages must unroll, or the register sets become memory)
            __syncthreads();
#pragma unroll
            for (int j = 0; j < kXPieces; ++j) xs[(j * kThreads + tid) / (CHUNK / 4)][(j * kThreads + tid) % (CHUNK / 4)] = xreg[s][j];
#pragma unroll
            for (int j = 0; j < kWPieces; ++j) ws[(j * kThreads + tid) / (CHUNK / 4)][(j * kThreads + tid) % (CHUNK / 4)] = wreg[s][j];
            __syncthreads();
            fetch_rows<ROWS, CHUNK, kThreads>(xreg[s], x, tid, 0, M, K_all, K, kk + STAGES * CHUNK);
            fetch_rows<COLS, CHUNK, kThreads>(wreg[s], w, tid, col0, N, K_all, K, kk + STAGES * CHUNK);
            // The whole chunk always (beyond K it holds zeros, which leave the sum as it is).  The reads of
            // eight steps are asked for while the eight steps before them are summed: the chain of
            // dependent additions is all a wavefront does here, and it should not wait for shared memory.
            constexpr int kBatch = 8;
            float4 a[2][kBatch], b[2][kBatch];
#pragma unroll
            for (int i = 0; i < kBatch; ++i) {
                a[0][i] = xs[r][i];
                b[0][i] = ws[c][i];
            }
#pragma unroll
            for (int k4 = 0; k4 < CHUNK / 4; k4 += kBatch) {
                const int cur = (k4 / kBatch) % 2, nxt = cur ^ 1;
                if (k4 + kBatch < CHUNK / 4) {
#pragma unroll
                    for (int i = 0; i < kBatch; ++i) {
                        a[nxt][i] = xs[r][k4 + kBatch + i];
                        b[nxt][i] = ws[c][k4 + kBatch + i];
                    }
                }
#pragma unroll
                for (int i = 0; i < kBatch; ++i) {
                    acc = fmaf(a[cur][i].x, b[cur][i].x, acc);
                    acc = fmaf(a[cur][i].y, b[cur][i].y, acc);
                    acc = fmaf(a[cur][i].z, b[cur][i].z, acc);
                    acc = fmaf(a[cur][i].w, b[cur][i].w, acc);
                }
            }
        }
    }
    if (r < M && col0 + c < N) out[static_cast<size_t>(r) * N + col0 + c] = acc;
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

// Segments of the K axis, and with them the floats of `partial` that `wllm_gemm_generic` needs for a
// float32 product of at most 16 rows: segments * M * N if there are several segments, none otherwise.
WLLM_API int wllm_gemm_generic_segments(int K) { return (K + kSegment - 1) / kSegment; }

WLLM_API int wllm_gemm_generic(const void* x, const void* w, int in_bf16, void* out, int out_bf16, void* partial, int M,
                               int N, int K, hipStream_t stream) {
    if (!in_bf16 && !out_bf16 && M >= 1 && M <= kFewRows && K % 4 == 0 && K >= 4 && N >= 1) {
        const int segments = (K + kSegment - 1) / kSegment;
        if (segments > 1 && !partial) return -1;
        if (segments > 65535) return -1;
        float* dst = segments > 1 ? static_cast<float*>(partial) : static_cast<float*>(out);
#define FEW(ROWS, COLS, CHUNK, STAGES)                                                                       \
    gemm_nt_few_rows_kernel<ROWS, COLS, CHUNK, STAGES><<<dim3((N + COLS - 1) / COLS, segments), ROWS * COLS, 0, stream>>>( \
        static_cast<const float*>(x), static_cast<const float*>(w), dst, M, N, K)
        // many workgroups: the large tile with one chunk on its way; few: small tiles, each with several
        if (static_cast<long long>((N + kFewRows - 1) / kFewRows) * segments > 512) FEW(16, 16, 128, 1);
        else if (M <= 8) FEW(8, 8, 128, 4);
        else FEW(16, 8, 128, 4);
#undef FEW
        if (int err = launch_status()) return err;
        if (segments > 1)
            gemm_segments_sum_kernel<<<(M * N + 255) / 256, 256, 0, stream>>>(dst, static_cast<float*>(out), M * N, segments);
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
