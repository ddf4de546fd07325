// out[M, N] = x[M, K] * w[N, K]^T for float32 and bfloat16 operands, accumulated in float32 with
// fused multiply-adds on the vector units.  No matrix-core instruction and no reduced-precision
// mode is involved, so with float32 operands this is a true 32-bit product; it is the product
// of the float32 path, and the product of last resort for bfloat16 (shapes the matrix-core
// kernels do not take, float32 results from bfloat16 operands).
//
// A workgroup of 256 threads makes a 64x64 tile of the result; the K axis is walked in steps of
// 16 through shared memory; a thread holds a 4x4 block.  Each result element is the sum over k
// in ascending order, whatever the shape of the batch, so a row's result does not depend on the
// other rows.
#include "common.h"

constexpr int kTile = 64;
constexpr int kStep = 16;

template <typename TI, typename TO>
__global__ void __launch_bounds__(256)
gemm_nt_kernel(const TI* __restrict__ x, const TI* __restrict__ w, TO* __restrict__ out, int M, int N, int K) {
    __shared__ float xs[kStep][kTile + 4];
    __shared__ float ws[kStep][kTile + 4];
    const int tid = threadIdx.x;
    const int row0 = blockIdx.y * kTile, col0 = blockIdx.x * kTile;
    const int tr = (tid / 16) * 4, tc = (tid % 16) * 4;
    float acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;
    // each thread stages 4 elements of x and 4 of w per step: row = tid / 4, k = (tid % 4) * 4 ..
    const int lr = tid / 4, lk = (tid % 4) * 4;
    for (int k0 = 0; k0 < K; k0 += kStep) {
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
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int r = row0 + tr + i;
        if (r >= M) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int c = col0 + tc + j;
            if (c < N) out[static_cast<size_t>(r) * N + c] = from_float<TO>(acc[i][j]);
        }
    }
}

// The same product for at most 16 rows of float32 (the decode steps of the float32 path).  The big
// tile would leave all but N/64 workgroups idle and seven eighths of each tile empty; here a
// workgroup makes 16 rows x 16 columns, a thread one element, and the K axis is walked in chunks
// of 128 through shared memory.  An element is still the sum over k in ascending order of fused
// multiply-adds from zero, so it has the same bits as the kernel above gives it.
constexpr int kFewRows = 16;
constexpr int kFewChunk = 128;

__global__ void __launch_bounds__(256)
gemm_nt_few_rows_kernel(const float* __restrict__ x, const float* __restrict__ w, float* __restrict__ out, int M,
                        int N, int K) {
    __shared__ float4 xs[kFewRows][kFewChunk / 4 + 1];
    __shared__ float4 ws[kFewRows][kFewChunk / 4 + 1];
    const int tid = threadIdx.x;
    const int col0 = blockIdx.x * kFewRows;
    const int r = tid / 16, c = tid % 16;
    // staging: a thread moves two 16-byte pieces of x and two of w per chunk
    const int srow[2] = {tid / 32, tid / 32 + 8};
    const int sk = (tid % 32) * 4;
    float4 xreg[2], wreg[2];
    auto fetch = [&](int k0) {
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const bool in_k = k0 + sk < K;
            xreg[j] = (srow[j] < M && in_k) ? *reinterpret_cast<const float4*>(x + static_cast<size_t>(srow[j]) * K + k0 + sk)
                                            : make_float4(0.f, 0.f, 0.f, 0.f);
            wreg[j] = (col0 + srow[j] < N && in_k)
                          ? *reinterpret_cast<const float4*>(w + static_cast<size_t>(col0 + srow[j]) * K + k0 + sk)
                          : make_float4(0.f, 0.f, 0.f, 0.f);
        }
    };
    float acc = 0.f;
    fetch(0);
    for (int k0 = 0; k0 < K; k0 += kFewChunk) {
        __syncthreads();
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            xs[srow[j]][sk / 4] = xreg[j];
            ws[srow[j]][sk / 4] = wreg[j];
        }
        __syncthreads();
        if (k0 + kFewChunk < K) fetch(k0 + kFewChunk);
        const int len = min(kFewChunk, K - k0);     // a multiple of 4
        for (int k = 0; k < len; k += 4) {
            const float4 a = xs[r][k / 4], b = ws[c][k / 4];
            acc = fmaf(a.x, b.x, acc);
            acc = fmaf(a.y, b.y, acc);
            acc = fmaf(a.z, b.z, acc);
            acc = fmaf(a.w, b.w, acc);
        }
    }
    if (r < M && col0 + c < N) out[static_cast<size_t>(r) * N + col0 + c] = acc;
}

WLLM_API int wllm_gemm_generic(const void* x, const void* w, int in_bf16, void* out, int out_bf16, int M, int N,
                               int K, hipStream_t stream) {
    if (!in_bf16 && !out_bf16 && M <= kFewRows && K % 4 == 0) {
        gemm_nt_few_rows_kernel<<<(N + kFewRows - 1) / kFewRows, 256, 0, stream>>>(
            static_cast<const float*>(x), static_cast<const float*>(w), static_cast<float*>(out), M, N, K);
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
