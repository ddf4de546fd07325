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

WLLM_API int wllm_gemm_generic(const void* x, const void* w, int in_bf16, void* out, int out_bf16, int M, int N,
                               int K, hipStream_t stream) {
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
