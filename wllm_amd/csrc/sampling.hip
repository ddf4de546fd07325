// Sampling kernels: one workgroup per row of float32 logits.
#include "common.h"

// ---- argmax: the largest value of a row, the lowest index among equals -------------------------
__global__ void __launch_bounds__(256) argmax_rows_kernel(const float* __restrict__ logits, int* __restrict__ out,
                                                         int vocab) {
    __shared__ float best_v[4];
    __shared__ int best_i[4];
    const float* row = logits + static_cast<size_t>(blockIdx.x) * vocab;
    float bv = -INFINITY;
    int bi = 0x7fffffff;
    for (int i = threadIdx.x; i < vocab; i += blockDim.x) {
        const float v = row[i];
        // NaN never wins; ascending i per thread, so ">" keeps the lowest index
        if (v > bv || bi == 0x7fffffff) {
            bv = v == v ? v : -INFINITY;
            bi = i;
        }
    }
#pragma unroll
    for (int off = kWave / 2; off > 0; off >>= 1) {
        const float ov = __shfl_xor(bv, off, kWave);
        const int oi = __shfl_xor(bi, off, kWave);
        if (ov > bv || (ov == bv && oi < bi)) {
            bv = ov;
            bi = oi;
        }
    }
    const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
    if (lane == 0) {
        best_v[wave] = bv;
        best_i[wave] = bi;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < 4; ++w)
            if (best_v[w] > bv || (best_v[w] == bv && best_i[w] < bi)) {
                bv = best_v[w];
                bi = best_i[w];
            }
        out[blockIdx.x] = bi == 0x7fffffff ? 0 : bi;
    }
}

WLLM_API int wllm_argmax_rows(const float* logits, int* out, int rows, int vocab, hipStream_t stream) {
    argmax_rows_kernel<<<rows, 256, 0, stream>>>(logits, out, vocab);
    return launch_status();
}
