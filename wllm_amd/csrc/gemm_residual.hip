// residual[M, N] += x[M, K] . w[N, K]^T for bfloat16 x and w with at most 16 rows, the sum going
// straight into the float32 residual stream; beside it the kernel leaves, for every row and band
// of 16 columns, the sum of squares of the new residual values.  The kernel that reads the stream
// next (a projection with the norm folded into its load of x) adds those sums per row and has the
// row's mean square without a pass of its own over the stream, and no norm kernel runs between.
//
// The product is made as in `qkv_rope.hip`: a workgroup owns one band of 16 columns (16 rows of w,
// read row by row or from the tile-major copy); its wavefronts split the K axis, keep 8 steps of
// 32 keys in flight each (a register is refilled as soon as its product is issued), read x as the
// B operand straight from memory, and add their sums through shared memory in the order of the
// pieces.  So every output element is summed in one fixed order, whatever the batch holds.
#include "common.h"

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float float4_t __attribute__((ext_vector_type(4)));

union RFrag {
    uint4 u;
    bf16x8_t v;
};

template <int WAVES, bool TILED>
__global__ void __launch_bounds__(WAVES * 64)
gemm_residual_kernel(const bf16* __restrict__ x, const bf16* __restrict__ w, float* __restrict__ residual,
                     float* __restrict__ sumsq, int M, int N, int K) {
    __shared__ float4_t red[(WAVES - 1) * kWave];
    const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
    const int i = lane % 16, g = lane / 16;
    const int band = blockIdx.x, bands = gridDim.x;
    const int steps = K / 32;
    const int per = (steps + WAVES - 1) / WAVES;
    const int s0 = wave * per, s1 = min(steps, s0 + per);
    constexpr int kStep = TILED ? 512 : 32;             // elements from one step of 32 keys to the next
    const bf16* wp = TILED ? w + static_cast<size_t>(band) * steps * 512 + lane * 8
                           : w + (static_cast<size_t>(band) * 16 + i) * K + 8 * g;
    const bf16* xp = x + static_cast<size_t>(min(i, M - 1)) * K + 8 * g;
    const bool x_row = i < M;
    constexpr int U = 8;
    RFrag cw[U], cx[U];
    auto load_step = [&](int u, int at) {
        const bool ok = at < s1;
        cw[u].u = ok ? load_streamed(wp + static_cast<size_t>(at) * kStep) : make_uint4(0, 0, 0, 0);
        cx[u].u = ok && x_row ? *reinterpret_cast<const uint4*>(xp + static_cast<size_t>(at) * 32) : make_uint4(0, 0, 0, 0);
    };
#pragma unroll
    for (int u = 0; u < U; ++u) load_step(u, s0 + u);
    // the residual values this lane will add to, asked for now
    const int n = band * 16 + 4 * g;
    float4_t old = float4_t{0.f, 0.f, 0.f, 0.f};
    if (wave == 0 && x_row) old = *reinterpret_cast<const float4_t*>(residual + static_cast<size_t>(i) * N + n);
    float4_t acc[2] = {float4_t{0.f, 0.f, 0.f, 0.f}, float4_t{0.f, 0.f, 0.f, 0.f}};
    for (int s = s0; s < s1; s += U) {
#pragma unroll
        for (int u = 0; u < U; ++u) {
            acc[u % 2] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(cw[u].v, cx[u].v, acc[u % 2], 0, 0, 0);
            load_step(u, s + U + u);
        }
    }
    float4_t sum = acc[0] + acc[1];
    if (WAVES > 1) {
        if (wave > 0) red[(wave - 1) * kWave + lane] = sum;
        __syncthreads();
        if (wave > 0) return;
#pragma unroll
        for (int q = 0; q < WAVES - 1; ++q) sum += red[q * kWave + lane];
    }
    // lane (i, g): row m = i, columns n .. n + 3
    float sq = 0.f;
    if (x_row) {
        const float4_t now = old + sum;
        *reinterpret_cast<float4_t*>(residual + static_cast<size_t>(i) * N + n) = now;
        sq = now[0] * now[0] + now[1] * now[1] + now[2] * now[2] + now[3] * now[3];
    }
    // the band's 16 columns of a row lie in the four lanes i, i + 16, i + 32, i + 48
    sq = sum_across(sum_across(sq, 16), 32);
    if (x_row && g == 0) sumsq[static_cast<size_t>(i) * bands + band] = sq;
}

// Returns 0, a HIP error code, or -1 for sizes this kernel does not take.  sumsq is float32
// [M, N / 16].
WLLM_API int wllm_gemm_residual(const void* x, const void* w, int tiled, float* residual, float* sumsq, int M, int N,
                                int K, hipStream_t stream) {
    if (M < 1 || M > 16 || N < 16 || N % 16 != 0 || K < 32 || K % 32 != 0) return -1;
    const int bands = N / 16;
#define LAUNCH(W, T)                                                                                                  \
    gemm_residual_kernel<W, T><<<bands, W * 64, 0, stream>>>(static_cast<const bf16*>(x), static_cast<const bf16*>(w), \
                                                             residual, sumsq, M, N, K)
    // sixteen wavefronts a band where the K axis is long, so that enough of them stream at once
    if (K > 2048) {
        if (tiled) LAUNCH(16, true);
        else LAUNCH(16, false);
    } else {
        if (tiled) LAUNCH(8, true);
        else LAUNCH(8, false);
    }
#undef LAUNCH
    return launch_status();
}
