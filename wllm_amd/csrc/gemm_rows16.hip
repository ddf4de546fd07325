// out[M, N] = x[M, K] * w[N, K]^T for bfloat16 with at most 16 rows of x: the products of a decode
// step of a small batch, bound by reading w once from HBM.
//
// What fills the memory system here is many short-lived wavefronts that each issue all their loads
// at once.  A wavefront owns 16 rows of w and a piece of the K axis; it issues the 16-byte loads
// of U steps of 32 keys (weights as the A operand of v_mfma_f32_16x16x32_bf16, lane (i, g) reading
// w[n0 + i][k + 8g .. +8]; the rows of x as the B operand, the same pattern on x, which stays in
// the caches) before the first product, and refills a register as soon as its product is issued.
// There is no staging through shared memory and no barrier in the stream.  A workgroup is WAVES
// pieces of the K axis of one tile of 16 weight rows; their sums are added through shared memory
// in the order of the pieces.  The K axis may be split over workgroups as well (grid.y); those
// partial sums are float32 and left to the consumer or added by `split_sum` in split order.  All
// splits depend on N and K only, so a row's result does not depend on the other rows of the batch.
#include "common.h"

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float float4_t __attribute__((ext_vector_type(4)));

union Frag16 {
    uint4 u;
    bf16x8_t v;
};

__device__ __forceinline__ uint4 load16(const bf16* p) { return *reinterpret_cast<const uint4*>(p); }

template <typename TO> __device__ __forceinline__ void store_columns(TO* o, float4_t v, int n, int N);
template <> __device__ __forceinline__ void store_columns<float>(float* o, float4_t v, int n, int N) {
    if (n + 3 < N && N % 4 == 0) {
        *reinterpret_cast<float4_t*>(o) = v;
    } else {
#pragma unroll
        for (int c = 0; c < 4; ++c)
            if (n + c < N) o[c] = v[c];
    }
}
template <> __device__ __forceinline__ void store_columns<bf16>(bf16* o, float4_t v, int n, int N) {
    if (n + 3 < N && N % 4 == 0) {
        uint2 w;
        w.x = pack2_bf16(v[0], v[1]);
        w.y = pack2_bf16(v[2], v[3]);
        *reinterpret_cast<uint2*>(o) = w;
    } else {
#pragma unroll
        for (int c = 0; c < 4; ++c)
            if (n + c < N) o[c] = from_float<bf16>(v[c]);
    }
}

template <int WAVES, int U, typename TO>
__global__ void __launch_bounds__(WAVES * 64, 4)
gemm_rows16_kernel(const bf16* __restrict__ x, const bf16* __restrict__ w, TO* __restrict__ out,
                   float* __restrict__ partial, int M, int N, int K, int k_per_split) {
    __shared__ float4_t red[(WAVES > 1 ? WAVES - 1 : 1) * kWave];
    const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
    const int i = lane % 16, g = lane / 16;
    const int n0 = blockIdx.x * 16;
    const int k_begin = blockIdx.y * k_per_split;
    const int steps = k_per_split / 32;
    const int per = (steps + WAVES - 1) / WAVES;
    const int s0 = wave * per, s1 = min(steps, s0 + per);
    const bf16* wp = w + static_cast<size_t>(min(n0 + i, N - 1)) * K + k_begin + 8 * g;
    const bf16* xp = x + static_cast<size_t>(min(i, M - 1)) * K + k_begin + 8 * g;
    const bool x_row = i < M;
    const uint4 zero = make_uint4(0, 0, 0, 0);
    Frag16 cw[U], cx[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
        const bool ok = s0 + u < s1;
        cw[u].u = ok ? load16(wp + (s0 + u) * 32) : zero;
        cx[u].u = ok && x_row ? load16(xp + (s0 + u) * 32) : zero;
    }
    float4_t acc[2] = {float4_t{0.f, 0.f, 0.f, 0.f}, float4_t{0.f, 0.f, 0.f, 0.f}};
    for (int s = s0; s < s1; s += U) {
#pragma unroll
        for (int u = 0; u < U; ++u) {
            acc[u % 2] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(cw[u].v, cx[u].v, acc[u % 2], 0, 0, 0);
            const bool ok = s + U + u < s1;
            cw[u].u = ok ? load16(wp + (s + U + u) * 32) : zero;
            cx[u].u = ok && x_row ? load16(xp + (s + U + u) * 32) : zero;
        }
    }
    float4_t sum = acc[0] + acc[1];
    if (WAVES > 1) {
        if (wave > 0) red[(wave - 1) * kWave + lane] = sum;
        __syncthreads();
        if (wave > 0) return;
#pragma unroll
        for (int p = 0; p < WAVES - 1; ++p) sum += red[p * kWave + lane];
    }
    // lane (i, g) holds columns n .. n + 3 of row m = i
    const int n = n0 + 4 * g, m = i;
    if (m >= M || n >= N) return;
    if (gridDim.y == 1) store_columns<TO>(out + static_cast<size_t>(m) * N + n, sum, n, N);
    else store_columns<float>(partial + (static_cast<size_t>(blockIdx.y) * M + m) * N + n, sum, n, N);
}

template <typename TO>
__global__ void rows16_split_sum_kernel(const float* __restrict__ partial, TO* __restrict__ out, int total, int splits) {
    const int idx = blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= total) return;
    float s = 0.f;
    for (int p = 0; p < splits; ++p) s += partial[static_cast<size_t>(p) * total + idx];
    out[idx] = from_float<TO>(s);
}

// Returns 0, a HIP error code, or -1 for sizes this kernel does not take.  `partial` must hold
// splits * M * N floats when splits > 1; with `out` null the partial sums are the result.
WLLM_API int wllm_gemm_rows16(const void* x, const void* w, void* out, int out_bf16, float* partial, int M, int N, int K,
                              int splits, hipStream_t stream) {
    if (M < 1 || M > 16 || N < 1 || K % 32 != 0 || splits < 1 || K % splits != 0 || (K / splits) % 32 != 0) return -1;
    if ((splits > 1 && partial == nullptr) || (splits == 1 && out == nullptr)) return -1;
    const int k_per_split = K / splits;
    const dim3 grid((N + 15) / 16, splits);
    constexpr int kWaves = 8, kU = 8;
    if (out_bf16)
        gemm_rows16_kernel<kWaves, kU, bf16><<<grid, kWaves * 64, 0, stream>>>(
            static_cast<const bf16*>(x), static_cast<const bf16*>(w), static_cast<bf16*>(out), partial, M, N, K, k_per_split);
    else
        gemm_rows16_kernel<kWaves, kU, float><<<grid, kWaves * 64, 0, stream>>>(
            static_cast<const bf16*>(x), static_cast<const bf16*>(w), static_cast<float*>(out), partial, M, N, K, k_per_split);
    int err = launch_status();
    if (err) return err;
    if (splits > 1 && out != nullptr) {
        const int total = M * N;
        if (out_bf16) rows16_split_sum_kernel<bf16><<<(total + 255) / 256, 256, 0, stream>>>(partial, static_cast<bf16*>(out), total, splits);
        else rows16_split_sum_kernel<float><<<(total + 255) / 256, 256, 0, stream>>>(partial, static_cast<float*>(out), total, splits);
        err = launch_status();
    }
    return err;
}

// ---- gated feed-forward input: out[M, I] = act(x . Wg^T) * (x . Wu^T), w = [Wg; Wu] of 2I rows -----
// A wavefront streams 16 gate rows and the 16 up rows that belong to them over its piece of K;
// both results land in the same lanes, so after the pieces are added the activation and the
// product are made in registers and only [M, I] is written.
__device__ __forceinline__ float rows16_gelu_tanh(float z) {
    return 0.5f * z * (1.f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
}
__device__ __forceinline__ float rows16_silu(float z) { return z / (1.f + expf(-z)); }

template <int WAVES, int U, int ACT>
__global__ void __launch_bounds__(WAVES * 64, 4)
gemm_rows16_gated_kernel(const bf16* __restrict__ x, const bf16* __restrict__ w, bf16* __restrict__ out, int M, int inter,
                         int K) {
    __shared__ float4_t red[(WAVES - 1) * kWave * 2];
    const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
    const int i = lane % 16, g = lane / 16;
    const int n0 = blockIdx.x * 16;
    const int steps = K / 32;
    const int per = (steps + WAVES - 1) / WAVES;
    const int s0 = wave * per, s1 = min(steps, s0 + per);
    const int nrow = min(n0 + i, inter - 1);
    const bf16* gp = w + static_cast<size_t>(nrow) * K + 8 * g;
    const bf16* up = w + static_cast<size_t>(inter + nrow) * K + 8 * g;
    const bf16* xp = x + static_cast<size_t>(min(i, M - 1)) * K + 8 * g;
    const bool x_row = i < M;
    const uint4 zero = make_uint4(0, 0, 0, 0);
    Frag16 cg[U], cu[U], cx[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
        const bool ok = s0 + u < s1;
        cg[u].u = ok ? load16(gp + (s0 + u) * 32) : zero;
        cu[u].u = ok ? load16(up + (s0 + u) * 32) : zero;
        cx[u].u = ok && x_row ? load16(xp + (s0 + u) * 32) : zero;
    }
    float4_t accg = float4_t{0.f, 0.f, 0.f, 0.f}, accu = float4_t{0.f, 0.f, 0.f, 0.f};
    for (int s = s0; s < s1; s += U) {
#pragma unroll
        for (int u = 0; u < U; ++u) {
            accg = __builtin_amdgcn_mfma_f32_16x16x32_bf16(cg[u].v, cx[u].v, accg, 0, 0, 0);
            accu = __builtin_amdgcn_mfma_f32_16x16x32_bf16(cu[u].v, cx[u].v, accu, 0, 0, 0);
            const bool ok = s + U + u < s1;
            cg[u].u = ok ? load16(gp + (s + U + u) * 32) : zero;
            cu[u].u = ok ? load16(up + (s + U + u) * 32) : zero;
            cx[u].u = ok && x_row ? load16(xp + (s + U + u) * 32) : zero;
        }
    }
    if (wave > 0) {
        red[((wave - 1) * kWave + lane) * 2] = accg;
        red[((wave - 1) * kWave + lane) * 2 + 1] = accu;
    }
    __syncthreads();
    if (wave > 0) return;
#pragma unroll
    for (int p = 0; p < WAVES - 1; ++p) {
        accg += red[(p * kWave + lane) * 2];
        accu += red[(p * kWave + lane) * 2 + 1];
    }
    const int n = n0 + 4 * g, m = i;
    if (m >= M || n >= inter) return;
    float4_t r;
#pragma unroll
    for (int c = 0; c < 4; ++c) r[c] = (ACT == 0 ? rows16_gelu_tanh(accg[c]) : rows16_silu(accg[c])) * accu[c];
    store_columns<bf16>(out + static_cast<size_t>(m) * inter + n, r, n, inter);
}

WLLM_API int wllm_gemm_rows16_gated(const void* x, const void* w, void* out, int M, int inter, int K, int activation,
                                    hipStream_t stream) {
    if (M < 1 || M > 16 || inter < 1 || K % 32 != 0 || activation < 0 || activation > 1) return -1;
    constexpr int kWaves = 8, kU = 8;
    const dim3 grid((inter + 15) / 16);
    if (activation == 0)
        gemm_rows16_gated_kernel<kWaves, kU, 0><<<grid, kWaves * 64, 0, stream>>>(
            static_cast<const bf16*>(x), static_cast<const bf16*>(w), static_cast<bf16*>(out), M, inter, K);
    else
        gemm_rows16_gated_kernel<kWaves, kU, 1><<<grid, kWaves * 64, 0, stream>>>(
            static_cast<const bf16*>(x), static_cast<const bf16*>(w), static_cast<bf16*>(out), M, inter, K);
    return launch_status();
}
