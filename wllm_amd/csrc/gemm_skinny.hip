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

template <typename TO> __device__ __forceinline__ void store4(TO* p, float4_t v);
template <> __device__ __forceinline__ void store4<float>(float* p, float4_t v) { *reinterpret_cast<float4_t*>(p) = v; }
template <> __device__ __forceinline__ void store4<bf16>(bf16* p, float4_t v) {
    uint2 w;
    w.x = from_float<bf16>(v[0]).bits | (static_cast<uint32_t>(from_float<bf16>(v[1]).bits) << 16);
    w.y = from_float<bf16>(v[2]).bits | (static_cast<uint32_t>(from_float<bf16>(v[3]).bits) << 16);
    *reinterpret_cast<uint2*>(p) = w;
}

template <int MT, typename TO>
__global__ void __launch_bounds__(256)
gemm_skinny_kernel(const bf16* __restrict__ x, const bf16* __restrict__ w, TO* __restrict__ out,
                   float* __restrict__ partial, int M, int N, int K, int k_per_split, int chunk) {
    extern __shared__ uint4 xs[];                 // [MT*16][chunk/8 + 1]
    const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
    const int i = lane % 16, g = lane / 16;
    const int n0 = (blockIdx.x * 4 + wave) * 16;
    const int k_begin = blockIdx.y * k_per_split, k_end = min(K, k_begin + k_per_split);
    const int stride = chunk / 8 + 1;             // in uint4; the odd stride spreads rows over the banks
    const bf16* wrow = w + static_cast<size_t>(min(n0 + i, N - 1)) * K;
    float4_t acc[MT];
#pragma unroll
    for (int t = 0; t < MT; ++t) acc[t] = float4_t{0.f, 0.f, 0.f, 0.f};

    for (int kc = k_begin; kc < k_end; kc += chunk) {
        const int len = min(chunk, k_end - kc);   // a multiple of 32
        const int vecs = len / 8;
        __syncthreads();
        for (int idx = threadIdx.x; idx < MT * 16 * vecs; idx += blockDim.x) {
            const int m = idx / vecs, c = idx % vecs;
            uint4 v = make_uint4(0, 0, 0, 0);
            if (m < M) v = *reinterpret_cast<const uint4*>(x + static_cast<size_t>(m) * K + kc + c * 8);
            xs[m * stride + c] = v;
        }
        __syncthreads();
        if (n0 < N) {
            const bf16* wp = wrow + kc + 8 * g;
            int k = 0;
            // four weight loads in flight per lane before the first product needs one
            for (; k + 128 <= len; k += 128) {
                Frag a[4];
#pragma unroll
                for (int u = 0; u < 4; ++u) a[u].u = *reinterpret_cast<const uint4*>(wp + k + 32 * u);
#pragma unroll
                for (int u = 0; u < 4; ++u) {
#pragma unroll
                    for (int t = 0; t < MT; ++t) {
                        Frag b;
                        b.u = xs[(t * 16 + i) * stride + (k + 32 * u) / 8 + g];
                        acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[u].v, b.v, acc[t], 0, 0, 0);
                    }
                }
            }
            for (; k < len; k += 32) {
                Frag a;
                a.u = *reinterpret_cast<const uint4*>(wp + k);
#pragma unroll
                for (int t = 0; t < MT; ++t) {
                    Frag b;
                    b.u = xs[(t * 16 + i) * stride + k / 8 + g];
                    acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a.v, b.v, acc[t], 0, 0, 0);
                }
            }
        }
    }
    if (n0 >= N) return;
    // lane (i, g) holds columns n0 + 4g .. +3 of row m = 16t + i
    const int n = n0 + 4 * g;
#pragma unroll
    for (int t = 0; t < MT; ++t) {
        const int m = t * 16 + i;
        if (m >= M) continue;
        if (gridDim.y == 1) {
            TO* o = out + static_cast<size_t>(m) * N + n;
            if (n + 3 < N && (N % 4 == 0)) {
                store4<TO>(o, acc[t]);
            } else {
#pragma unroll
                for (int v = 0; v < 4; ++v)
                    if (n + v < N) o[v] = from_float<TO>(acc[t][v]);
            }
        } else {
            float* o = partial + (static_cast<size_t>(blockIdx.y) * M + m) * N + n;
            if (n + 3 < N && (N % 4 == 0)) {
                *reinterpret_cast<float4_t*>(o) = acc[t];
            } else {
#pragma unroll
                for (int v = 0; v < 4; ++v)
                    if (n + v < N) o[v] = acc[t][v];
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

// Returns 0, a HIP error code, or -1 for sizes this kernel does not take.
// `partial` must hold splits * M * N floats when splits > 1; with `out` null the partial sums
// are the result and nothing adds them.
WLLM_API int wllm_gemm_skinny(const void* x, const void* w, void* out, int out_bf16, float* partial, int M, int N,
                              int K, int splits, int chunk, hipStream_t stream) {
    if (M < 1 || M > 64 || K % 32 != 0 || splits < 1 || K % splits != 0 || (K / splits) % 32 != 0 || chunk % 32 != 0)
        return -1;
    const int mt = (M + 15) / 16;
    const int k_per_split = K / splits;
    if (chunk > k_per_split) chunk = k_per_split;
    const size_t smem = static_cast<size_t>(mt) * 16 * (chunk / 8 + 1) * sizeof(uint4);
    if (smem > 65536) return -1;
    const dim3 grid((N + 63) / 64, splits);
#define LAUNCH(MT, TO)                                                                                       \
    gemm_skinny_kernel<MT, TO><<<grid, 256, smem, stream>>>(static_cast<const bf16*>(x), static_cast<const bf16*>(w), \
                                                            static_cast<TO*>(out), partial, M, N, K, k_per_split, chunk)
#define BY_MT(TO)                    \
    switch (mt) {                    \
        case 1: LAUNCH(1, TO); break; \
        case 2: LAUNCH(2, TO); break; \
        case 3: LAUNCH(3, TO); break; \
        default: LAUNCH(4, TO); break; \
    }
    if (out_bf16) { BY_MT(bf16) } else { BY_MT(float) }
#undef BY_MT
#undef LAUNCH
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
__device__ __forceinline__ float act_gelu_tanh(float z) {
    return 0.5f * z * (1.f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
}
__device__ __forceinline__ float act_silu(float z) { return z / (1.f + expf(-z)); }

template <int MT, int ACT>
__global__ void __launch_bounds__(256)
gemm_skinny_gated_kernel(const bf16* __restrict__ x, const bf16* __restrict__ w, bf16* __restrict__ out, int M,
                         int inter, int K, int chunk) {
    extern __shared__ uint4 xs[];
    const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
    const int i = lane % 16, g = lane / 16;
    const int n0 = (blockIdx.x * 4 + wave) * 16;
    const int stride = chunk / 8 + 1;
    const int nrow = min(n0 + i, inter - 1);
    const bf16* grow = w + static_cast<size_t>(nrow) * K;
    const bf16* urow = w + static_cast<size_t>(inter + nrow) * K;
    float4_t accg[MT], accu[MT];
#pragma unroll
    for (int t = 0; t < MT; ++t) {
        accg[t] = float4_t{0.f, 0.f, 0.f, 0.f};
        accu[t] = float4_t{0.f, 0.f, 0.f, 0.f};
    }
    for (int kc = 0; kc < K; kc += chunk) {
        const int len = min(chunk, K - kc);
        const int vecs = len / 8;
        __syncthreads();
        for (int idx = threadIdx.x; idx < MT * 16 * vecs; idx += blockDim.x) {
            const int m = idx / vecs, c = idx % vecs;
            uint4 v = make_uint4(0, 0, 0, 0);
            if (m < M) v = *reinterpret_cast<const uint4*>(x + static_cast<size_t>(m) * K + kc + c * 8);
            xs[m * stride + c] = v;
        }
        __syncthreads();
        if (n0 < inter) {
            const bf16* gp = grow + kc + 8 * g;
            const bf16* up = urow + kc + 8 * g;
            int k = 0;
            for (; k + 64 <= len; k += 64) {
                Frag a[4];
                a[0].u = *reinterpret_cast<const uint4*>(gp + k);
                a[1].u = *reinterpret_cast<const uint4*>(up + k);
                a[2].u = *reinterpret_cast<const uint4*>(gp + k + 32);
                a[3].u = *reinterpret_cast<const uint4*>(up + k + 32);
#pragma unroll
                for (int u2 = 0; u2 < 2; ++u2) {
#pragma unroll
                    for (int t = 0; t < MT; ++t) {
                        Frag b;
                        b.u = xs[(t * 16 + i) * stride + (k + 32 * u2) / 8 + g];
                        accg[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[2 * u2].v, b.v, accg[t], 0, 0, 0);
                        accu[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[2 * u2 + 1].v, b.v, accu[t], 0, 0, 0);
                    }
                }
            }
            for (; k < len; k += 32) {
                Frag ag, au;
                ag.u = *reinterpret_cast<const uint4*>(gp + k);
                au.u = *reinterpret_cast<const uint4*>(up + k);
#pragma unroll
                for (int t = 0; t < MT; ++t) {
                    Frag b;
                    b.u = xs[(t * 16 + i) * stride + k / 8 + g];
                    accg[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ag.v, b.v, accg[t], 0, 0, 0);
                    accu[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(au.v, b.v, accu[t], 0, 0, 0);
                }
            }
        }
    }
    if (n0 >= inter) return;
    const int n = n0 + 4 * g;
#pragma unroll
    for (int t = 0; t < MT; ++t) {
        const int m = t * 16 + i;
        if (m >= M) continue;
        float4_t r;
#pragma unroll
        for (int v = 0; v < 4; ++v) r[v] = (ACT == 0 ? act_gelu_tanh(accg[t][v]) : act_silu(accg[t][v])) * accu[t][v];
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

WLLM_API int wllm_gemm_skinny_gated(const void* x, const void* w, void* out, int M, int inter, int K, int activation,
                                    int chunk, hipStream_t stream) {
    if (M < 1 || M > 64 || K % 32 != 0 || chunk % 32 != 0 || activation < 0 || activation > 1) return -1;
    const int mt = (M + 15) / 16;
    if (chunk > K) chunk = K;
    const size_t smem = static_cast<size_t>(mt) * 16 * (chunk / 8 + 1) * sizeof(uint4);
    if (smem > 65536) return -1;
    const dim3 grid((inter + 63) / 64);
#define LAUNCH(MT, A)                                                                                              \
    gemm_skinny_gated_kernel<MT, A><<<grid, 256, smem, stream>>>(static_cast<const bf16*>(x), static_cast<const bf16*>(w), \
                                                                 static_cast<bf16*>(out), M, inter, K, chunk)
#define BY_MT(A)                     \
    switch (mt) {                    \
        case 1: LAUNCH(1, A); break; \
        case 2: LAUNCH(2, A); break; \
        case 3: LAUNCH(3, A); break; \
        default: LAUNCH(4, A); break; \
    }
    if (activation == 0) { BY_MT(0) } else { BY_MT(1) }
#undef BY_MT
#undef LAUNCH
    return launch_status();
}
