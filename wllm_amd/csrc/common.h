// Shared by all kernels: element types, conversions, reductions over a 64-wide
// wavefront and over a workgroup, launch checks.  gfx950 only.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#define WLLM_API extern "C" __attribute__((visibility("default")))

constexpr int kWave = 64;

// bfloat16 as its bits; conversions are explicit so that every rounding is visible.
struct bf16 {
    uint16_t bits;
};

__device__ __forceinline__ float to_float(float v) { return v; }
__device__ __forceinline__ float to_float(bf16 v) { return __uint_as_float(static_cast<uint32_t>(v.bits) << 16); }

template <typename T> __device__ __forceinline__ T from_float(float v);
template <> __device__ __forceinline__ float from_float<float>(float v) { return v; }
template <> __device__ __forceinline__ bf16 from_float<bf16>(float v) {
    // round to nearest, ties to even, NaN stays NaN: gfx950 converts in hardware (v_cvt_pk_bf16_f32)
    const __bf16 h = static_cast<__bf16>(v);
    return bf16{*reinterpret_cast<const uint16_t*>(&h)};
}

// Two floats to two bfloat16 in one word, the first in the low half (one v_cvt_pk_bf16_f32).
__device__ __forceinline__ uint32_t pack2_bf16(float lo, float hi) {
    typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
    typedef float float2_t __attribute__((ext_vector_type(2)));
    const float2_t f = {lo, hi};
    const bf16x2_t r = __builtin_convertvector(f, bf16x2_t);
    return *reinterpret_cast<const uint32_t*>(&r);
}

// The sum (maximum) of a lane's value and that of the lane 16 (32) further on or back, as `v op
// __shfl_xor(v, 16)` gives it, bit for bit, but with one swap instruction of the vector unit (gfx950's
// v_permlane16_swap / v_permlane32_swap) where a shuffle takes a trip through the LDS pipeline.
__device__ __forceinline__ void swap_halves(float v, int distance, float& a, float& b) {
    typedef unsigned uint2_t __attribute__((ext_vector_type(2)));
    const uint2_t r = distance == 16 ? __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false)
                                     : __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    a = __uint_as_float(r.x);
    b = __uint_as_float(r.y);
}
__device__ __forceinline__ float sum_across(float v, int distance) {
    float a, b;
    swap_halves(v, distance, a, b);
    return a + b;
}
__device__ __forceinline__ float max_across(float v, int distance) {
    float a, b;
    swap_halves(v, distance, a, b);
    return fmaxf(a, b);
}

// The value of another lane of the same row of 16 through the vector unit's own lane permutation
// (no trip through the LDS pipeline).  kCtrl: 0xB1 and 0x4E exchange the lanes 1 and 2 apart, 0x124 and
// 0x128 turn a row by 4 and by 8 lanes; a turn by 8 is the lane 8 apart, and a turn by 4 is the lane 4
// apart for values that are already the same 8 lanes apart, as they are in the butterflies below.
template <int kCtrl>
__device__ __forceinline__ float row_permuted(float v) {
    return __uint_as_float(static_cast<uint32_t>(
        __builtin_amdgcn_update_dpp(0, static_cast<int>(__float_as_uint(v)), kCtrl, 0xf, 0xf, false)));
}

// Butterflies over the 64 lanes, from the lanes 32 apart down to neighbours: the operands and their
// order are those of `v op __shfl_xor(v, off)` for off = 32 .. 1, so the results have the same bits.
__device__ __forceinline__ float wave_sum(float v) {
    v = sum_across(v, 32);
    v = sum_across(v, 16);
    v += row_permuted<0x128>(v);
    v += row_permuted<0x124>(v);
    v += row_permuted<0x4E>(v);
    v += row_permuted<0xB1>(v);
    return v;
}

__device__ __forceinline__ float wave_max(float v) {
    v = max_across(v, 32);
    v = max_across(v, 16);
    v = fmaxf(v, row_permuted<0x128>(v));
    v = fmaxf(v, row_permuted<0x124>(v));
    v = fmaxf(v, row_permuted<0x4E>(v));
    v = fmaxf(v, row_permuted<0xB1>(v));
    return v;
}

// Sum over a workgroup of up to 1024 threads; `scratch` holds 16 floats.  Every thread
// gets the result.  The order of the additions is fixed by the thread ids.
__device__ __forceinline__ float block_sum(float v, float* scratch) {
    const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
    const int waves = (blockDim.x + kWave - 1) / kWave;
    v = wave_sum(v);
    __syncthreads();
    if (lane == 0) scratch[wave] = v;
    __syncthreads();
    float total = 0.f;
    for (int w = 0; w < waves; ++w) total += scratch[w];
    return total;
}

// The sum of `splits` partial sums `stride` elements apart, added in stack order.  The loads of
// eight slices are issued before the first addition needs one.
__device__ __forceinline__ float stack_sum(const float* __restrict__ p, int splits, size_t stride) {
    float total = p[0];
    for (int s0 = 1; s0 < splits; s0 += 8) {
        float t[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) t[j] = s0 + j < splits ? p[(s0 + j) * stride] : 0.f;
#pragma unroll
        for (int j = 0; j < 8; ++j) total += t[j];
    }
    return total;
}

// 2^x by the hardware instruction alone, for the arguments of a softmax (x <= 0, -inf included):
// results below the smallest normal number become 0 instead of passing through the library's
// rescaling, which a probability does not need.
__device__ __forceinline__ float exp2_probability(float x) { return __builtin_amdgcn_exp2f(x); }

// The activations of a gated feed-forward, by the number the host passes (the table `ACTIVATIONS` of
// the Python side holds the same numbers): every kernel that applies one goes through `activate`,
// so a new activation is one line here, one there, and a case in `WLLM_BY_ACTIVATION`.
constexpr int kActGeluTanh = 0;      // 0.5 z (1 + tanh(sqrt(2/pi) (z + 0.044715 z^3)))
constexpr int kActSilu = 1;          // z / (1 + exp(-z))
constexpr int kActivations = 2;

template <int ACT>
__device__ __forceinline__ float activate(float z) {
    static_assert(ACT >= 0 && ACT < kActivations, "unknown activation");
    if (ACT == kActGeluTanh) return 0.5f * z * (1.f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
    return z / (1.f + expf(-z));
}

// Runs `statement` with the compile-time constant ACT set to the activation's number.
#define WLLM_BY_ACTIVATION(activation, statement)                                     \
    switch (activation) {                                                              \
        case kActGeluTanh: { constexpr int ACT = kActGeluTanh; statement; } break;     \
        default: { constexpr int ACT = kActSilu; statement; } break;                   \
    }

// One rotated pair (a, b) -> (a cos - b sin, b cos + a sin).  The products are fused in one fixed
// way, so that every kernel that rotates gives the same bits for the same numbers.
__device__ __forceinline__ void rotate_pair(float a, float b, float s, float c, float& ra, float& rb) {
    ra = __fmaf_rn(a, c, -(b * s));
    rb = __fmaf_rn(b, c, a * s);
}

// 16 bytes that are read once (weights, the cache's keys and values): the load carries the
// non-temporal bit, so the line is not kept where lines that are read again live.  A stream of such
// loads reads HBM at 7.1 TB/s where plain loads reach 6.3.
__device__ __forceinline__ uint4 load_streamed(const void* p) {
    typedef unsigned uint4_t __attribute__((ext_vector_type(4)));
    const uint4_t v = __builtin_nontemporal_load(reinterpret_cast<const uint4_t*>(p));
    return make_uint4(v.x, v.y, v.z, v.w);
}

__device__ __forceinline__ uint2 load_streamed8(const void* p) {
    typedef unsigned uint2_t __attribute__((ext_vector_type(2)));
    const uint2_t v = __builtin_nontemporal_load(reinterpret_cast<const uint2_t*>(p));
    return make_uint2(v.x, v.y);
}

// The error a launch left, as an int for the caller (0 = hipSuccess).
__host__ inline int launch_status() { return static_cast<int>(hipGetLastError()); }
