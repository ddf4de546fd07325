// Sampling kernels over rows of float32 logits.
#include "common.h"
#include "wllm_no_alloc.h"

#include <mutex>

// ---- argmax: the largest value of a row, the lowest index among equals -------------------------
// Two stages, so that a handful of rows still use many compute units: a row is cut into
// kArgmaxSplits segments, one workgroup each, then one wavefront per row picks among them.
constexpr int kArgmaxThreads = 256;
constexpr int kArgmaxSplits = 32;

__device__ __forceinline__ void argmax_take(float v, int i, float& bv, int& bi) {
    // NaN never wins; among equals the lowest index
    if (v > bv || (v == bv && i < bi) || bi == 0x7fffffff) {
        bv = v == v ? v : -INFINITY;
        bi = i;
    }
}

__device__ __forceinline__ void argmax_wave(float& bv, int& bi) {
#pragma unroll
    for (int off = kWave / 2; off > 0; off >>= 1) {
        const float ov = __shfl_xor(bv, off, kWave);
        const int oi = __shfl_xor(bi, off, kWave);
        if (ov > bv || (ov == bv && oi < bi)) {
            bv = ov;
            bi = oi;
        }
    }
}

__global__ void __launch_bounds__(kArgmaxThreads)
argmax_partial_kernel(const float* __restrict__ logits, float* __restrict__ part_v, int* __restrict__ part_i,
                      int vocab, int segment) {
    __shared__ float best_v[kArgmaxThreads / kWave];
    __shared__ int best_i[kArgmaxThreads / kWave];
    const float* row = logits + static_cast<size_t>(blockIdx.x) * vocab;
    const int begin = blockIdx.y * segment, end = min(vocab, begin + segment);
    float bv = -INFINITY;
    int bi = 0x7fffffff;
    if (vocab % 4 == 0) {
        // rows and segments are 16-byte aligned: four values per load
        const float4* row4 = reinterpret_cast<const float4*>(row);
        for (int q = begin / 4 + threadIdx.x; q < end / 4; q += blockDim.x) {
            const float4 v = row4[q];
            argmax_take(v.x, 4 * q, bv, bi);
            argmax_take(v.y, 4 * q + 1, bv, bi);
            argmax_take(v.z, 4 * q + 2, bv, bi);
            argmax_take(v.w, 4 * q + 3, bv, bi);
        }
    } else {
        for (int i = begin + threadIdx.x; i < end; i += blockDim.x) argmax_take(row[i], i, bv, bi);
    }
    argmax_wave(bv, bi);
    const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
    if (lane == 0) {
        best_v[wave] = bv;
        best_i[wave] = bi;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < kArgmaxThreads / kWave; ++w)
            if (best_v[w] > bv || (best_v[w] == bv && best_i[w] < bi)) {
                bv = best_v[w];
                bi = best_i[w];
            }
        part_v[blockIdx.x * kArgmaxSplits + blockIdx.y] = bv;
        part_i[blockIdx.x * kArgmaxSplits + blockIdx.y] = bi;
    }
}

__global__ void __launch_bounds__(kWave)
argmax_final_kernel(const float* __restrict__ part_v, const int* __restrict__ part_i, int* __restrict__ out) {
    const int lane = threadIdx.x;
    float bv = lane < kArgmaxSplits ? part_v[blockIdx.x * kArgmaxSplits + lane] : -INFINITY;
    int bi = lane < kArgmaxSplits ? part_i[blockIdx.x * kArgmaxSplits + lane] : 0x7fffffff;
    argmax_wave(bv, bi);
    if (lane == 0) out[blockIdx.x] = bi == 0x7fffffff ? 0 : bi;
}

// `workspace` holds rows * 64 four-byte words.
WLLM_API int wllm_argmax_rows(const float* logits, int* out, void* workspace, int rows, int vocab, hipStream_t stream) {
    float* part_v = static_cast<float*>(workspace);
    int* part_i = reinterpret_cast<int*>(part_v + static_cast<size_t>(rows) * kArgmaxSplits);
    int segment = (vocab + kArgmaxSplits - 1) / kArgmaxSplits;
    segment = (segment + 3) / 4 * 4;
    argmax_partial_kernel<<<dim3(rows, kArgmaxSplits), kArgmaxThreads, 0, stream>>>(logits, part_v, part_i, vocab, segment);
    argmax_final_kernel<<<rows, kWave, 0, stream>>>(part_v, part_i, out);
    return launch_status();
}

// ---- sampling with temperature, top-k, top-p, min-p and repetition penalty -----------------------
// One workgroup of 1024 threads per row.  The steps follow the reference's sampler in its order
// (src/wllm/engine/sampling.py:101-143): repetition penalty on the ids already generated
// (positive logits divided, negative multiplied, :45-58), temperature (:122-123), the three
// truncations on the full temperature-scaled distribution (:61-98: rank < k; cumulative
// probability in descending order <= p, the top token always kept; probability >= min_p times
// the top probability), a draw from what is left, and the log-probability of the drawn token
// before truncation (:125-130,142).  Two things differ by design.  The draw is the inverse of
// the cumulative distribution, in index order, at one uniform number from a counter-based
// generator keyed by (seed, counter), so a row's token does not depend on the other rows of the
// batch.  And all sums that decide a threshold or the draw are made in 40-bit fixed point with
// integer additions, so they do not depend on the order of the additions: the same row gives
// the same token on every run.  Equal logits are kept or dropped together.
constexpr int kSampleThreads = 1024;
constexpr double kFixedOne = 1099511627776.0;   // 2^40

__device__ __forceinline__ uint32_t sortable_key(float v) {
    const uint32_t u = __float_as_uint(v);
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

__device__ __forceinline__ void philox4x32_10(uint32_t ctr[4], uint32_t key0, uint32_t key1) {
#pragma unroll
    for (int r = 0; r < 10; ++r) {
        const uint32_t hi0 = __umulhi(0xD2511F53u, ctr[0]), lo0 = 0xD2511F53u * ctr[0];
        const uint32_t hi1 = __umulhi(0xCD9E8D57u, ctr[2]), lo1 = 0xCD9E8D57u * ctr[2];
        const uint32_t c0 = hi1 ^ ctr[1] ^ key0, c2 = hi0 ^ ctr[3] ^ key1;
        ctr[0] = c0;
        ctr[1] = lo1;
        ctr[2] = c2;
        ctr[3] = lo0;
        key0 += 0x9E3779B9u;
        key1 += 0xBB67AE85u;
    }
}

// Walks the radix tree of the keys, most significant byte first, to the key at which the
// running total (of counts, or of fixed-point mass), taken over keys in descending order,
// first goes beyond `target` (counts: reaches it).  Returns false if it never does.
template <bool MASS>
__device__ bool radix_descend(const float* __restrict__ row, int vocab, float row_max, float inv_t,
                              unsigned long long target, unsigned long long* hist, uint32_t* shared_sel,
                              uint32_t* result_key) {
    uint32_t prefix = 0, prefix_mask = 0;
    unsigned long long above = 0;
    for (int level = 0; level < 4; ++level) {
        const int shift = 24 - 8 * level;
        for (int b = threadIdx.x; b < 256; b += blockDim.x) hist[b] = 0ull;
        __syncthreads();
        for (int i = threadIdx.x; i < vocab; i += blockDim.x) {
            const float v = row[i];
            const uint32_t key = sortable_key(v);
            if ((key & prefix_mask) == prefix) {
                unsigned long long w = 1ull;
                if (MASS) w = static_cast<unsigned long long>(static_cast<double>(expf((v - row_max) * inv_t)) * kFixedOne);
                atomicAdd(&hist[(key >> shift) & 255u], w);
            }
        }
        __syncthreads();
        if (threadIdx.x == 0) {
            unsigned long long cum = above;
            int sel = -1;
            for (int b = 255; b >= 0; --b) {
                const unsigned long long next = cum + hist[b];
                if (MASS ? next > target : next >= target) {
                    sel = b;
                    break;
                }
                cum = next;
            }
            shared_sel[0] = static_cast<uint32_t>(sel);
            reinterpret_cast<unsigned long long*>(shared_sel + 2)[0] = cum;
        }
        __syncthreads();
        const int sel = static_cast<int>(shared_sel[0]);
        above = reinterpret_cast<unsigned long long*>(shared_sel + 2)[0];
        __syncthreads();
        if (sel < 0) return false;
        prefix |= static_cast<uint32_t>(sel) << shift;
        prefix_mask |= 255u << shift;
    }
    *result_key = prefix;
    return true;
}

__global__ void __launch_bounds__(kSampleThreads)
sample_rows_kernel(float* __restrict__ logits, const float* __restrict__ params, const long long* __restrict__ seeds,
                   const int* __restrict__ penalty_ids, const int* __restrict__ penalty_offsets,
                   int* __restrict__ out_tokens, float* __restrict__ out_logprobs, int vocab) {
    __shared__ unsigned long long hist[256];
    __shared__ unsigned long long scan[kSampleThreads / kWave];
    __shared__ float red_v[kSampleThreads / kWave];
    __shared__ int red_i[kSampleThreads / kWave];
    __shared__ __align__(8) uint32_t sel_s[4];
    __shared__ int found_s;
    const int r = blockIdx.x, tid = threadIdx.x, lane = tid % kWave, wave = tid / kWave;
    constexpr int kWavesHere = kSampleThreads / kWave;
    float* row = logits + static_cast<size_t>(r) * vocab;
    const float temperature = params[r * 5 + 0];
    const int top_k = static_cast<int>(params[r * 5 + 1]);
    const float top_p = params[r * 5 + 2], min_p = params[r * 5 + 3], penalty = params[r * 5 + 4];

    // repetition penalty, in place; the ids of a row are distinct
    if (penalty_ids && penalty != 1.0f) {
        for (int j = penalty_offsets[r] + tid; j < penalty_offsets[r + 1]; j += blockDim.x) {
            const int id = penalty_ids[j];
            if (id >= 0 && id < vocab) {
                const float v = row[id];
                row[id] = v > 0.f ? v / penalty : v * penalty;
            }
        }
        __syncthreads();
    }

    // maximum and its lowest index
    float bv = -INFINITY;
    int bi = 0x7fffffff;
    for (int i = tid; i < vocab; i += blockDim.x) {
        const float v = row[i];
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
    if (lane == 0) {
        red_v[wave] = bv;
        red_i[wave] = bi;
    }
    __syncthreads();
    bv = red_v[0];
    bi = red_i[0];
    for (int w = 1; w < kWavesHere; ++w)
        if (red_v[w] > bv || (red_v[w] == bv && red_i[w] < bi)) {
            bv = red_v[w];
            bi = red_i[w];
        }
    __syncthreads();
    const float row_max = bv;
    const int arg_max = bi == 0x7fffffff ? 0 : bi;
    const bool greedy = temperature == 0.0f;
    const float inv_t = greedy ? 1.0f : 1.0f / fmaxf(temperature, 1e-5f);

    // normaliser of the whole (scaled) distribution, in fixed point
    unsigned long long part = 0;
    for (int i = tid; i < vocab; i += blockDim.x)
        part += static_cast<unsigned long long>(static_cast<double>(expf((row[i] - row_max) * inv_t)) * kFixedOne);
#pragma unroll
    for (int off = kWave / 2; off > 0; off >>= 1) part += __shfl_xor(part, off, kWave);
    if (lane == 0) scan[wave] = part;
    __syncthreads();
    unsigned long long z_fixed = 0;
    for (int w = 0; w < kWavesHere; ++w) z_fixed += scan[w];
    __syncthreads();
    const float log_z = static_cast<float>(log(static_cast<double>(z_fixed) / kFixedOne));

    if (greedy) {
        if (tid == 0) {
            out_tokens[r] = arg_max;
            out_logprobs[r] = -log_z;      // (max - max) * 1 - log Z
        }
        return;
    }

    // thresholds of the truncations, as keys
    const uint32_t max_key = sortable_key(row_max);
    uint32_t k_key = 0;          // keep key >= k_key
    uint32_t p_key = 0;          // keep key >  p_key
    bool k_on = top_k > 0 && top_k < vocab, p_on = top_p < 1.0f;
    if (k_on) k_on = radix_descend<false>(row, vocab, row_max, inv_t, static_cast<unsigned long long>(top_k), hist, sel_s, &k_key);
    if (p_on) {
        const unsigned long long target = static_cast<unsigned long long>(static_cast<double>(top_p) * static_cast<double>(z_fixed));
        p_on = radix_descend<true>(row, vocab, row_max, inv_t, target, hist, sel_s, &p_key);
    }
    const bool mp_on = min_p > 0.0f;

    // mass kept, per thread over a contiguous range of indices, then the draw
    const int chunk = (vocab + kSampleThreads - 1) / kSampleThreads;
    const int begin = min(vocab, tid * chunk), end = min(vocab, begin + chunk);
    auto kept_mass = [&](int i) -> unsigned long long {
        const float v = row[i];
        const uint32_t key = sortable_key(v);
        const float e = expf((v - row_max) * inv_t);
        const bool keep = key == max_key || ((!k_on || key >= k_key) && (!p_on || key > p_key) && (!mp_on || e >= min_p));
        return keep ? static_cast<unsigned long long>(static_cast<double>(e) * kFixedOne) : 0ull;
    };
    unsigned long long mine = 0;
    for (int i = begin; i < end; ++i) mine += kept_mass(i);
    // exclusive scan over the threads
    unsigned long long incl = mine;
#pragma unroll
    for (int off = 1; off < kWave; off <<= 1) {
        const unsigned long long o = __shfl_up(incl, off, kWave);
        if (lane >= off) incl += o;
    }
    if (lane == kWave - 1) scan[wave] = incl;
    __syncthreads();
    unsigned long long wave_base = 0, total = 0;
    for (int w = 0; w < kWavesHere; ++w) {
        if (w < wave) wave_base += scan[w];
        total += scan[w];
    }
    const unsigned long long excl = wave_base + incl - mine;

    uint32_t ctr[4] = {static_cast<uint32_t>(seeds[r * 2 + 1]), static_cast<uint32_t>(seeds[r * 2 + 1] >> 32), 0u, 0u};
    philox4x32_10(ctr, static_cast<uint32_t>(seeds[r * 2]), static_cast<uint32_t>(seeds[r * 2] >> 32));
    const double u = static_cast<double>(((static_cast<unsigned long long>(ctr[0]) << 32) | ctr[1]) >> 11) * (1.0 / 9007199254740992.0);
    unsigned long long target = static_cast<unsigned long long>(u * static_cast<double>(total));
    if (target >= total) target = total - 1;
    if (tid == 0) found_s = -1;
    __syncthreads();
    if (mine > 0 && target >= excl && target < excl + mine) {
        unsigned long long cum = excl;
        int tok = begin;
        for (int i = begin; i < end; ++i) {
            const unsigned long long w = kept_mass(i);
            if (w > 0 && target < cum + w) {
                tok = i;
                break;
            }
            cum += w;
        }
        found_s = tok;
    }
    __syncthreads();
    if (tid == 0) {
        const int tok = found_s >= 0 ? found_s : arg_max;
        out_tokens[r] = tok;
        out_logprobs[r] = (row[tok] - row_max) * inv_t - log_z;
    }
}

// ---- the same sampler with a row spread over many workgroups -------------------------------------
// One workgroup per row leaves most of the chip idle when a decode step has a few rows of a large
// vocabulary: a pass over 256,000 logits with an exponential each takes one compute unit about
// 60 us.  Here a row is cut into kSampleSegments contiguous segments, one workgroup each, and the
// passes become kernels; what the segments of a row have to agree on goes through a scratch area
// per row in integer sums, so every number is the one the kernel above computes and the token is
// the same.  Kernels: prepare (zero the scratch, maximum per segment), histogram level 0 (which
// also gives the normaliser), levels 1 to 3 (only when a row has top-k or top-p), kept mass per
// segment, draw.
constexpr int kSampleSegments = 32;
constexpr int kSegmentThreads = 256;
constexpr int kHistWords = 2 * 4 * 256;                  // [counts | mass][level][byte]
constexpr int kRowWords = kHistWords + kSampleSegments   // kept mass per segment
                          + kSampleSegments              // maximum per segment: (index << 32) | float bits
                          + 8;                           // thresholds and normaliser for the draw
typedef unsigned long long u64;

struct RowSetup {
    float temperature, top_p, min_p, inv_t, row_max;
    int top_k, arg_max;
    bool greedy;
};

__device__ __forceinline__ int segment_length(int vocab) {
    return (((vocab + kSampleSegments - 1) / kSampleSegments) + 3) & ~3;
}

__device__ __forceinline__ RowSetup row_setup(const float* __restrict__ params, const u64* __restrict__ row_ws, int r) {
    RowSetup rs;
    rs.temperature = params[r * 5 + 0];
    rs.top_k = static_cast<int>(params[r * 5 + 1]);
    rs.top_p = params[r * 5 + 2];
    rs.min_p = params[r * 5 + 3];
    rs.greedy = rs.temperature == 0.0f;
    rs.inv_t = rs.greedy ? 1.0f : 1.0f / fmaxf(rs.temperature, 1e-5f);
    // the segments' maxima, in index order: the largest value, the lowest index among equals
    float bv = -INFINITY;
    int bi = 0x7fffffff;
    const u64* seg_max = row_ws + kHistWords + kSampleSegments;
    for (int sgm = 0; sgm < kSampleSegments; ++sgm) {
        const u64 w = seg_max[sgm];
        const float v = __uint_as_float(static_cast<uint32_t>(w));
        const int i = static_cast<int>(w >> 32);
        if (v > bv || (v == bv && i < bi)) {
            bv = v;
            bi = i;
        }
    }
    rs.row_max = bv;
    rs.arg_max = bi == 0x7fffffff ? 0 : bi;
    return rs;
}

__device__ __forceinline__ u64 fixed_mass(float v, float row_max, float inv_t) {
    return static_cast<u64>(static_cast<double>(expf((v - row_max) * inv_t)) * kFixedOne);
}

// One level of `radix_descend`, by a wavefront alone: the bin (descending) at which the running
// total first goes beyond `target` (counts: reaches it), and the total above it.
template <bool MASS>
__device__ __forceinline__ bool descend_level(const u64* __restrict__ hist, u64 target, u64& above, int& sel) {
    const int lane = threadIdx.x % kWave;
    u64 c[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) c[j] = hist[255 - 4 * lane - j];
    const u64 mine = c[0] + c[1] + c[2] + c[3];
    u64 incl = mine;
#pragma unroll
    for (int off = 1; off < kWave; off <<= 1) {
        const u64 o = __shfl_up(incl, off, kWave);
        if (lane >= off) incl += o;
    }
    u64 cum = above + incl - mine;
    int found = -1;
    u64 found_above = 0;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const u64 next = cum + c[j];
        if (found < 0 && (MASS ? next > target : next >= target)) {
            found = 255 - 4 * lane - j;
            found_above = cum;
        }
        cum = next;
    }
    const u64 hits = __ballot(found >= 0);
    if (hits == 0) return false;
    const int first = __ffsll(static_cast<long long>(hits)) - 1;
    sel = __shfl(found, first, kWave);
    above = __shfl(found_above, first, kWave);
    return true;
}

// The prefix of the threshold key after `levels` levels; false when the running total never gets there.
template <bool MASS>
__device__ __forceinline__ bool descend(const u64* __restrict__ hist4, int levels, u64 target, uint32_t& prefix,
                                        uint32_t& mask) {
    prefix = 0;
    mask = 0;
    u64 above = 0;
    for (int level = 0; level < levels; ++level) {
        int sel = -1;
        if (!descend_level<MASS>(hist4 + level * 256, target, above, sel)) return false;
        const int shift = 24 - 8 * level;
        prefix |= static_cast<uint32_t>(sel) << shift;
        mask |= 255u << shift;
    }
    return true;
}

__device__ __forceinline__ u64 wave_sum(u64 v) {
#pragma unroll
    for (int off = kWave / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, kWave);
    return v;
}

// The normaliser: every element is in the level-0 histogram of mass.
__device__ __forceinline__ u64 normaliser(const u64* __restrict__ row_ws) {
    const int lane = threadIdx.x % kWave;
    const u64* h = row_ws + 4 * 256;
    return wave_sum(h[lane] + h[lane + 64] + h[lane + 128] + h[lane + 192]);
}

__global__ void sample_penalty_kernel(float* __restrict__ logits, const float* __restrict__ params,
                                      const int* __restrict__ penalty_ids, const int* __restrict__ penalty_offsets,
                                      int vocab) {
    const int r = blockIdx.x;
    const float penalty = params[r * 5 + 4];
    if (penalty == 1.0f) return;
    float* row = logits + static_cast<size_t>(r) * vocab;
    for (int j = penalty_offsets[r] + threadIdx.x; j < penalty_offsets[r + 1]; j += blockDim.x) {
        const int id = penalty_ids[j];
        if (id >= 0 && id < vocab) {
            const float v = row[id];
            row[id] = v > 0.f ? v / penalty : v * penalty;
        }
    }
}

// Visits the elements of the workgroup's segment, four consecutive ones a thread at a time.
template <typename F>
__device__ __forceinline__ void for_segment(const float* __restrict__ row, int vocab, F&& f) {
    const int len = segment_length(vocab);
    const int begin = min(vocab, static_cast<int>(blockIdx.x) * len), end = min(vocab, begin + len);
    const bool vec = vocab % 4 == 0;        // then rows and segments begin at multiples of 16 bytes
    for (int i = begin + 4 * threadIdx.x; i < end; i += 4 * blockDim.x) {
        float v[4];
        if (vec) {
            const float4 q = *reinterpret_cast<const float4*>(row + i);
            v[0] = q.x; v[1] = q.y; v[2] = q.z; v[3] = q.w;
        } else {
#pragma unroll
            for (int e = 0; e < 4; ++e) v[e] = i + e < end ? row[i + e] : 0.f;
        }
#pragma unroll
        for (int e = 0; e < 4; ++e)
            if (i + e < end) f(i + e, v[e]);
    }
}

__global__ void __launch_bounds__(kSegmentThreads)
sample_prepare_kernel(const float* __restrict__ logits, u64* __restrict__ ws, int vocab) {
    __shared__ float red_v[kSegmentThreads / kWave];
    __shared__ int red_i[kSegmentThreads / kWave];
    const int r = blockIdx.y, sgm = blockIdx.x, tid = threadIdx.x;
    u64* row_ws = ws + static_cast<size_t>(r) * kRowWords;
    for (int j = tid; j < kHistWords / kSampleSegments; j += blockDim.x) row_ws[sgm * (kHistWords / kSampleSegments) + j] = 0ull;
    float bv = -INFINITY;
    int bi = 0x7fffffff;
    for_segment(logits + static_cast<size_t>(r) * vocab, vocab, [&](int i, float v) { argmax_take(v, i, bv, bi); });
    argmax_wave(bv, bi);
    if (tid % kWave == 0) {
        red_v[tid / kWave] = bv;
        red_i[tid / kWave] = bi;
    }
    __syncthreads();
    if (tid == 0) {
        for (int w = 1; w < kSegmentThreads / kWave; ++w)
            if (red_v[w] > bv || (red_v[w] == bv && red_i[w] < bi)) {
                bv = red_v[w];
                bi = red_i[w];
            }
        row_ws[kHistWords + kSampleSegments + sgm] = (static_cast<u64>(static_cast<uint32_t>(bi)) << 32) | __float_as_uint(bv);
    }
}

// Level `level` of both histograms: counts of keys for top-k, mass for top-p, of the elements whose
// key has the prefix the levels before chose.  Level 0 of the mass always: it holds the normaliser.
__global__ void __launch_bounds__(kSegmentThreads)
sample_histogram_kernel(const float* __restrict__ logits, const float* __restrict__ params, u64* __restrict__ ws,
                        int vocab, int level) {
    __shared__ u64 hist[2][256];
    const int r = blockIdx.y, tid = threadIdx.x;
    u64* row_ws = ws + static_cast<size_t>(r) * kRowWords;
    const RowSetup rs = row_setup(params, row_ws, r);
    bool k_on = !rs.greedy && rs.top_k > 0 && rs.top_k < vocab, p_on = !rs.greedy && rs.top_p < 1.0f;
    if (level > 0 && !k_on && !p_on) return;
    uint32_t k_prefix = 0, k_mask = 0, p_prefix = 0, p_mask = 0;
    if (level > 0) {
        if (k_on) k_on = descend<false>(row_ws, level, static_cast<u64>(rs.top_k), k_prefix, k_mask);
        if (p_on) {
            const u64 z = normaliser(row_ws);
            const u64 target = static_cast<u64>(static_cast<double>(rs.top_p) * static_cast<double>(z));
            p_on = descend<true>(row_ws + 4 * 256, level, target, p_prefix, p_mask);
        }
        if (!k_on && !p_on) return;
    }
    const bool mass_on = level == 0 || p_on;
    hist[0][tid] = 0ull;
    hist[1][tid] = 0ull;
    __syncthreads();
    const int shift = 24 - 8 * level;
    for_segment(logits + static_cast<size_t>(r) * vocab, vocab, [&](int, float v) {
        const uint32_t key = sortable_key(v);
        const int bin = (key >> shift) & 255u;
        if (k_on && (key & k_mask) == k_prefix) atomicAdd(&hist[0][bin], 1ull);
        if (mass_on && (key & p_mask) == p_prefix) atomicAdd(&hist[1][bin], fixed_mass(v, rs.row_max, rs.inv_t));
    });
    __syncthreads();
#pragma unroll
    for (int kind = 0; kind < 2; ++kind) {
        const u64 v = hist[kind][tid];
        if (v) atomicAdd(row_ws + (kind * 4 + level) * 256 + tid, v);
    }
}

// The thresholds from the finished histograms, and the mass each segment keeps.
__global__ void __launch_bounds__(kSegmentThreads)
sample_kept_kernel(const float* __restrict__ logits, const float* __restrict__ params, u64* __restrict__ ws, int vocab) {
    __shared__ u64 part_s[kSegmentThreads / kWave];
    const int r = blockIdx.y, sgm = blockIdx.x, tid = threadIdx.x;
    u64* row_ws = ws + static_cast<size_t>(r) * kRowWords;
    const RowSetup rs = row_setup(params, row_ws, r);
    const u64 z = normaliser(row_ws);
    u64* out_words = row_ws + kHistWords + 2 * kSampleSegments;
    if (rs.greedy) {
        if (sgm == 0 && tid == 0) out_words[2] = z;
        return;
    }
    bool k_on = rs.top_k > 0 && rs.top_k < vocab, p_on = rs.top_p < 1.0f;
    uint32_t k_key = 0, p_key = 0, mask = 0;
    if (k_on) k_on = descend<false>(row_ws, 4, static_cast<u64>(rs.top_k), k_key, mask);
    if (p_on) {
        const u64 target = static_cast<u64>(static_cast<double>(rs.top_p) * static_cast<double>(z));
        p_on = descend<true>(row_ws + 4 * 256, 4, target, p_key, mask);
    }
    const bool mp_on = rs.min_p > 0.0f;
    const uint32_t max_key = sortable_key(rs.row_max);
    u64 mine = 0;
    for_segment(logits + static_cast<size_t>(r) * vocab, vocab, [&](int, float v) {
        const uint32_t key = sortable_key(v);
        const float e = expf((v - rs.row_max) * rs.inv_t);
        const bool keep = key == max_key || ((!k_on || key >= k_key) && (!p_on || key > p_key) && (!mp_on || e >= rs.min_p));
        if (keep) mine += static_cast<u64>(static_cast<double>(e) * kFixedOne);
    });
    mine = wave_sum(mine);
    if (tid % kWave == 0) part_s[tid / kWave] = mine;
    __syncthreads();
    if (tid == 0) {
        u64 total = 0;
        for (int w = 0; w < kSegmentThreads / kWave; ++w) total += part_s[w];
        row_ws[kHistWords + sgm] = total;
        if (sgm == 0) {
            out_words[0] = k_on ? (1ull << 32) | k_key : 0ull;
            out_words[1] = p_on ? (1ull << 32) | p_key : 0ull;
            out_words[2] = z;
        }
    }
}

// The draw: the segment that holds the target, then, within it, the thread and the element, all in
// index order.
__global__ void __launch_bounds__(kSampleThreads)
sample_draw_kernel(const float* __restrict__ logits, const float* __restrict__ params, const long long* __restrict__ seeds,
                   const u64* __restrict__ ws, int* __restrict__ out_tokens, float* __restrict__ out_logprobs, int vocab) {
    __shared__ u64 scan[kSampleThreads / kWave];
    __shared__ int found_s;
    const int r = blockIdx.x, tid = threadIdx.x, lane = tid % kWave, wave = tid / kWave;
    constexpr int kWavesHere = kSampleThreads / kWave;
    const float* row = logits + static_cast<size_t>(r) * vocab;
    const u64* row_ws = ws + static_cast<size_t>(r) * kRowWords;
    const RowSetup rs = row_setup(params, row_ws, r);
    const u64* words = row_ws + kHistWords + 2 * kSampleSegments;
    const u64 z_fixed = words[2];
    const float log_z = static_cast<float>(log(static_cast<double>(z_fixed) / kFixedOne));
    if (rs.greedy) {
        if (tid == 0) {
            out_tokens[r] = rs.arg_max;
            out_logprobs[r] = -log_z;
        }
        return;
    }
    const bool k_on = (words[0] >> 32) != 0, p_on = (words[1] >> 32) != 0, mp_on = rs.min_p > 0.0f;
    const uint32_t k_key = static_cast<uint32_t>(words[0]), p_key = static_cast<uint32_t>(words[1]);
    const uint32_t max_key = sortable_key(rs.row_max);
    const u64* seg_kept = row_ws + kHistWords;
    u64 total = 0;
    for (int sgm = 0; sgm < kSampleSegments; ++sgm) total += seg_kept[sgm];

    uint32_t ctr[4] = {static_cast<uint32_t>(seeds[r * 2 + 1]), static_cast<uint32_t>(seeds[r * 2 + 1] >> 32), 0u, 0u};
    philox4x32_10(ctr, static_cast<uint32_t>(seeds[r * 2]), static_cast<uint32_t>(seeds[r * 2] >> 32));
    const double u = static_cast<double>(((static_cast<u64>(ctr[0]) << 32) | ctr[1]) >> 11) * (1.0 / 9007199254740992.0);
    u64 target = static_cast<u64>(u * static_cast<double>(total));
    if (target >= total) target = total - 1;
    // the segment whose interval holds the target
    int sgm = 0;
    u64 seg_base = 0;
    for (; sgm < kSampleSegments - 1; ++sgm) {
        if (target < seg_base + seg_kept[sgm]) break;
        seg_base += seg_kept[sgm];
    }
    const int len = segment_length(vocab);
    const int seg_begin = min(vocab, sgm * len), seg_end = min(vocab, seg_begin + len);
    const int chunk = (len + kSampleThreads - 1) / kSampleThreads;
    const int begin = min(seg_end, seg_begin + tid * chunk), end = min(seg_end, begin + chunk);
    auto kept_mass = [&](int i) -> u64 {
        const float v = row[i];
        const uint32_t key = sortable_key(v);
        const float e = expf((v - rs.row_max) * rs.inv_t);
        const bool keep = key == max_key || ((!k_on || key >= k_key) && (!p_on || key > p_key) && (!mp_on || e >= rs.min_p));
        return keep ? static_cast<u64>(static_cast<double>(e) * kFixedOne) : 0ull;
    };
    u64 mine = 0;
    for (int i = begin; i < end; ++i) mine += kept_mass(i);
    u64 incl = mine;
#pragma unroll
    for (int off = 1; off < kWave; off <<= 1) {
        const u64 o = __shfl_up(incl, off, kWave);
        if (lane >= off) incl += o;
    }
    if (lane == kWave - 1) scan[wave] = incl;
    if (tid == 0) found_s = -1;
    __syncthreads();
    u64 wave_base = seg_base;
    for (int w = 0; w < wave; ++w) wave_base += scan[w];
    const u64 excl = wave_base + incl - mine;
    if (mine > 0 && target >= excl && target < excl + mine) {
        u64 cum = excl;
        int tok = begin;
        for (int i = begin; i < end; ++i) {
            const u64 w = kept_mass(i);
            if (w > 0 && target < cum + w) {
                tok = i;
                break;
            }
            cum += w;
        }
        found_s = tok;
    }
    __syncthreads();
    if (tid == 0) {
        const int tok = found_s >= 0 ? found_s : rs.arg_max;
        out_tokens[r] = tok;
        out_logprobs[r] = (row[tok] - rs.row_max) * rs.inv_t - log_z;
    }
}

// Words of scratch a row needs in `wllm_sample_rows_split`.
WLLM_API int wllm_sample_split_row_words() { return kRowWords; }

// The launches of the sampler with each row spread over kSampleSegments workgroups; `ws` holds
// rows * kRowWords words on the device.  The prepare kernel clears what must start at zero.
static int launch_sample_rows_split(float* logits, const float* params, const long long* seeds, const int* penalty_ids,
                                    const int* penalty_offsets, int* out_tokens, float* out_logprobs, u64* ws, int rows,
                                    int vocab, int truncations, hipStream_t stream) {
    if (penalty_ids) {
        sample_penalty_kernel<<<rows, 256, 0, stream>>>(logits, params, penalty_ids, penalty_offsets, vocab);
        if (int err = launch_status()) return err;
    }
    const dim3 grid(kSampleSegments, rows);
    sample_prepare_kernel<<<grid, kSegmentThreads, 0, stream>>>(logits, ws, vocab);
    if (int err = launch_status()) return err;
    for (int level = 0; level < (truncations ? 4 : 1); ++level) {
        sample_histogram_kernel<<<grid, kSegmentThreads, 0, stream>>>(logits, params, ws, vocab, level);
        if (int err = launch_status()) return err;
    }
    sample_kept_kernel<<<grid, kSegmentThreads, 0, stream>>>(logits, params, ws, vocab);
    if (int err = launch_status()) return err;
    sample_draw_kernel<<<rows, kSampleThreads, 0, stream>>>(logits, params, seeds, ws, out_tokens, out_logprobs, vocab);
    return launch_status();
}

// The sampler with each row spread over kSampleSegments workgroups.  `workspace` holds rows *
// wllm_sample_split_row_words() 8-byte words; `truncations` says whether any row has top-k or top-p
// (then three more histogram levels run).  Same tokens and log-probabilities as `wllm_sample_rows`.
WLLM_API int wllm_sample_rows_split(float* logits, const float* params, const long long* seeds, const int* penalty_ids,
                                    const int* penalty_offsets, int* out_tokens, float* out_logprobs, void* workspace,
                                    int rows, int vocab, int truncations, hipStream_t stream) {
    if (rows < 1 || vocab < 1 || !workspace) return -1;
    return launch_sample_rows_split(logits, params, seeds, penalty_ids, penalty_offsets, out_tokens, out_logprobs,
                                    static_cast<u64*>(workspace), rows, vocab, truncations, stream);
}

// ---- the same sampler for callers that cannot allocate (wllm_no_alloc.h) -------------------------
// The scratch area is a device array of the library's image.  In host code its name is only a
// handle for the runtime, not a device address: the address of each GPU's copy comes from
// hipGetSymbolAddress, once per device, and only that pointer is ever handed to a kernel.
constexpr int kStaticSampleRows = 64;
constexpr int kStaticMaxDevices = 64;
static __device__ __align__(256) u64 scratch[static_cast<size_t>(kStaticSampleRows) * kRowWords];
static u64* scratch_of_device[kStaticMaxDevices];       // host side: device address of `scratch` per GPU
static std::mutex scratch_lock;

// The current device's copy of `scratch`; resolved at the first call on that device.
static int static_scratch(u64** out) {
    int device = -1;
    if (hipError_t err = hipGetDevice(&device)) return static_cast<int>(err);
    if (device < 0 || device >= kStaticMaxDevices) return static_cast<int>(hipErrorInvalidDevice);
    std::lock_guard<std::mutex> hold(scratch_lock);
    if (!scratch_of_device[device]) {
        void* address = nullptr;
        if (hipError_t err = hipGetSymbolAddress(&address, HIP_SYMBOL(scratch))) return static_cast<int>(err);
        if (!address) return static_cast<int>(hipErrorInvalidSymbol);
        scratch_of_device[device] = static_cast<u64*>(address);
    }
    *out = scratch_of_device[device];
    return 0;
}

WLLM_NO_ALLOC_API int wllm_sample_static_max_rows(void) { return kStaticSampleRows; }

WLLM_NO_ALLOC_API int wllm_sample_static_init(void) {
    u64* ws = nullptr;
    return static_scratch(&ws);
}

WLLM_NO_ALLOC_API const char* wllm_sample_static_error(int code) {
    switch (code) {
        case 0: return "success";
        case WLLM_STATIC_BAD_ARGUMENT: return "wllm_sample_rows_static: rows < 1, vocab < 1 or a null pointer";
        case WLLM_STATIC_TOO_MANY_ROWS: return "wllm_sample_rows_static: more rows than wllm_sample_static_max_rows() (64)";
        default: return code > 0 ? hipGetErrorString(static_cast<hipError_t>(code)) : "wllm_sample_rows_static: unknown error code";
    }
}

WLLM_NO_ALLOC_API int wllm_sample_rows_static(float* logits, const float* params, const long long* seeds,
                                              const int* penalty_ids, const int* penalty_offsets, int* out_tokens,
                                              float* out_logprobs, int rows, int vocab, int truncations,
                                              hipStream_t stream) {
    if (rows < 1 || vocab < 1 || !logits || !params || !seeds || !out_tokens || !out_logprobs) return WLLM_STATIC_BAD_ARGUMENT;
    if ((penalty_ids == nullptr) != (penalty_offsets == nullptr)) return WLLM_STATIC_BAD_ARGUMENT;
    if (rows > kStaticSampleRows) return WLLM_STATIC_TOO_MANY_ROWS;
    u64* ws = nullptr;
    if (int err = static_scratch(&ws)) return err;
    return launch_sample_rows_split(logits, params, seeds, penalty_ids, penalty_offsets, out_tokens, out_logprobs, ws,
                                    rows, vocab, truncations, stream);
}

WLLM_API int wllm_sample_rows(float* logits, const float* params, const long long* seeds, const int* penalty_ids,
                              const int* penalty_offsets, int* out_tokens, float* out_logprobs, int rows, int vocab,
                              hipStream_t stream) {
    sample_rows_kernel<<<rows, kSampleThreads, 0, stream>>>(logits, params, seeds, penalty_ids, penalty_offsets,
                                                            out_tokens, out_logprobs, vocab);
    return launch_status();
}
