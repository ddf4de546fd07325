// Embedding lookup, RMS norm with residual add, rotation with cache write, gated
// activation.  Each is bound by memory traffic; the fusions are the ones that save
// a pass over the residual stream or over the q/k/v rows.
#include "common.h"

// ---- embedding: out[i] = float(table[ids[i]]) * scale ---------------------------------
template <typename T>
__global__ void embed_lookup_kernel(const int* __restrict__ ids, const T* __restrict__ table, float scale,
                                    float* __restrict__ out, int hidden, int vocab) {
    const int row = blockIdx.x;
    int id = ids[row];
    // ids are checked on the host; clamp all the same so that a bad id cannot fault
    id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);
    const T* src = table + static_cast<size_t>(id) * hidden;
    float* dst = out + static_cast<size_t>(row) * hidden;
    for (int i = threadIdx.x; i < hidden; i += blockDim.x) dst[i] = to_float(src[i]) * scale;
}

template <typename T>
static int embed_lookup_launch(const int* ids, const void* table, float scale, float* out, int n, int hidden,
                               int vocab, hipStream_t stream) {
    embed_lookup_kernel<T><<<n, 256, 0, stream>>>(ids, static_cast<const T*>(table), scale, out, hidden, vocab);
    return launch_status();
}

WLLM_API int wllm_embed_lookup(const int* ids, const void* table, int is_bf16, float scale, float* out, int n,
                               int hidden, int vocab, hipStream_t stream) {
    return is_bf16 ? embed_lookup_launch<bf16>(ids, table, scale, out, n, hidden, vocab, stream)
                   : embed_lookup_launch<float>(ids, table, scale, out, n, hidden, vocab, stream);
}

// ---- token ids that come from the device: ids[dst[j]] = source[src[j]] for every j with dst[j] >= 0.
// A step that is started before the step before it has been read takes the tokens that step sampled
// straight from its output, without a trip through the host.
__global__ void feed_tokens_kernel(int* __restrict__ ids, const int* __restrict__ dst, const int* __restrict__ src,
                                   const int* __restrict__ source, int count, int num_ids, int num_source) {
    const int j = blockIdx.x * blockDim.x + threadIdx.x;
    if (j >= count) return;
    const int d = dst[j], s = src[j];
    if (d >= 0 && d < num_ids && s >= 0 && s < num_source) ids[d] = source[s];
}

WLLM_API int wllm_feed_tokens(int* ids, const int* dst, const int* src, const int* source, int count, int num_ids,
                              int num_source, hipStream_t stream) {
    if (count <= 0) return 0;
    feed_tokens_kernel<<<(count + 255) / 256, 256, 0, stream>>>(ids, dst, src, source, count, num_ids, num_source);
    return launch_status();
}

// ---- RMS norm: out = v * rsqrt(mean(v^2) + eps) * (offset + w), v = x (+ delta) ------------
// One workgroup per output row.  Without `rows` the sum x + delta is written back to x.  `delta`
// may be a stack of `splits` partial sums (a product split over K), `split_stride` elements apart;
// they are added in stack order.
__device__ __forceinline__ float delta_value(const bf16* p, int, size_t) { return to_float(*p); }
__device__ __forceinline__ float delta_value(const float* p, int splits, size_t stride) {
    return splits > 1 ? stack_sum(p, splits, stride) : *p;
}

constexpr int kNormPerThread = 8;    // elements a thread may keep in registers between the passes

template <typename TD, typename TO>
__global__ void rms_norm_kernel(float* __restrict__ x, const TD* __restrict__ delta, int splits, size_t split_stride,
                                const float* __restrict__ weight, const int* __restrict__ rows, TO* __restrict__ out,
                                int hidden, float eps, float offset) {
    __shared__ float scratch[16];
    const int orow = blockIdx.x;
    const int irow = rows ? rows[orow] : orow;
    float* xr = x + static_cast<size_t>(irow) * hidden;
    const TD* dr = delta ? delta + static_cast<size_t>(irow) * hidden : nullptr;
    TO* o = out + static_cast<size_t>(orow) * hidden;
    const bool in_registers = hidden <= static_cast<int>(blockDim.x) * kNormPerThread;
    float keep[kNormPerThread];
    float ss = 0.f;
    if (in_registers) {
#pragma unroll
        for (int e = 0; e < kNormPerThread; ++e) {
            const int i = threadIdx.x + e * blockDim.x;
            float v = 0.f;
            if (i < hidden) {
                v = xr[i];
                if (dr) {
                    v += delta_value(dr + i, splits, split_stride);
                    if (!rows) xr[i] = v;
                }
            }
            keep[e] = v;
            ss += v * v;
        }
    } else {
        for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
            float v = xr[i];
            if (dr) {
                v += delta_value(dr + i, splits, split_stride);
                if (!rows) xr[i] = v;
            }
            ss += v * v;
        }
    }
    ss = block_sum(ss, scratch);
    const float inv = rsqrtf(ss / static_cast<float>(hidden) + eps);
    if (in_registers) {
#pragma unroll
        for (int e = 0; e < kNormPerThread; ++e) {
            const int i = threadIdx.x + e * blockDim.x;
            if (i < hidden) o[i] = from_float<TO>(keep[e] * inv * (offset + weight[i]));
        }
    } else {
        for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
            float v = xr[i];
            if (dr && rows) v += delta_value(dr + i, splits, split_stride);
            o[i] = from_float<TO>(v * inv * (offset + weight[i]));
        }
    }
}

// The same with 16-byte accesses, for a width that is a multiple of 4 and fits the registers: a
// thread keeps up to kNormGroups groups of 4 consecutive elements.
constexpr int kNormGroups = 2;

template <typename T> struct alignas(4 * sizeof(T)) Quad { T v[4]; };

template <typename TD, typename TO>
__global__ void rms_norm_vec_kernel(float* __restrict__ x, const TD* __restrict__ delta, int splits,
                                    size_t split_stride, const float* __restrict__ weight,
                                    const int* __restrict__ rows, TO* __restrict__ out, int hidden, float eps,
                                    float offset) {
    __shared__ float scratch[16];
    const int orow = blockIdx.x;
    const int irow = rows ? rows[orow] : orow;
    float* xr = x + static_cast<size_t>(irow) * hidden;
    const TD* dr = delta ? delta + static_cast<size_t>(irow) * hidden : nullptr;
    TO* o = out + static_cast<size_t>(orow) * hidden;
    Quad<float> keep[kNormGroups], w[kNormGroups];
    float ss = 0.f;
    // the norm's weights are asked for with everything else, not after the sum of squares
#pragma unroll
    for (int e = 0; e < kNormGroups; ++e) {
        const int i = (threadIdx.x + e * blockDim.x) * 4;
        w[e] = i < hidden ? *reinterpret_cast<const Quad<float>*>(weight + i) : Quad<float>{{0.f, 0.f, 0.f, 0.f}};
    }
#pragma unroll
    for (int e = 0; e < kNormGroups; ++e) {
        const int i = (threadIdx.x + e * blockDim.x) * 4;
        Quad<float> v = {{0.f, 0.f, 0.f, 0.f}};
        if (i < hidden) {
            v = *reinterpret_cast<const Quad<float>*>(xr + i);
            if (dr) {
                // the partial sums of a stack are added in stack order, then their sum to x
                const int stack = (sizeof(TD) == sizeof(float) && splits > 1) ? splits : 1;
                Quad<float> d = {{0.f, 0.f, 0.f, 0.f}};
                constexpr int kInFlight = 16;
                for (int s0 = 0; s0 < stack; s0 += kInFlight) {
                    Quad<TD> q[kInFlight];       // loads in flight
#pragma unroll
                    for (int j = 0; j < kInFlight; ++j)
                        q[j] = *reinterpret_cast<const Quad<TD>*>(dr + min(s0 + j, stack - 1) * split_stride + i);
#pragma unroll
                    for (int j = 0; j < kInFlight; ++j) {
                        if (s0 + j >= stack) break;
#pragma unroll
                        for (int k = 0; k < 4; ++k) d.v[k] = s0 + j == 0 ? to_float(q[j].v[k]) : d.v[k] + to_float(q[j].v[k]);
                    }
                }
#pragma unroll
                for (int k = 0; k < 4; ++k) v.v[k] += d.v[k];
                if (!rows) *reinterpret_cast<Quad<float>*>(xr + i) = v;
            }
        }
        keep[e] = v;
#pragma unroll
        for (int k = 0; k < 4; ++k) ss += v.v[k] * v.v[k];
    }
    ss = block_sum(ss, scratch);
    const float inv = rsqrtf(ss / static_cast<float>(hidden) + eps);
#pragma unroll
    for (int e = 0; e < kNormGroups; ++e) {
        const int i = (threadIdx.x + e * blockDim.x) * 4;
        if (i < hidden) {
            Quad<TO> r;
#pragma unroll
            for (int k = 0; k < 4; ++k) r.v[k] = from_float<TO>(keep[e].v[k] * inv * (offset + w[e].v[k]));
            *reinterpret_cast<Quad<TO>*>(o + i) = r;
        }
    }
}

WLLM_API int wllm_rms_norm(float* x, const void* delta, int delta_bf16, int splits, long long split_stride,
                           const float* weight, const int* rows, void* out, int out_bf16, int num_out_rows,
                           int hidden, float eps, float offset, hipStream_t stream) {
    if (hidden % 4 == 0 && hidden <= 1024 * 4 * kNormGroups && (splits <= 1 || split_stride % 4 == 0)) {
        const int quads = hidden / 4;
        const int vthreads = quads >= 1024 ? 1024 : ((quads + 63) / 64) * 64;
#define LAUNCH(TD, TO)                                                                                          \
    rms_norm_vec_kernel<TD, TO><<<num_out_rows, vthreads, 0, stream>>>(                                         \
        x, static_cast<const TD*>(delta), splits, static_cast<size_t>(split_stride), weight, rows,             \
        static_cast<TO*>(out), hidden, eps, offset)
        if (delta_bf16 && out_bf16) LAUNCH(bf16, bf16);
        else if (delta_bf16) LAUNCH(bf16, float);
        else if (out_bf16) LAUNCH(float, bf16);
        else LAUNCH(float, float);
#undef LAUNCH
        return launch_status();
    }
    const int threads = hidden >= 4096 ? 1024 : (hidden >= 1024 ? 512 : (hidden >= 256 ? 128 : 64));
#define LAUNCH(TD, TO)                                                                                          \
    rms_norm_kernel<TD, TO><<<num_out_rows, threads, 0, stream>>>(x, static_cast<const TD*>(delta), splits,      \
                                                                  static_cast<size_t>(split_stride), weight, rows, \
                                                                  static_cast<TO*>(out), hidden, eps, offset)
    if (delta_bf16 && out_bf16) LAUNCH(bf16, bf16);
    else if (delta_bf16) LAUNCH(bf16, float);
    else if (out_bf16) LAUNCH(float, bf16);
    else LAUNCH(float, float);
#undef LAUNCH
    return launch_status();
}

// ---- rotation of queries and keys, bias, and the write of keys and values into pages ----------
// One workgroup per token.  A row of qkv is [num_heads | num_kv_heads | num_kv_heads] heads of
// head_dim.  Element j < rotary_dim/2 of a query or key head is paired with j + rotary_dim/2 and
// the pair is turned by position * inv_freq[j]; angle, sine and cosine are float32.  Keys go to
// the cache as [page_size, head_dim], values transposed as [head_dim, page_size].
template <typename T>
__global__ void rope_cache_kernel(T* __restrict__ qkv, const float* __restrict__ parts, int splits, size_t split_stride,
                                  const float* __restrict__ bias, const int* __restrict__ positions,
                                  const float* __restrict__ inv_freq, const int* __restrict__ slots,
                                  T* __restrict__ cache, int num_heads, int num_kv_heads, int head_dim, int rotary_dim,
                                  int page_size, long long num_pages) {
    const int token = blockIdx.x;
    const int width = (num_heads + 2 * num_kv_heads) * head_dim;
    T* row = qkv + static_cast<size_t>(token) * width;
    const float* prow = parts ? parts + static_cast<size_t>(token) * width : nullptr;
    // a value of the projection: the row itself, or the sum of the partial sums of a split product
    auto value = [&](int idx) -> float {
        if (!prow) return to_float(row[idx]);
        return stack_sum(prow + idx, splits, split_stride);
    };
    const bool rewrite = bias || prow;      // every element of the row must be written
    const float pos = static_cast<float>(positions[token]);
    const int half = rotary_dim / 2;
    const size_t page_elems = static_cast<size_t>(2) * num_kv_heads * page_size * head_dim;
    T* kpage = nullptr;
    T* vpage = nullptr;
    int off = 0;
    if (cache) {
        const int slot = slots[token];
        const long long page = slot / page_size;
        off = slot % page_size;
        if (slot >= 0 && page < num_pages) {
            kpage = cache + page * page_elems;
            vpage = kpage + static_cast<size_t>(num_kv_heads) * page_size * head_dim;
        }
    }
    // rotated pairs of query and key heads
    const int rot_heads = num_heads + num_kv_heads;
    // a thread keeps one pair index j and walks the heads, so the sine and cosine of its angle are
    // computed once; threads beyond `half` start at further heads
    const int lanes_j = max(1, min(static_cast<int>(blockDim.x), half));
    const int head_step = max(1, static_cast<int>(blockDim.x) / lanes_j);
    for (int j = threadIdx.x % lanes_j; j < half; j += lanes_j) {
        const int head_first = threadIdx.x / lanes_j;
        if (head_first >= head_step) break;          // threads that do not fit a whole group of heads idle
        float s, c;
        sincosf(pos * inv_freq[j], &s, &c);
        for (int head = head_first; head < rot_heads; head += head_step) {
            const int ia = head * head_dim + j, ib = ia + half;
            float a = value(ia), b = value(ib);
            if (bias) {
                a += bias[ia];
                b += bias[ib];
            }
            float fa, fb;
            rotate_pair(a, b, s, c, fa, fb);
            const T ra = from_float<T>(fa), rb = from_float<T>(fb);
            row[ia] = ra;
            row[ib] = rb;
            if (kpage && head >= num_heads) {
                T* dst = kpage + (static_cast<size_t>(head - num_heads) * page_size + off) * head_dim;
                dst[j] = ra;
                dst[j + half] = rb;
            }
        }
    }
    // the part of query and key heads that is not rotated
    const int rest = head_dim - rotary_dim;
    if (rest > 0 && (rewrite || kpage)) {
        for (int idx = threadIdx.x; idx < rot_heads * rest; idx += blockDim.x) {
            const int head = idx / rest, j = rotary_dim + idx % rest;
            const int i = head * head_dim + j;
            T v = row[i];
            if (rewrite) {
                v = from_float<T>(value(i) + (bias ? bias[i] : 0.f));
                row[i] = v;
            }
            if (kpage && head >= num_heads)
                kpage[(static_cast<size_t>(head - num_heads) * page_size + off) * head_dim + j] = v;
        }
    }
    // values
    if (rewrite || vpage) {
        const int vbase = rot_heads * head_dim;
        for (int idx = threadIdx.x; idx < num_kv_heads * head_dim; idx += blockDim.x) {
            const int head = idx / head_dim, j = idx % head_dim;
            T v = row[vbase + idx];
            if (rewrite) {
                v = from_float<T>(value(vbase + idx) + (bias ? bias[vbase + idx] : 0.f));
                row[vbase + idx] = v;
            }
            if (vpage) vpage[(static_cast<size_t>(head) * head_dim + j) * page_size + off] = v;
        }
    }
}

// The same for the common case (the row holds the projection itself, no bias, every size a multiple
// of 16 bytes): a thread moves 16 bytes at a time.  Sines and cosines of the token's angles are
// computed once into LDS; then each thread takes units of W pairs (W elements at j and W at
// j + rotary_dim/2 of one head), of W unrotated key elements or of W value elements.
template <typename T>
__global__ void rope_cache_vec_kernel(T* __restrict__ qkv, const int* __restrict__ positions,
                                      const float* __restrict__ inv_freq, const int* __restrict__ slots,
                                      T* __restrict__ cache, int num_heads, int num_kv_heads, int head_dim,
                                      int rotary_dim, int page_size, long long num_pages) {
    constexpr int W = 16 / sizeof(T);
    struct alignas(16) Vec { T v[W]; };
    extern __shared__ float sincos_lds[];        // [rotary_dim/2] sines, then as many cosines
    const int token = blockIdx.x;
    const int width = (num_heads + 2 * num_kv_heads) * head_dim;
    T* row = qkv + static_cast<size_t>(token) * width;
    const int half = rotary_dim / 2;
    const float pos = static_cast<float>(positions[token]);
    for (int j = threadIdx.x; j < half; j += blockDim.x) {
        float s, c;
        sincosf(pos * inv_freq[j], &s, &c);
        sincos_lds[j] = s;
        sincos_lds[half + j] = c;
    }
    const size_t page_elems = static_cast<size_t>(2) * num_kv_heads * page_size * head_dim;
    T* kpage = nullptr;
    T* vpage = nullptr;
    int off = 0;
    if (cache) {
        const int slot = slots[token];
        const long long page = slot / page_size;
        off = slot % page_size;
        if (slot >= 0 && page < num_pages) {
            kpage = cache + page * page_elems;
            vpage = kpage + static_cast<size_t>(num_kv_heads) * page_size * head_dim;
        }
    }
    __syncthreads();
    const int rot_heads = num_heads + num_kv_heads;
    const int pair_units = half / W, rest_units = (head_dim - rotary_dim) / W, value_units = head_dim / W;
    const int n_pairs = rot_heads * pair_units;
    const int n_rest = kpage ? num_kv_heads * rest_units : 0;
    const int n_values = vpage ? num_kv_heads * value_units : 0;
    for (int unit = threadIdx.x; unit < n_pairs + n_rest + n_values; unit += blockDim.x) {
        if (unit < n_pairs) {
            const int head = unit / pair_units, j = (unit % pair_units) * W;
            T* pa = row + head * head_dim + j;
            const Vec a = *reinterpret_cast<const Vec*>(pa), b = *reinterpret_cast<const Vec*>(pa + half);
            Vec ra, rb;
#pragma unroll
            for (int i = 0; i < W; ++i) {
                const float s = sincos_lds[j + i], c = sincos_lds[half + j + i];
                const float x = to_float(a.v[i]), y = to_float(b.v[i]);
                float fa, fb;
                rotate_pair(x, y, s, c, fa, fb);
                ra.v[i] = from_float<T>(fa);
                rb.v[i] = from_float<T>(fb);
            }
            *reinterpret_cast<Vec*>(pa) = ra;
            *reinterpret_cast<Vec*>(pa + half) = rb;
            if (kpage && head >= num_heads) {
                T* dst = kpage + (static_cast<size_t>(head - num_heads) * page_size + off) * head_dim + j;
                *reinterpret_cast<Vec*>(dst) = ra;
                *reinterpret_cast<Vec*>(dst + half) = rb;
            }
        } else if (unit < n_pairs + n_rest) {
            const int u = unit - n_pairs;
            const int head = u / rest_units, j = rotary_dim + (u % rest_units) * W;
            const Vec v = *reinterpret_cast<const Vec*>(row + (num_heads + head) * head_dim + j);
            *reinterpret_cast<Vec*>(kpage + (static_cast<size_t>(head) * page_size + off) * head_dim + j) = v;
        } else {
            const int idx = (unit - n_pairs - n_rest) * W;       // element of the row's value part
            const Vec v = *reinterpret_cast<const Vec*>(row + rot_heads * head_dim + idx);
#pragma unroll
            for (int i = 0; i < W; ++i) vpage[static_cast<size_t>(idx + i) * page_size + off] = v.v[i];
        }
    }
}

WLLM_API int wllm_rope_cache_write(void* qkv, int is_bf16, const float* parts, int splits, long long split_stride,
                                   const float* bias, const int* positions, const float* inv_freq, const int* slots,
                                   void* cache, long long num_pages, int n, int num_heads, int num_kv_heads,
                                   int head_dim, int rotary_dim, int page_size, hipStream_t stream) {
    const int pairs = (num_heads + num_kv_heads) * (rotary_dim / 2);
    const int w = is_bf16 ? 8 : 4;          // elements in 16 bytes
    if (!bias && !parts && head_dim % w == 0 && (rotary_dim / 2) % w == 0 && rotary_dim % 2 == 0 &&
        rotary_dim / 2 <= 4096) {
        const int units = (pairs + num_kv_heads * (2 * head_dim - rotary_dim)) / w;
        const int vthreads = units >= 1024 ? 1024 : ((units + 63) / 64) * 64;
        const size_t lds = static_cast<size_t>(rotary_dim) * sizeof(float);
        if (is_bf16)
            rope_cache_vec_kernel<bf16><<<n, vthreads, lds, stream>>>(
                static_cast<bf16*>(qkv), positions, inv_freq, slots, static_cast<bf16*>(cache), num_heads,
                num_kv_heads, head_dim, rotary_dim, page_size, num_pages);
        else
            rope_cache_vec_kernel<float><<<n, vthreads, lds, stream>>>(
                static_cast<float*>(qkv), positions, inv_freq, slots, static_cast<float*>(cache), num_heads,
                num_kv_heads, head_dim, rotary_dim, page_size, num_pages);
        return launch_status();
    }
    const int threads = pairs >= 1024 ? 1024 : (pairs >= 512 ? 512 : 256);
    if (is_bf16)
        rope_cache_kernel<bf16><<<n, threads, 0, stream>>>(static_cast<bf16*>(qkv), parts, splits,
                                                       static_cast<size_t>(split_stride), bias, positions, inv_freq,
                                                       slots, static_cast<bf16*>(cache), num_heads, num_kv_heads,
                                                       head_dim, rotary_dim, page_size, num_pages);
    else
        rope_cache_kernel<float><<<n, threads, 0, stream>>>(static_cast<float*>(qkv), parts, splits,
                                                        static_cast<size_t>(split_stride), bias, positions, inv_freq,
                                                        slots, static_cast<float*>(cache), num_heads, num_kv_heads,
                                                        head_dim, rotary_dim, page_size, num_pages);
    return launch_status();
}

// ---- gated activation: out = act(g) * u with g, u the two halves of a row -----------------------

template <typename T, int ACT>
__global__ void gated_activation_kernel(const T* __restrict__ gate_up, T* __restrict__ out, long long total,
                                        int inter) {
    const long long stride = static_cast<long long>(gridDim.x) * blockDim.x;
    for (long long i = static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x; i < total; i += stride) {
        const long long r = i / inter;
        const int c = static_cast<int>(i % inter);
        const float g = to_float(gate_up[r * 2 * inter + c]);
        const float u = to_float(gate_up[r * 2 * inter + inter + c]);
        out[i] = from_float<T>(activate<ACT>(g) * u);
    }
}

// bfloat16 rows whose halves are multiples of 8: eight values per 16-byte load; a workgroup walks one
// row (blockIdx.y and on), so no thread divides, and the product of the matrix kernel before it is
// read once
template <int ACT>
__global__ void __launch_bounds__(256)
gated_activation_bf16x8_kernel(const bf16* __restrict__ gate_up, bf16* __restrict__ out, int rows, int inter) {
    const int vecs = inter / 8;
    for (int r = blockIdx.y; r < rows; r += gridDim.y) {
        const bf16* src = gate_up + static_cast<size_t>(r) * 2 * inter;
        bf16* dst = out + static_cast<size_t>(r) * inter;
        for (int v = blockIdx.x * 256 + threadIdx.x; v < vecs; v += gridDim.x * 256) {
            const uint4 g4 = load_streamed(src + v * 8);
            const uint4 u4 = load_streamed(src + inter + v * 8);
            const uint32_t gw[4] = {g4.x, g4.y, g4.z, g4.w}, uw[4] = {u4.x, u4.y, u4.z, u4.w};
            uint32_t ow[4];
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const float g0 = __uint_as_float(gw[k] << 16), g1 = __uint_as_float(gw[k] & 0xffff0000u);
                const float u0 = __uint_as_float(uw[k] << 16), u1 = __uint_as_float(uw[k] & 0xffff0000u);
                ow[k] = pack2_bf16(activate<ACT>(g0) * u0, activate<ACT>(g1) * u1);
            }
            *reinterpret_cast<uint4*>(dst + v * 8) = make_uint4(ow[0], ow[1], ow[2], ow[3]);
        }
    }
}

WLLM_API int wllm_gated_activation(const void* gate_up, void* out, int is_bf16, int activation, int n, int inter,
                                   hipStream_t stream) {
    if (activation < 0 || activation >= kActivations) return -1;
    const long long total = static_cast<long long>(n) * inter;
    if (is_bf16 && inter % 8 == 0) {
        const int vecs = inter / 8;
        const dim3 grid(vecs < 2048 ? (vecs + 255) / 256 : 8, n < 16384 ? n : 16384);
        WLLM_BY_ACTIVATION(activation, (gated_activation_bf16x8_kernel<ACT><<<grid, 256, 0, stream>>>(
                                           static_cast<const bf16*>(gate_up), static_cast<bf16*>(out), n, inter)));
        return launch_status();
    }
    long long blocks = (total + 255) / 256;
    if (blocks > 65536) blocks = 65536;
#define LAUNCH(T)                                                                                                   \
    WLLM_BY_ACTIVATION(activation, (gated_activation_kernel<T, ACT><<<static_cast<int>(blocks), 256, 0, stream>>>( \
                                       static_cast<const T*>(gate_up), static_cast<T*>(out), total, inter)))
    if (is_bf16) { LAUNCH(bf16); } else { LAUNCH(float); }
#undef LAUNCH
    return launch_status();
}
