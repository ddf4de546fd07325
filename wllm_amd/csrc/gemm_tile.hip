// out[M, N] = x[M, K] . w[N, K]^T for bfloat16 with a few hundred rows (the prompt portions of a mixed
// step), on the matrix cores, and the gated form out[M, I] = act(x . Wg^T) * (x . Wu^T) with
// w = [Wg; Wu], whose activation and product are made in the registers the sums are in, so that
// only [M, I] is written.
//
// A workgroup of four wavefronts makes a tile of 128 rows of x by 128 rows of w; the wavefronts are
// 2 x 2, each with 64 x 64 of the tile as 4 x 4 products v_mfma_f32_16x16x32_bf16 a step of 32 keys
// (w is the A operand, x the B operand: lane (i, g) ends with four consecutive columns of one output
// row).  In the gated form the tile's 128 rows of w are 64 gate rows and the 64 up rows that belong
// to them, and a wavefront's 64 are 32 and 32.
//
// The K axis is walked in stages of 64 keys.  A stage's tiles of x and w (16 KB each) go from
// memory straight into shared memory (global_load_lds_dwordx4: a wavefront's 64 lanes bring 8 rows
// of 8 chunks of 16 bytes, lane l's chunk to base + 16 l), two stages in turn (four where a compute
// unit has one workgroup), the next ones' loads in flight during this one's products.  Chunk c of row r lies at place c ^ (r % 8) of its row, so
// that the 16 lanes of a fragment read meet 8 different places in each of two passes and no bank
// twice.  A lane's eight source offsets never change; the stage's 128 bytes go into the scalar base.
//
// Few tiles (a down projection: 2,048 columns) leave compute units idle; then the K axis is cut
// into `splits` pieces over workgroups (grid.z) that leave float32 partial sums [splits, M, N] for
// the consumer to add in order.  Every output element is summed over k in ascending order within a
// piece; pieces depend on K and `splits` alone.
//
// Workgroups that share rows of w get indices 8 apart: they are dispatched one after the other to
// the same XCD (workgroup index modulo 8), and all but the first find the tile of w in its L2.
#include "common.h"

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float float4_t __attribute__((ext_vector_type(4)));

constexpr int kTileRows = 128;      // rows of x, and rows of w, a workgroup
constexpr int kStageKeys = 64;
constexpr int kRowBytes = kStageKeys * 2;

union TFrag {
    uint4 u;
    bf16x8_t v;
};

// 16 bytes a lane from base + offset into shared memory at `dst` + 16 * lane.  M0 is put back as it
// was: naming it as clobbered instead makes the compiler wait for every load in flight before the
// next read of shared memory.  The compiler does not see these loads; the kernel waits for them
// itself (s_waitcnt vmcnt(0) and a barrier before a tile is read).
static __device__ __forceinline__ void load_to_shared(const void* base, uint32_t offset, void* dst) {
    const uint32_t lds_address = __builtin_amdgcn_readfirstlane(
        static_cast<uint32_t>(reinterpret_cast<uintptr_t>((__attribute__((address_space(3))) void*)dst)));
    uint32_t saved_m0;
    asm volatile("s_mov_b32 %0, m0\n\ts_mov_b32 m0, %3\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2\n\ts_mov_b32 m0, %0"
                 : "=&s"(saved_m0) : "v"(offset), "s"(base), "s"(lds_address) : "memory");
}


// GATED: 0 plain, 1 + the activation's number for the gated product.  N is the number of rows of w (plain) or of gate rows (gated).
// (Tiles of 256 rows of x with eight wavefronts were no faster: the rate is set by the reads of
// fragments from shared memory, which take as long as the products they feed.)
// STAGES: how many stages' tiles shared memory holds.  Two, and two workgroups a compute unit, as
// a rule; four, one workgroup a compute unit and three stages (96 KB) on their way, where the launch has
// no more workgroups than the machine has compute units (a step of at most 128 rows, a down projection
// of 256): the tiles of w then come from HBM, and the rate is set by how much a compute unit has in
// flight (the gated product of 128 rows: 53 to 29 us).
template <int GATED, int STAGES>
__global__ void __launch_bounds__(256, STAGES == 2 ? 2 : 1)
gemm_tile_kernel(const bf16* __restrict__ x, const bf16* __restrict__ w, bf16* __restrict__ out,
                 float* __restrict__ partial, int M, int N, int K, int m_tiles, int k_per_split) {
    constexpr int kXRows = kTileRows, kWaves = 4;
    constexpr int kWBytes = kTileRows * kRowBytes, kXBytes = kXRows * kRowBytes;
    constexpr int kLoads = (kTileRows + kXRows) / 8 / kWaves;      // loads a wavefront and stage: 8 rows each
    constexpr int kStageBytes = kWBytes + kXBytes;
    extern __shared__ __align__(16) unsigned char tiles_s[];       // [STAGES][w rows, x rows]
    const int lane = threadIdx.x % kWave;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    const int i = lane % 16, g = lane / 16;
    const int wm = wave / 2, wn = wave % 2;
    // workgroup -> (tile of x rows, tile of w rows): the tiles of x rows of one tile of w rows 8 apart
    const int xcd = blockIdx.x % 8, j = blockIdx.x / 8;
    const int m_tile = j % m_tiles;
    const int n_tile = (j / m_tiles) * 8 + xcd;
    constexpr int kColumns = GATED ? kTileRows / 2 : kTileRows;     // output columns a workgroup
    const int n_base = n_tile * kColumns;
    if (n_base >= N) return;
    const int m_base = m_tile * kXRows;
    const int k_begin = blockIdx.z * k_per_split;
    const int stages = min(k_per_split, K - k_begin) / kStageKeys;

    // ---- what this lane brings in every stage.  Load q covers rows 8q .. 8q + 7 of the stage's
    //      rows (the 128 of w, then those of x); this lane's row is 8q + lane / 8, its chunk
    //      (lane % 8) ^ (lane / 8).  A wavefront takes the loads wave, wave + kWaves, ... ----
    const int chunk = (lane % 8) ^ (lane / 8);
    uint32_t offset[kLoads];
#pragma unroll
    for (int u = 0; u < kLoads; ++u) {
        const int r = 8 * (wave + kWaves * u) + lane / 8;              // row of the stage
        size_t row;
        if (r < kTileRows) {
            if (GATED) row = r < 64 ? min(n_base + r, N - 1) : N + min(n_base + r - 64, N - 1);
            else row = min(n_base + r, N - 1);
        } else {
            row = min(m_base + r - kTileRows, M - 1);
        }
        offset[u] = static_cast<uint32_t>((row * K + chunk * 8) * 2);
    }
    const unsigned char* w_bytes = reinterpret_cast<const unsigned char*>(w) + static_cast<size_t>(k_begin) * 2;
    const unsigned char* x_bytes = reinterpret_cast<const unsigned char*>(x) + static_cast<size_t>(k_begin) * 2;
    auto issue = [&](int stage, int s) {
        const unsigned char* wb = w_bytes + static_cast<size_t>(s) * kRowBytes;
        const unsigned char* xb = x_bytes + static_cast<size_t>(s) * kRowBytes;
#pragma unroll
        for (int u = 0; u < kLoads; ++u) {
            const int q = wave + kWaves * u;        // the same for all lanes
            load_to_shared(q < kTileRows / 8 ? wb : xb, offset[u], tiles_s + stage * kStageBytes + q * 1024);
        }
    };

    float4_t acc[4][4];         // [tile of 16 w rows][tile of 16 x rows]
#pragma unroll
    for (int a = 0; a < 4; ++a)
#pragma unroll
        for (int b = 0; b < 4; ++b) acc[a][b] = float4_t{0.f, 0.f, 0.f, 0.f};

    // the rows of the tiles this wavefront reads: w rows wn * 64 + 16 a + i (gated: 32 gate rows, then
    // the 32 up rows, which lie 64 further on in the tile), x rows wm * 64 + 16 b + i
    int w_row_s[4], x_row_s[4];
#pragma unroll
    for (int a = 0; a < 4; ++a) {
        w_row_s[a] = GATED ? (a < 2 ? wn * 32 + 16 * a + i : 64 + wn * 32 + 16 * (a - 2) + i) : wn * 64 + 16 * a + i;
        x_row_s[a] = wm * 64 + 16 * a + i;
    }
#pragma unroll
    for (int p = 0; p < STAGES - 1; ++p)
        if (p < stages) issue(p, p);
    for (int s = 0; s < stages; ++s) {
        const int stage = s % STAGES;
        // This lane's loads of the stage have landed: loads come back in the order they went out, so
        // only those of the stages after it may still be on their way (STAGES - 2 of them at most).
        const int later = min(STAGES - 2, stages - 1 - s);
        if (later >= 2) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * kLoads) : "memory");
        else if (later == 1) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(kLoads) : "memory");
        else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();                                     // everyone's have, and everyone is done with the stage before
        if (s + STAGES - 1 < stages) issue((s + STAGES - 1) % STAGES, s + STAGES - 1);
        const unsigned char* ws = tiles_s + stage * kStageBytes;
        const unsigned char* xs = ws + kWBytes;
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) {
            const int place = ((ks * 4 + g) ^ (i % 8)) * 16;
            TFrag fw[4], fx[4];
#pragma unroll
            for (int a = 0; a < 4; ++a) {
                fw[a].u = *reinterpret_cast<const uint4*>(ws + w_row_s[a] * 128 + place);
                fx[a].u = *reinterpret_cast<const uint4*>(xs + x_row_s[a] * 128 + place);
            }
#pragma unroll
            for (int a = 0; a < 4; ++a)
#pragma unroll
                for (int b = 0; b < 4; ++b)
                    acc[a][b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fw[a].v, fx[b].v, acc[a][b], 0, 0, 0);
        }
    }

    // ---- lane (i, g) holds, of tile (a, b), output row m = 16 b + i and columns 4g .. 4g + 3 of the
    //      tile's 16 ----
#pragma unroll
    for (int b = 0; b < 4; ++b) {
        const int m = m_base + wm * 64 + 16 * b + i;
        if (m >= M) continue;
        if (GATED) {
#pragma unroll
            for (int a = 0; a < 2; ++a) {
                const int n = n_base + wn * 32 + 16 * a + 4 * g;
                if (n >= N) continue;
                float r[4];
#pragma unroll
                for (int v = 0; v < 4; ++v) {
                    const float gate = acc[a][b][v], up = acc[a + 2][b][v];
                    r[v] = activate<(GATED > 0 ? GATED - 1 : 0)>(gate) * up;
                }
                bf16* o = out + static_cast<size_t>(m) * N + n;
                if (n + 3 < N && N % 4 == 0) {
                    uint2 p;
                    p.x = pack2_bf16(r[0], r[1]);
                    p.y = pack2_bf16(r[2], r[3]);
                    *reinterpret_cast<uint2*>(o) = p;
                } else {
#pragma unroll
                    for (int v = 0; v < 4; ++v)
                        if (n + v < N) o[v] = from_float<bf16>(r[v]);
                }
            }
        } else {
#pragma unroll
            for (int a = 0; a < 4; ++a) {
                const int n = n_base + wn * 64 + 16 * a + 4 * g;
                if (n >= N) continue;
                const bool whole = n + 3 < N && N % 4 == 0;
                if (partial != nullptr) {
                    float* o = partial + (static_cast<size_t>(blockIdx.z) * M + m) * N + n;
                    if (whole) {
                        *reinterpret_cast<float4_t*>(o) = acc[a][b];
                    } else {
#pragma unroll
                        for (int v = 0; v < 4; ++v)
                            if (n + v < N) o[v] = acc[a][b][v];
                    }
                } else {
                    bf16* o = out + static_cast<size_t>(m) * N + n;
                    if (whole) {
                        uint2 p;
                        p.x = pack2_bf16(acc[a][b][0], acc[a][b][1]);
                        p.y = pack2_bf16(acc[a][b][2], acc[a][b][3]);
                        *reinterpret_cast<uint2*>(o) = p;
                    } else {
#pragma unroll
                        for (int v = 0; v < 4; ++v)
                            if (n + v < N) o[v] = from_float<bf16>(acc[a][b][v]);
                    }
                }
            }
        }
    }
}

// out[M, N] = x . w^T (gated 0, w [N, K]), or the gated product (gated = 1 + the activation's number;
// w [2N, K], gate rows first).  splits > 1 (plain only): `out` is null and `partial` float32
// [splits, M, N] takes the pieces' sums.  K must be a multiple of 64 * splits and the operands smaller
// than 4 GiB.  Returns 0, a HIP error code, or -1 for sizes it does not take.
WLLM_API int wllm_gemm_tile(const void* x, const void* w, void* out, float* partial, int M, int N, int K, int splits,
                            int activation, hipStream_t stream) {
    if (M < 1 || N < 1 || K < kStageKeys || splits < 1 || K % (kStageKeys * splits) != 0 || activation < 0 || activation > kActivations)
        return -1;
    if ((splits > 1) != (partial != nullptr) || (splits == 1 && out == nullptr) || (splits > 1 && activation != 0)) return -1;
    const size_t w_rows = static_cast<size_t>(activation ? 2 : 1) * N;
    if (w_rows * K * 2 >= (size_t(1) << 32) || static_cast<size_t>(M) * K * 2 >= (size_t(1) << 32)) return -1;
    const int m_tiles = (M + kTileRows - 1) / kTileRows;
    const int columns = activation ? kTileRows / 2 : kTileRows;
    const int n_tiles = (N + columns - 1) / columns;
    const long long blocks = static_cast<long long>((n_tiles + 7) / 8 * 8) * m_tiles;
    if (blocks > 0x7fffffffLL) return -1;
    const dim3 grid(static_cast<unsigned>(blocks), 1, splits);
    const bf16* xp = static_cast<const bf16*>(x);
    const bf16* wp = static_cast<const bf16*>(w);
    bf16* op = static_cast<bf16*>(out);
    const int per = K / splits;
    constexpr int kStageBytes = 2 * kTileRows * kRowBytes;
#define LAUNCH(GATED, STAGES)                                                                                      \
    do {                                                                                                            \
        static bool roomy = false;     /* more than 64 KiB of shared memory must be asked for once */              \
        if (STAGES * kStageBytes > 65536 && !roomy) {                                                               \
            if (hipFuncSetAttribute(reinterpret_cast<const void*>(&gemm_tile_kernel<GATED, STAGES>),                \
                                    hipFuncAttributeMaxDynamicSharedMemorySize, STAGES * kStageBytes) != hipSuccess) \
                return launch_status();                                                                             \
            roomy = true;                                                                                           \
        }                                                                                                           \
        gemm_tile_kernel<GATED, STAGES><<<grid, 256, STAGES * kStageBytes, stream>>>(xp, wp, op, partial, M, N, K,  \
                                                                                     m_tiles, per);                 \
    } while (0)
    // at most a workgroup a compute unit: nothing is lost by holding one, and it can have more on its way
    static int compute_units = 0;
    if (compute_units == 0) {
        int device = 0;
        if (hipGetDevice(&device) != hipSuccess ||
            hipDeviceGetAttribute(&compute_units, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess)
            return launch_status();
    }
    const bool deep = static_cast<long long>(n_tiles) * m_tiles * splits <= compute_units;
#define BY_STAGES(GATED)                \
    if (deep) LAUNCH(GATED, 4);         \
    else LAUNCH(GATED, 2)
    if (activation == 0) { BY_STAGES(0); }
    else { WLLM_BY_ACTIVATION(activation - 1, BY_STAGES(ACT + 1)) }
#undef BY_STAGES
#undef LAUNCH
    return launch_status();
}
