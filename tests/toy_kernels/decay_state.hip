// A kernel that a test brings with it: the state update of a toy mixer, s = decay * s + h token by
// token, with the state of every request in its row of a state tensor.  It shows that a part's kernel
// is a file of the part's own: it is compiled with the framework's flags and headers into a library
// beside it and registered as an operation from the test.
#include "common.h"

// One workgroup per segment, a thread per element of the width (in steps of the workgroup's size).
// state float32 [slots, hidden]; slots int32 [segments]; h T [tokens, hidden]; mixed float32 [tokens, hidden].
template <typename T>
__global__ void __launch_bounds__(256)
toy_decay_state_kernel(const T* __restrict__ h, float* __restrict__ state, const int* __restrict__ slots,
                       const int* __restrict__ seg_q_start, const int* __restrict__ seg_q_len,
                       float* __restrict__ mixed, int hidden, float decay) {
    const int seg = blockIdx.x;
    const int first = seg_q_start[seg], count = seg_q_len[seg];
    float* row = state + static_cast<size_t>(slots[seg]) * hidden;
    for (int d = threadIdx.x; d < hidden; d += blockDim.x) {
        float s = row[d];
        for (int t = first; t < first + count; ++t) {
            s = decay * s + to_float(h[static_cast<size_t>(t) * hidden + d]);
            mixed[static_cast<size_t>(t) * hidden + d] = s;
        }
        row[d] = s;
    }
}

// Returns 0, a HIP error code, or -1 for sizes the kernel does not take.
WLLM_API int toy_decay_state(const void* h, int is_bf16, float* state, const int* slots, const int* seg_q_start,
                             const int* seg_q_len, float* mixed, int segments, int hidden, float decay,
                             hipStream_t stream) {
    if (segments < 1 || hidden < 1) return -1;
    if (is_bf16)
        toy_decay_state_kernel<bf16><<<segments, 256, 0, stream>>>(static_cast<const bf16*>(h), state, slots, seg_q_start,
                                                                   seg_q_len, mixed, hidden, decay);
    else
        toy_decay_state_kernel<float><<<segments, 256, 0, stream>>>(static_cast<const float*>(h), state, slots, seg_q_start,
                                                                    seg_q_len, mixed, hidden, decay);
    return launch_status();
}
