// An entry point of the kernel library that allocates nothing.
//
// It has no counterpart in the reference.  It is for callers that cannot call
// hipMalloc: code under HIP graph capture, tight serving loops that must not touch the allocator,
// harnesses that forbid allocation.  The caller passes inputs and outputs; everything else the
// kernels need lives in a device array that is part of the library's image.
#pragma once
#include <hip/hip_runtime.h>

#define WLLM_NO_ALLOC_API extern "C" __attribute__((visibility("default")))

// Error codes of the functions below (0 is success; positive values are hipError_t codes).
#define WLLM_STATIC_BAD_ARGUMENT (-1)     // rows < 1, vocab < 1 or a null pointer
#define WLLM_STATIC_TOO_MANY_ROWS (-2)    // rows > wllm_sample_static_max_rows()

// The most rows one call of `wllm_sample_rows_static` takes (64).  The device array behind it is
// 64 rows * 2,120 words * 8 bytes = 1,085,440 bytes; every GPU the library runs on holds its own
// copy at its own address until the process ends.
WLLM_NO_ALLOC_API int wllm_sample_static_max_rows(void);

// Resolves the address of the current device's copy of the array (hipGetSymbolAddress) and keeps
// it.  Optional: `wllm_sample_rows_static` does the same at its first call on a device.  A caller
// that captures graphs calls this once, outside the capture, on each device it uses.  Returns 0 or
// a hipError_t code.
WLLM_NO_ALLOC_API int wllm_sample_static_init(void);

// What an error code of the two functions above means, as text.
WLLM_NO_ALLOC_API const char* wllm_sample_static_error(int code);

// Samples one token per row, exactly as `wllm_sample_rows_split` does (same kernels, same tokens and
// log-probabilities bit for bit), with the kernels' scratch area in the library's own device array
// instead of a buffer the caller allocates.  No hipMalloc, hipFree or other allocating call is made.
//
//   logits            float32 [rows, vocab] on the device; rows with a repetition penalty are changed in place
//   params            float32 [rows, 5]: temperature (0: greedy), top_k (0: off), top_p (1: off), min_p (0: off),
//                     repetition_penalty (1: off)
//   seeds             int64 [rows, 2]: key and counter of the row's uniform draw
//   penalty_ids       int32 [P] with penalty_offsets int32 [rows + 1], or both null
//   out_tokens        int32 [rows];  out_logprobs float32 [rows]
//   truncations       non-zero if any row has top_k or top_p on
//
// rows beyond wllm_sample_static_max_rows() are refused with WLLM_STATIC_TOO_MANY_ROWS and nothing
// is launched.  All calls on one GPU share that GPU's array: it keeps the last call's contents (the
// first kernel of a call clears what must start at zero), and two calls that overlap in time on one
// GPU (different streams, or different threads) race.  Calls on one stream are ordered and safe.
WLLM_NO_ALLOC_API int wllm_sample_rows_static(float* logits, const float* params, const long long* seeds,
                                              const int* penalty_ids, const int* penalty_offsets, int* out_tokens,
                                              float* out_logprobs, int rows, int vocab, int truncations,
                                              hipStream_t stream);
