// C entry points of the sampling library (libsoc_sampling). Every entry point takes raw
// device pointers, sizes and a HIP stream, and returns a hipError_t as int.
#pragma once

#include <hip/hip_runtime.h>

#ifdef __cplusplus
extern "C" {
#endif

// logits [n, V] float32 -> out [n] int32, the lowest index among equal maxima.
// partial: workspace of n * n_chunks (float, int) pairs that the caller allocates.
int soc_argmax(const float* logits, void* partial, int* out, int n, int V, int n_chunks,
               hipStream_t stream);

// logits [n, V] float32; temperature [n] float32 or null (all greedy); seed, draws [n] int64.
int soc_sample(const float* logits, const float* temperature, const long long* seed,
               const long long* draws, int* out, int n, int V, hipStream_t stream);

// The same result as soc_argmax without a workspace argument and without any allocation.
// It has no counterpart in the reference:
// it is for callers that cannot allocate device memory, such as code under HIP graph capture,
// tight serving loops and harnesses that forbid hipMalloc. The chunk results live in a
// file-scope device array of SOC_ARGMAX_STATIC_MAX_ROWS * SOC_ARGMAX_STATIC_MAX_CHUNKS pairs
// (128 KiB) that every GPU the library runs on holds until the process ends. All calls on
// one GPU share that array: calls that overlap on one GPU (two streams, two threads) race,
// so keep them on one stream or order them with events. Nothing in the array has to start at
// zero: every pair that the second stage reads is written by the first stage of the same call.
// n > SOC_ARGMAX_STATIC_MAX_ROWS is refused with hipErrorInvalidValue and, if `message` is
// not null, a sentence in message[0 .. message_len). soc_argmax_static_init() looks up the
// array's address on the current device (once per device); the entry point does the same at
// its first call on a device, so calling init is only needed ahead of a graph capture.
#define SOC_ARGMAX_STATIC_MAX_ROWS 256
#define SOC_ARGMAX_STATIC_MAX_CHUNKS 64
int soc_argmax_static_init(char* message, int message_len);
int soc_argmax_static(const float* logits, int* out, int n, int V, hipStream_t stream, char* message,
                      int message_len);

#ifdef __cplusplus
}
#endif
