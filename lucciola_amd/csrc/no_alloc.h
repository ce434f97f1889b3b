// An entry point that allocates nothing.
//
// It has no counterpart in the reference, whose kernels get every buffer from their caller
// (include/kernels/argmax.h).  It is for callers that cannot allocate device memory: code under
// HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  lc_sample needs a
// workspace of lc_sample_workspace(R) words from its caller; lc_sample_static does the same
// work with the same kernels and keeps that workspace in a file-scope __device__ array of the
// library (sampling.hip), so a caller passes inputs and outputs only.
//
//   * At most LC_SAMPLE_STATIC_MAX_ROWS rows a call; more is refused with an error.  The array
//     takes LC_SAMPLE_STATIC_MAX_ROWS * 32 parts * 3 words * 4 bytes = 384 KiB on every GPU
//     the library runs on, until the process ends.
//   * The array's device address is looked up once per device (hipGetSymbolAddress, at the
//     first call with that device current); no call allocates or frees anything.
//   * Every call on a GPU shares that GPU's array, which keeps the last call's contents.
//     Nothing in it has to start at zero: every word a call reads, that call has written
//     before.  Calls that overlap on one GPU (two streams, two threads) race on it; calls on
//     one stream are ordered and safe.
#pragma once

#include <hip/hip_runtime.h>

#define LC_SAMPLE_STATIC_MAX_ROWS 1024
#define LC_NO_ALLOC_API extern "C" __attribute__((visibility("default")))

// As lc_sample (sampling.hip): token ids out[R] from float32 logits [R, V]; temperature and
// uniform may both be null (all rows greedy).  Returns 0, or non-zero with lc_last_error() set.
LC_NO_ALLOC_API int lc_sample_static(const float* logits, const float* temperature, const float* uniform,
                                int* out, int R, int V, hipStream_t stream);

// The most rows lc_sample_static takes.
LC_NO_ALLOC_API int lc_sample_static_max_rows(void);
