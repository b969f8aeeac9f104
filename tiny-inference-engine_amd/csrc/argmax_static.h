// Row-wise argmax that allocates nothing: the C interface of one entry point of the
// elementwise library.
//
// This entry point has no counterpart in the reference engine. It exists for callers that
// cannot allocate device memory: code running under HIP graph capture, tight serving loops
// that must not touch the allocator, and harnesses that forbid hipMalloc. It does what
// tie_argmax does (same kernels, same results), but the candidates that the first stage hands
// to the second - 64 (value, index) pairs per row - live in a file-scope __device__ array of the
// library instead of a workspace that the caller brings.
//
// Limits and rules:
//   * at most TIE_ARGMAX_STATIC_MAX_ROWS rows per call (the array holds 64 pairs for each:
//     TIE_ARGMAX_STATIC_MAX_ROWS * 64 * 8 bytes = 512 KiB on every GPU the library runs on, kept
//     until the process ends). More rows return TIE_EXCEEDS_STATIC_SCRATCH and launch nothing.
//   * the device that `stream` belongs to must be the current device of the calling thread; the
//     array's address on that device is looked up once per device and kept.
//   * nothing in the array has to start at zero: the second stage reads only the pairs that the
//     first stage of the same call has written. The array keeps the last call's contents.
//   * all calls on one GPU share that GPU's array: two calls whose kernels may overlap (different
//     streams, or graphs replayed side by side) race on it. Calls on one stream are ordered.
//   * no hipMalloc, hipFree or any other allocating call is made, on the first call or later.
#pragma once

#include <hip/hip_runtime.h>

#define TIE_ARGMAX_STATIC_MAX_ROWS 1024
#define TIE_EXCEEDS_STATIC_SCRATCH (-2)

// out[r] = lowest index of the maximum of logits[r, 0 .. V) for r < R (float32, rows V apart);
// -1 marks a row that holds a NaN. max_out (may be null) receives the maxima. Returns 0,
// TIE_BAD_ARGUMENT (-1) for sizes that are no sizes or null pointers, TIE_EXCEEDS_STATIC_SCRATCH
// (-2, with a line on stderr) for more rows than the array takes, or a hipError_t (> 0).
extern "C" int tie_argmax_static(const float* logits, int* out, float* max_out, int R, int V, hipStream_t stream);
