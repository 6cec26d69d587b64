// Entry points of the sampling library that are not declared by their use alone.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

// Greedy choice for callers that cannot allocate device memory: code that runs under hipGraph capture, tight
// serving loops, harnesses that forbid hipMalloc. It has no counterpart in the reference, whose greedy choice is a
// library call (engine/dryft_qwen3/model.py:187, 262) that allocates as it pleases.
//
// The same kernels as dryft_argmax_rows (the largest logit of each row, the lowest index among equals), with the
// per-stretch results of the two-stage form kept in a fixed array in device memory that belongs to the library
// instead of in buffers the caller brings: DRYFT_ARGMAX_NOALLOC_ENTRIES entries of a float and an int, 128 KiB,
// held on every GPU the library runs on until the process ends. The call itself allocates and frees nothing.
//
//   logits      float32 [n_rows, vocab], rows `row_stride` floats apart, on the current device
//   out         int32 [n_rows] on the current device
//   chunks      stretches per row (1: one stage, no scratch); n_rows * chunks <= DRYFT_ARGMAX_NOALLOC_ENTRIES
//
// Returns 0, a HIP error code, -1 for arguments the kernels do not take, or -2 (with one line on stderr) when
// n_rows * chunks exceeds the array. Nothing in the array has to start at zero: every entry a call reads it has
// written before. All calls on one GPU share that GPU's array: calls that overlap there (different streams, or
// different threads) race; calls on one stream do not. The first call on a device looks the array's address up
// (hipGetSymbolAddress); make that call outside any capture.
#define DRYFT_ARGMAX_NOALLOC_ENTRIES 16384
__attribute__((visibility("default"))) int dryft_argmax_rows_noalloc(const float* logits, int n_rows, int vocab,
                                                                     int64_t row_stride, int* out, int chunks,
                                                                     hipStream_t stream);

#ifdef __cplusplus
}
#endif
