// An entry point for callers that cannot allocate device memory: code under HIP graph
// capture, tight serving loops, harnesses that forbid hipMalloc.  It has no counterpart
// in the reference.
//
// za_argmax_no_alloc is za_argmax (sampling.hip) with the workspace of the chunked form
// taken from an array that lives in the library's own device image instead of from the
// caller: the first index of each row's maximum of `logits` [n_rows, vocab] (32-bit)
// goes to `out` [n_rows] (int32).  With chunks > 1 every row is cut into `chunks`
// ranges whose (maximum, first index) pairs meet in the array, n_rows * chunks of
// them, at most ZA_ARGMAX_NO_ALLOC_MAX_PARTIALS (8 bytes each: 512 KiB on every GPU the
// library runs on, held until the process ends).
//
//   * Nothing is allocated or freed, on the device or through any library, by the call.
//   * Returns 0, ZA_ERR_ARG (-1: a null pointer, a count below zero, chunks < 1),
//     ZA_ERR_UNSUPPORTED (-2: n_rows * chunks exceeds the maximum, chunks > 65535, or a
//     device number of 64 and more), or the hipError_t of the HIP call that failed (a
//     launch, hipGetDevice, hipGetSymbolAddress); za_no_alloc_last_error() gives the
//     reason as text for the calling thread's last failed call.
//   * Every partial result the merge reads is written by the same call first, so
//     nothing has to be cleared between calls.
//   * All calls on one GPU share that GPU's array: calls that overlap there (two
//     streams, two threads) race.  Calls on one stream, or ordered by events, do not.
#pragma once

#include <hip/hip_runtime.h>

#define ZA_ARGMAX_NO_ALLOC_MAX_PARTIALS 65536

extern "C" __attribute__((visibility("default")))
int za_argmax_no_alloc(const float* logits, int n_rows, int vocab, int* out, int chunks,
                       hipStream_t stream);

extern "C" __attribute__((visibility("default")))
const char* za_no_alloc_last_error(void);
