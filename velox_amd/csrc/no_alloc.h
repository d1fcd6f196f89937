// The one entry point of the core library that allocates nothing.
//
// It has no counterpart in the reference, whose sampler takes its arg-max through torch and lets
// torch allocate what that needs.  It is for callers that cannot allocate device memory: code
// under HIP graph capture, tight serving loops that must not reach the allocator, harnesses that
// forbid hipMalloc.  Such a caller passes its inputs and outputs only; the kernels' scratch (the
// best (value, index) pair of every chunk of every row) lives in a file-scope device array of
// VELOX_ARGMAX_STATIC_BYTES that every GPU the library runs on holds until the process ends.
//
// velox_argmax_static gives, for the same arguments, the same indices as velox_argmax (it shares
// that entry point's kernels).  All calls on one GPU share that GPU's array: calls that overlap
// on one GPU (two streams, two threads) race on it and must be ordered by the caller.  Nothing
// in the array has to start at zero: every pair that the merge reads is written by the same call
// before, so what an earlier call left is never seen.
#pragma once

#include <hip/hip_runtime.h>

// Most (row, chunk) pairs of one call, and the bytes that the array takes on every GPU.
#define VELOX_ARGMAX_STATIC_MAX_PAIRS 65536
#define VELOX_ARGMAX_STATIC_BYTES (VELOX_ARGMAX_STATIC_MAX_PAIRS * 8)

// Return codes beside HIP's own (positive) error numbers.
#define VELOX_NO_ALLOC_BAD_ARGUMENT (-1)
#define VELOX_NO_ALLOC_TOO_LARGE (-2)
#define VELOX_NO_ALLOC_NO_SCRATCH (-3)

extern "C" {

// Looks up this GPU's copy of the scratch array (once per device, with that device current) and
// keeps its address.  velox_argmax_static does the same at its first call on a device; a caller
// that captures graphs calls this before the capture begins.  0, or HIP's error number.
int velox_argmax_static_init(void);

// out[r] = index of the largest of logits[r, 0 .. vocab) (the smallest index among equal values),
// for r in [0, rows); the vocabulary is cut into `chunks` pieces that run as workgroups of their own.
// Allocates nothing.  rows * chunks beyond VELOX_ARGMAX_STATIC_MAX_PAIRS is refused with
// VELOX_NO_ALLOC_TOO_LARGE and nothing is launched.  0 on success.
int velox_argmax_static(const float* logits, int* out, int rows, int vocab, int chunks, hipStream_t stream);

// A sentence for a return code of the two functions above (a static string).
const char* velox_no_alloc_error_text(int code);

}
