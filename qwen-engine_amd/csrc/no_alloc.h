// The one entry point of the library that allocates nothing.
//
// It has no counterpart in the reference.  It is for callers that cannot allocate device memory:
// code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.
//
// qe_argmax_static is qe_argmax (lowest index of the largest logit per row, logits float32 [R, V]
// -> int32 [R], same kernels, same result) without the workspace argument: what the first stage
// leaves for the second (8 bytes per row and span of 2048 logits, when V > 4096) goes into an array
// of QE_ARGMAX_STATIC_BYTES bytes inside the library, of which every GPU the library runs on holds
// its own copy until the process ends.  It calls no hipMalloc, hipFree or allocating routine.
//
// Limits: R * ceil(V / 2048) * 8 <= QE_ARGMAX_STATIC_BYTES (436 rows of a vocabulary of 151 936);
// beyond that it returns -1 and qe_last_error() says so.  All calls on one GPU share that GPU's
// array, which keeps the last call's contents (nothing in it has to start at zero): two calls
// that overlap on one GPU (different streams, or different threads without an order between them)
// race on it.  Calls on one stream are safe.
#pragma once
#include <hip/hip_runtime.h>

#define QE_ARGMAX_STATIC_BYTES (256 * 1024)

extern "C" long qe_argmax_static_max_bytes();
extern "C" int qe_argmax_static(const float* logits, int* out, int R, int V, hipStream_t stream);
