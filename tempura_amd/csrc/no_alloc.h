// An entry point of the kernel library that allocates nothing.
//
// It has no counterpart in the reference.  It is for callers that cannot allocate device memory around a
// call: code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  tp_argmax, the
// entry point it is a variant of, takes its scratch memory (the partial maxima of a row's chunks) as a
// workspace argument that the caller allocates; here that memory is a fixed array inside the library.
#pragma once
#include <hip/hip_runtime.h>

// most rows of logits one call takes (the array holds 64 partial results of 8 bytes per row: 256 KiB, held by
// every GPU the library runs on until the process ends)
#define TP_ARGMAX_STATIC_MAX_ROWS 512

extern "C" {

// Looks up the array's address on the current device (once per device; later calls return at once).  Called by
// tp_argmax_static itself when needed; a caller that captures a graph calls it beforehand, outside the capture.
// Returns 0, or nonzero with the reason in tp_last_error().
int tp_argmax_static_init(void);

// out[r] = index of the largest of logits[r, 0..vocab) (float32, row-major), the last one on exact ties:
// the same result as tp_argmax.  rows <= TP_ARGMAX_STATIC_MAX_ROWS, else an error and nothing is launched.
// Calls no hipMalloc, hipFree or any allocating routine; launches at most two kernels on `stream`.
// Every call on a GPU uses that GPU's one array: calls that overlap on one GPU (two streams, two threads)
// race on it.  Nothing in the array has to start at zero (every partial result that is read was written by
// the same call before), so it is never cleared.
int tp_argmax_static(const float* logits, int* out, int rows, int vocab, hipStream_t stream);

}
