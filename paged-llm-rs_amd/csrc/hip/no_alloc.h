// An entry point for callers that cannot allocate device memory.
//
// This one has no counterpart in the reference engine.  It is for callers that may not call hipMalloc,
// or anything that calls it, while they run: code under HIP graph capture, tight serving loops, and
// harnesses that forbid allocation.  The ordinary entry point of the same operation (pl_argmax) takes
// its scratch memory from the caller, who has to allocate it; this one keeps its scratch in a fixed
// array in device memory that belongs to the library.
#pragma once

#include <hip/hip_runtime.h>

// The most rows of logits one call of pl_argmax_static takes.  The array holds one candidate (a 32-bit
// value and a 32-bit index) for each of the 64 stretches of each row: 512 KB, which every GPU that the
// library runs on holds until the process ends.
#define PL_ARGMAX_STATIC_MAX_ROWS 1024

#ifdef __cplusplus
extern "C" {
#endif

// out[r] = the index of the largest of logits[r, 0..V), the first such index where several are equal,
// exactly as pl_argmax gives it (the same two kernels run).  logits is [m, V] 32-bit floats and out is
// m 32-bit integers, both in device memory of the current device; the kernels go onto ``stream``.
// It calls no allocating routine.  m beyond PL_ARGMAX_STATIC_MAX_ROWS is refused: -1 comes back and
// pl_last_error() says why.
//
// Every call on a GPU uses that GPU's one array.  Nothing in it has to start at zero (each candidate is
// written before it is read), and it keeps the last call's contents.  Calls that overlap on one GPU (two
// streams, two threads) race for it: a caller runs them one after the other.
int pl_argmax_static(const float* logits, int* out, int m, int V, hipStream_t stream);

#ifdef __cplusplus
}
#endif
