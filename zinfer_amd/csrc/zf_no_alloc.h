// An entry point that allocates nothing.
//
// It has no counterpart in the reference (a CPU engine, which allocates where it likes).  It is
// for callers that cannot allocate device memory: code under HIP graph capture, tight serving
// loops, harnesses that forbid hipMalloc.  zf_argmax (elementwise.hip) takes its partial
// results' buffer from the caller, who must have allocated it; zf_argmax_no_alloc runs the same
// two kernels with the partials in a file-scope device array of fixed size.
#pragma once
#include <hip/hip_runtime.h>

#ifdef __cplusplus
extern "C" {
#endif

// The most (value, index) pairs of partial results the array holds: n rows times
// ceil(V / 4096) chunks of a row may not exceed it.  The array is 8 bytes a pair = 256 KB and
// every GPU the library runs on holds its own copy until the process ends.
#define ZF_ARGMAX_NO_ALLOC_MAX_PARTIALS 32768

#define ZF_NO_ALLOC_OK 0
#define ZF_NO_ALLOC_BAD_ARGUMENT -1   // a null pointer, n < 0 or V < 1
#define ZF_NO_ALLOC_TOO_LARGE -2      // n * ceil(V / 4096) > ZF_ARGMAX_NO_ALLOC_MAX_PARTIALS
#define ZF_NO_ALLOC_NO_SCRATCH -3     // the device array's address could not be had

// out[r] = index of the first maximum of logits[r, 0 .. V) for r in [0, n), on `stream` of the
// current device.  logits: float32 [n, V], out: int32 [n], both device memory of the caller.
// Calls no hipMalloc, hipFree or other allocating routine.  Returns ZF_NO_ALLOC_OK, one of the
// codes above (with a line on stderr that says which size was refused), or a positive HIP
// error code of the launch.
//
// The first call on a device looks up the address of that device's copy of the array
// (hipGetSymbolAddress); make it outside a graph capture.  All calls on one GPU share that
// GPU's array, which keeps the last call's contents: nothing in it has to start at zero (every
// partial that is read was written by the same call before), but two calls whose kernels
// overlap on one GPU (different streams, or threads) race on it.  Calls on one stream, or
// ordered by events, are safe.
int zf_argmax_no_alloc(const float* logits, int* out, int n, int V, hipStream_t stream);

#ifdef __cplusplus
}
#endif
