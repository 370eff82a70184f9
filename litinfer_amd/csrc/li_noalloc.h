// The one entry point of the kernel libraries that allocates nothing.
//
// It has no counterpart in the reference.  It is for callers that cannot allocate device
// memory: code under HIP graph capture, tight serving loops, harnesses that forbid
// hipMalloc.  li_argmax_rows, the entry point it is a variant of, takes two buffers for the
// partial results of its first stage from the caller; this one keeps them in a device array
// of the library itself.
#pragma once
#include <hip/hip_runtime.h>

// Rows of logits that one call takes.  The array holds LI_ARGMAX_NOALLOC_MAX_ROWS * 32
// (maximum, index) pairs = 256 KiB; each GPU that the library runs on holds it until the
// process ends.
#define LI_ARGMAX_NOALLOC_MAX_ROWS 1024

#ifdef __cplusplus
extern "C" {
#endif

// out[i] = index of the maximum of row i of logits [n, V] (float32, contiguous), the lowest
// index on ties: the result of li_argmax_rows.  logits and out are device memory of the
// current device; the work is enqueued on `stream`.  Returns 0, or 2 when n exceeds
// LI_ARGMAX_NOALLOC_MAX_ROWS (or a size is not positive), or 3 when a runtime call failed;
// li_argmax_rows_noalloc_error() then says what.  It calls no hipMalloc, no hipFree and no
// allocating library routine.  The first call on a device asks the runtime for the array's
// address there (li_argmax_rows_noalloc_init does the same ahead of time, e.g. before a
// capture begins).
//
// Every call on a GPU uses that GPU's one array, which keeps the last call's contents;
// nothing in it has to start at zero, the first stage writes all that the second reads.
// Calls that overlap on one GPU (two streams, two threads) race on it: keep them in order.
int li_argmax_rows_noalloc(const float* logits, int* out, int n, int V, hipStream_t stream);

// Set-up for the current device, once; optional.
int li_argmax_rows_noalloc_init(void);
int li_argmax_rows_noalloc_max_rows(void);
// Text of the calling thread's last failure of the calls above ("" after a success).
const char* li_argmax_rows_noalloc_error(void);

#ifdef __cplusplus
}
#endif
