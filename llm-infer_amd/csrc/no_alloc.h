// An entry point that allocates nothing.  It has no counterpart in the reference.
//
// It is for callers that cannot call hipMalloc: code under HIP graph capture, tight serving loops,
// harnesses that forbid allocation.  li_argmax takes its partial results (one maximum and one index
// for every chunk of every row) in a workspace that the caller brings; li_argmax_static is the same
// operation with the same kernels, but the partial results lie in an array that is part of the
// library's device code.  Every GPU that the library runs on holds that array (LI_ARGMAX_STATIC_BYTES)
// from the first call to the end of the process.
//
// The caller still passes the logits and the output.  Sizes beyond the array are refused with
// LI_UNSUPPORTED; li_argmax_static_capacity says what fits.  No hipMalloc, hipFree or other
// allocating routine is called.  Nothing in the array has to start at zero: the first kernel writes
// every entry that the second reads.  All calls on one GPU share that GPU's array, so calls that
// overlap on one GPU (two streams, two threads) race; calls on one stream are ordered and safe.
#pragma once
#include <hip/hip_runtime.h>

#define LI_ARGMAX_STATIC_ENTRIES 8192                       /* rows * chunks of a row, at most */
#define LI_ARGMAX_STATIC_BYTES (LI_ARGMAX_STATIC_ENTRIES * 8)

extern "C" {
// Looks up the array's address on the current device (once per device; later calls are free).  The
// entry point does this by itself at its first call on a device; a caller that records graphs may
// call it beforehand, outside the capture.  0 or LI_HIP_ERROR.
int li_argmax_static_init(void);
// How many rows of V logits one call takes (0 if V <= 0).
int li_argmax_static_capacity(int V);
// out[r] = index of the first maximum of logits[r, 0..V), as li_argmax.  logits float32 [n_rows, V]
// and out int32 [n_rows] on the current device.
int li_argmax_static(const float* logits, int n_rows, int V, int* out, hipStream_t stream);
}
