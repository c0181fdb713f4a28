// The one entry point of the kernel library that allocates nothing.
//
// It has no counterpart in the reference.  It is for callers that cannot allocate device
// memory: code under HIP graph capture, tight serving loops, harnesses that forbid
// hipMalloc.  It is `xi_argmax` (sampling.hip) with the scratch of its two-stage form (each
// row's per-chunk winners) in a file-scope device array instead of buffers the caller brings.
#pragma once
#include <hip/hip_runtime.h>

extern "C" {

// Most rows of one call; the device array holds
// xi_argmax_static_max_rows() * 32 chunks * (4 + 4) bytes = 64 KiB per GPU until the process ends.
int xi_argmax_static_max_rows();

// Resolves the array's address on the current device (one runtime call, which is no stream
// operation and may load the code object); later calls on that device make no such call.  A caller
// that records `xi_argmax_static` into a HIP graph calls this, or the entry point itself once,
// before the capture begins.  Returns 0 or non-zero as below.
int xi_argmax_static_init();

// out[r] = index of the largest of logits[r, 0..V) (the lowest index among equals), for
// rows <= xi_argmax_static_max_rows().  `logits` float32 [rows, V] and `out` int32 [rows] are
// device memory of the current device; the kernels run on `stream`.  Calls no hipMalloc, hipFree
// or allocating library routine.  Returns 0, or non-zero with the reason in xi_last_error()
// (sizes beyond the maximum are refused, never cut).
//
// Every call on a GPU shares that GPU's array: the first kernel writes every slot that the
// second reads, so nothing has to start at zero, but two calls that overlap on one GPU (on
// different streams, or from different threads) race on it.  Calls on one stream are ordered.
int xi_argmax_static(const float* logits, int rows, int V, int* out, hipStream_t stream);

}  // extern "C"
