// An entry point of the kernel library that allocates nothing.
//
// It has no counterpart in the reference.  It is for callers that cannot call hipMalloc, or anything that does:
// code under HIP graph capture, tight serving loops, harnesses that forbid allocation.
#pragma once
#include <hip/hip_runtime.h>

// The most (row, piece) pairs a call may need; the scratch array holds one float and one int for each
// (32 KiB of device memory per GPU the library runs on, held until the process ends).
#define TA_ARGMAX_STATIC_PAIRS 4096
// Status of a call whose sizes are beyond that maximum (more than TA_ARGMAX_STATIC_PAIRS rows).
#define TA_STATIC_TOO_LARGE (-2)

extern "C" {

// The greedy pick of `ta_argmax` (first maximum of each row of `logits`, float32 [n_rows, vocab], into `out`,
// int32 [n_rows]) without a workspace argument: the pieces' maxima of its first stage go to a file-scope device
// array of the library instead, through the same two kernels.  The caller passes only input and output, both
// in device memory; nothing is allocated or freed, here or in anything this calls.
//
// Returns 0; a HIP error code (> 0) of a launch or of the look-up of the array's address on this device
// (done once per device, at the first call there, with that device current); -1 for vocab < 1; or
// TA_STATIC_TOO_LARGE for n_rows > TA_ARGMAX_STATIC_PAIRS (nothing is launched then).
//
// Every call on a GPU uses that GPU's one array.  Each call writes every pair it later reads, so nothing needs
// to start at zero and what the last call left does not matter; but two calls that overlap on one GPU (two
// streams, two threads) race on it: callers run them one after the other.
int ta_argmax_static(const void* logits, void* out, int n_rows, int vocab, hipStream_t stream);

}
