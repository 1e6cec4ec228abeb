// An entry point that allocates nothing.
//
// It has no counterpart in the reference.  It is for callers that cannot allocate device memory: code that is
// recording a HIP graph, tight serving loops, harnesses that forbid allocation.  It calls no hipMalloc, hipFree or
// allocating library routine; its scratch memory is a fixed array inside the library.
#pragma once

#include <hip/hip_runtime.h>

// Most rows one call of sia_sample_static takes; more are refused with SIA_BAD_ARGUMENT (10001).
#define SIA_SAMPLE_STATIC_MAX_ROWS 64

// exported from a library whose other symbols are hidden
#define SIA_NO_ALLOC_API __attribute__((visibility("default")))

extern "C" {

// SIA_SAMPLE_STATIC_MAX_ROWS, for callers that load the library at run time.
SIA_NO_ALLOC_API int sia_sample_static_max_rows(void);

// Looks up, for the current device, the address of the scratch array and keeps it.  The look-up is no stream
// operation and may load the library's code on that device, so it must not happen while a stream is recording a
// graph: call this (or sia_sample_static itself, once) on each device before any recording starts.  After that
// sia_sample_static only launches kernels.  Returns 0 or a HIP error code.
SIA_NO_ALLOC_API int sia_sample_static_init(void);

// sia_sample without the workspace argument: one token per row of float logits [rows, vocab] into out[rows], with
// the meaning of every other argument as in sia_sample.  Returns 0, a HIP error code, or SIA_BAD_ARGUMENT for
// rows > SIA_SAMPLE_STATIC_MAX_ROWS, vocab <= 0 or a missing parameter array.
//
// Every call on a GPU uses that GPU's one scratch array, which keeps the last call's contents; the call clears
// what has to start at zero itself.  The first call on a device does what sia_sample_static_init does, with the
// same condition.  Calls that overlap on one GPU (two streams, two threads) race: run them one
// after the other.
SIA_NO_ALLOC_API int sia_sample_static(const float* logits, const float* temperature, const int* top_k, const float* top_p,
                      const float* uniform, int* out, int rows, int vocab, int filters, hipStream_t stream);

}
