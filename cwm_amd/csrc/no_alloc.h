// Entry points that allocate nothing.
//
// They have no counterpart in the reference, whose sampling runs through torch
// routines that allocate as they go (cwm/fastgen/generate.py:1002-1014,
// cwm/fastgen/utils/sampling.py:6-45).  They are for callers that cannot allocate
// device memory: code under HIP graph capture, tight serving loops, harnesses that
// forbid hipMalloc.  Such an entry point calls no hipMalloc, hipFree or allocating
// library routine; the scratch memory that its sibling takes as a workspace argument
// lives in a file-scope device array of a fixed size instead, one copy on every GPU
// that loads the library, held until the process ends.
//
// All calls on one GPU share that GPU's array, and the array keeps what the last call
// left in it.  Calls that overlap on one GPU (two streams, two threads) race on it:
// the caller must order them.  Nothing in the array has to start at zero: every
// element a call reads it has written before.
//
// The array's address on a GPU is looked up at the first call on that GPU
// (hipGetSymbolAddress, under a mutex), which is not a call for a stream that is
// capturing: call `cwm_sample_static_init` (or `cwm_sample_static` once) on each device
// before any capture; later calls only launch kernels.
#pragma once

#include <hip/hip_runtime.h>

// floats of scratch per GPU: rows * vocab of one call may not exceed it (8 MiB; 16 rows
// of a 131,072-entry vocabulary)
#define CWM_SAMPLE_STATIC_MAX_FLOATS (1 << 21)

// `cwm_sample` without its workspace argument.  Inputs and outputs are the caller's, as
// there: logits float32 [n_rows, vocab] with `row_stride`, temperature / top_p / uniform
// float32 [n_rows], token_out int32 [n_rows], logprob_out / sample_logprob_out float32
// [n_rows].  Returns non-zero with a message (cwm_error_message) if n_rows * vocab
// exceeds CWM_SAMPLE_STATIC_MAX_FLOATS or the array's address cannot be found.
extern "C" int cwm_sample_static(const float* logits, long row_stride, int n_rows, int vocab,
                                 const float* temperature, const float* top_p, const float* uniform,
                                 int* token_out, float* logprob_out, float* sample_logprob_out,
                                 hipStream_t stream);

// Looks up the array's address on the current device (once; later calls return at once).  Allocates
// nothing.  Returns non-zero with a message if the address cannot be found.
extern "C" int cwm_sample_static_init();

// floats of the array (CWM_SAMPLE_STATIC_MAX_FLOATS), for callers that size their batches by it
extern "C" long cwm_sample_static_capacity();
