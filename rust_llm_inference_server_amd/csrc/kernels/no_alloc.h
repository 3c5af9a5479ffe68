// An entry point that allocates nothing.
//
// It has no counterpart in the reference.  It is for callers that cannot allocate device
// memory: code that runs under HIP graph capture, tight serving loops that must not reach the
// allocator, and harnesses that forbid hipMalloc.  The existing rlis_sample_rows takes the
// scratch for its per-chunk winners from the caller (who allocates it per call);
// rlis_sample_rows_static keeps that scratch in a file-scope device array instead and runs the
// same two kernels.
//
// Limits and rules:
//  * rows * chunks may not exceed rlis_sample_rows_static_max_parts() (16,384 partial results,
//    128 KiB of device memory that every GPU the library runs on holds until the process
//    ends); larger requests are refused with a message, nothing is launched.
//  * The array's address is looked up once per device, at the entry point's first call with
//    that device current; the caller must have the device of `stream` current.
//  * Every call on a GPU shares that GPU's array.  Nothing in it has to start at zero (each
//    call writes every entry it later reads), but two calls that overlap on one GPU (different
//    streams, or different threads) race on it: keep calls on one GPU in stream order.
//  * No hipMalloc, hipFree or allocating library routine is called; inputs and outputs are the
//    caller's.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

extern "C" {

// As rlis_sample_rows (one token per row of float32 logits: argmax where inv_temps[r] is 0,
// else Gumbel-max keyed by keys[r]), without the caller's scratch.  Returns 0, or nonzero with
// a message for rlis_last_error().
int rlis_sample_rows_static(const float* logits, long long row_stride, int rows, int vocab,
                            const uint32_t* keys, const float* inv_temps, int* out, int chunks,
                            hipStream_t stream);

// The largest rows * chunks that rlis_sample_rows_static accepts.
int rlis_sample_rows_static_max_parts(void);

}
