// Entry points that allocate nothing.
//
// These have no counterpart in the reference.  They are for callers that cannot allocate device memory: code under HIP
// graph capture, tight serving loops, harnesses that forbid hipMalloc.  The kernels are those of the ordinary entry
// point; only the scratch memory differs: it is a fixed array in the library's device image instead of a buffer the
// caller brings.
//
// Rules of use:
//   * Every GPU holds one copy of the array (LLMX_ARGMAX_STATIC_LEADERS entries of 8 bytes = 128 KB) from the moment
//     the library is loaded there until the process ends.
//   * The array of the device that is current at the call is used; the stream must belong to that device.
//   * Calls that overlap on one GPU (two streams, two threads) share the array and race; callers serialise them.
//   * The array keeps the last call's contents.  Nothing in it has to start at zero: every entry a call reads was
//     written by the same call before.
//   * llmx_no_alloc_init() resolves the array's address on the current device; the entry point does the same at its
//     first call on a device.  Under graph capture call llmx_no_alloc_init() before the capture begins.
#pragma once
#include <hip/hip_runtime.h>

#define LLMX_ARGMAX_STATIC_LEADERS 16384

extern "C" {

// Resolves the static scratch array's device address for the current device (once per device).  0, or the HIP error.
int llmx_no_alloc_init(void);

// llmx_argmax_rows without a scratch argument: out[r] = arg-max of scores[r, 0..n) with the same tie, NaN and `skip`
// rules.  Rows wider than 16,384 scores are cut into slices of 8,192 whose leaders go through the static array, so
// rows * ceil(n / 8192) may not exceed LLMX_ARGMAX_STATIC_LEADERS: beyond it the call returns -2, launches nothing and
// leaves its reason in llmx_no_alloc_last_error().  Calls no hipMalloc, hipFree or allocating library routine.
int llmx_argmax_rows_static(const float* scores, const int* skip, int* out, int rows, int n, hipStream_t stream);

// The reason of the calling thread's last refusal or failure ("" when there was none).
const char* llmx_no_alloc_last_error(void);
}
