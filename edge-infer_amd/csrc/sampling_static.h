// Greedy sampling for callers that must not allocate.
//
// This entry point has no counterpart in the reference.  It is for callers that cannot
// call hipMalloc or let a library do so for them: code under HIP graph capture, tight
// serving loops, harnesses that forbid allocation.  It is `ei_argmax` (sampling.hip) with
// the partial results of its many-blocks-a-row search held in a file-scope device array
// of the library instead of a buffer that the caller brings.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

// Most (row, chunk of 4096 logits) pairs one call may need: 256 rows of a vocabulary of
// 1,048,576, or any other product up to that.  The array is 512 KiB on every GPU the
// library has been used on and stays until the process ends.
#define EI_ARGMAX_STATIC_MAX_PARTIALS 65536

#ifdef __cplusplus
extern "C" {
#endif

// tokens[r] = index of the largest of logits[r, 0..V) (ties to the lowest index, NaN counts
// as -inf); probabilities[r] = 1 if the pointer is not null.  logits: float32 [rows, V];
// tokens: int32 [rows]; both on the current device.  Returns 0, or non-zero with a message
// in ei_last_error(): in particular when rows * ceil(V / 4096) exceeds
// EI_ARGMAX_STATIC_MAX_PARTIALS.  The call allocates nothing and frees nothing; its kernels
// run on `stream`.  Every call on a GPU shares that GPU's array (each call overwrites all
// the entries it later reads, so nothing has to be cleared): calls that overlap in time on
// one GPU, on different streams or from different threads, race; so do two replays of graphs
// that hold this call.
//
// The first call on a device looks up the array's address there, which a stream under
// capture does not allow: before capturing a call, run ei_argmax_static_prepare() (or one
// call of ei_argmax_static itself) on that device outside any capture.  A first call under
// capture is refused with an error and leaves the capture valid.
int ei_argmax_static(const float* logits, int rows, int V, int32_t* tokens, float* probabilities,
                     hipStream_t stream);

// Looks up the static array's address on the current device, once; allocates nothing.
// Returns 0, or non-zero with a message in ei_last_error().
int ei_argmax_static_prepare(void);

#ifdef __cplusplus
}
#endif
