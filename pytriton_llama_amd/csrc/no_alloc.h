// The one entry point of these libraries that is guaranteed to allocate nothing.
//
// It has no counterpart in the reference (lite_llama picks its greedy token with torch.argmax,
// lite_llama/generate_stream.py:150, and leaves memory to torch). It is for callers that cannot
// call hipMalloc: code under HIP graph capture, tight serving loops, harnesses that forbid
// allocation. ptl_argmax (sampling.hip) needs a workspace from its caller for the best value
// and index of every 4,096-logit chunk of every row; ptl_argmax_static runs the same two
// kernels with that workspace in a file-scope __device__ array of the library instead.
//
// Limits and rules:
//   * R * ceil(V / 4096) <= PTL_ARGMAX_STATIC_MAX_PARTIALS (16,384: 64 rows of a million logits,
//     or 512 rows of 128,256); more is refused with PTL_ERR_ARG and nothing is launched.
//   * The array takes 128 KiB of every GPU the library runs on, until the process ends.
//   * All calls on one GPU share that GPU's array. Every call overwrites the part it reads, so
//     nothing has to be cleared between calls, but two calls that overlap in time on one GPU
//     (different streams, or different threads) race: keep them on one stream or order them
//     with events.
//   * The array's address on a device is looked up once (hipGetSymbolAddress, with that device
//     current) and kept: by ptl_argmax_static_init for the current device, or by the first call
//     of ptl_argmax_static for the device of its stream. The look-up is no work for a stream
//     that is being captured: a call on a capturing stream whose device has not been looked up
//     returns -2 and records nothing, so call ptl_argmax_static_init (or ptl_argmax_static once)
//     before the capture begins. No call allocates or frees device or host memory.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#define PTL_ARGMAX_STATIC_MAX_PARTIALS 16384

// Looks the array's address up for the current device (see above). Returns 0 or -2.
extern "C" int ptl_argmax_static_init(void);

// out [R] int32 (device), logits [R, V] float32 with row stride ``stride`` (device), host_out:
// null, or pinned host memory [R] that receives the choices as well. Ties go to the lowest
// index; a NaN counts as -inf. Returns 0, -1 (sizes or arguments refused) or -2 (launch or
// symbol look-up failed).
extern "C" int ptl_argmax_static(int32_t* out, const float* logits, int R, int V, long stride,
                                 int32_t* host_out, hipStream_t stream);
