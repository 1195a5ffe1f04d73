// Arg-max of float logits rows that allocates nothing.
//
// This entry point has no counterpart in the reference.  It is for callers that cannot allocate
// device memory: code under HIP graph capture, tight serving loops that must not touch the
// allocator, and harnesses that forbid hipMalloc.  tl_argmax() takes the partial results of wide
// rows (one best value and index per row and chunk) in two buffers the caller allocates;
// tl_argmax_static() keeps them in a file-scope device array instead and runs the same kernels.
//
// Limits: at most TL_ARGMAX_STATIC_MAX_ROWS rows per call (more is refused with an error); any row
// width.  The array is TL_ARGMAX_STATIC_BYTES (512 KiB) per GPU and stays until the process ends.
// Every call on a GPU uses that GPU's one array: calls that overlap on one GPU (two streams, two
// threads) race and give wrong answers; calls on one stream, or ordered by events, are safe.
// Nothing in the array has to start at zero: a call writes every entry it later reads.
//
// tl_argmax_static_setup() looks the array's device address up for the current GPU (once per GPU).
// tl_argmax_static() does that itself at its first call on a GPU; a caller that records a graph
// calls tl_argmax_static_setup() beforehand so that nothing but kernel launches happens in capture.
// Both return 0 on success; otherwise a non-zero code, and tl_last_error() has the message.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#define TL_ARGMAX_STATIC_MAX_ROWS 1024
#define TL_ARGMAX_STATIC_CHUNKS 64
#define TL_ARGMAX_STATIC_BYTES (TL_ARGMAX_STATIC_MAX_ROWS * TL_ARGMAX_STATIC_CHUNKS * 8)

extern "C" int tl_argmax_static_setup(void);

// logits: float [R, ld >= V] on the current GPU; out: int32 [R]; the lowest index wins a tie.
extern "C" int tl_argmax_static(const float* logits, int ld, int R, int V, int32_t* out, hipStream_t stream);
