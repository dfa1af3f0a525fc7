// An entry point for callers that cannot allocate device memory.
//
// It has no counterpart in the reference (whose backend allocates its buffers
// as it likes).  It is for callers that may not call hipMalloc while they run:
// code under HIP graph capture, tight serving loops, harnesses that forbid
// allocation.  Such a caller cannot hand llmrs_argmax_rows the scratch memory
// that lets several blocks share a long row, so this variant brings its own:
// a file-scope array in device memory, LLMRS_ARGMAX_STATIC_BYTES (256 KiB) on
// every GPU the library runs on, held until the process ends.
#pragma once
#include <hip/hip_runtime.h>

#define LLMRS_ARGMAX_STATIC_MAX_ROWS 1024
#define LLMRS_ARGMAX_STATIC_BYTES (LLMRS_ARGMAX_STATIC_MAX_ROWS * 32 * 8)

// out[r] = index of the largest of logits[r * ld .. r * ld + V), of equal ones the
// lowest: the same kernels and the same result as llmrs_argmax_rows with scratch.
// logits and out are device memory of the current device; the call is queued on
// `stream`.  It calls no hipMalloc, hipFree or other allocating routine.  More
// than LLMRS_ARGMAX_STATIC_MAX_ROWS rows are refused (-1, message through
// llmrs_hip_error()).  Every call on a GPU uses that GPU's one array: the stage
// that reads it runs after the stage of the same call that fills all of what it
// reads, so nothing needs clearing between calls, but two calls that overlap on
// one GPU (different streams, or threads) race on it and must not be made.
extern "C" int llmrs_argmax_rows_static(hipStream_t stream, const float* logits, int ld, int n_rows, int V, int* out);
