// An entry point that allocates nothing.
//
// It has no counterpart in the reference (tracel-ai/burn-lm leaves every buffer to its tensor
// library).  It is for callers that cannot allocate device memory: code under HIP graph capture,
// tight serving loops, harnesses that forbid hipMalloc.
//
// blm_argmax_static is blm_argmax (first index of each row's maximum of float logits [R, V], row
// stride ld, lowest index wins ties) without the two workspace arguments: the slice maxima that
// its first kernel leaves for its second live in a file-scope __device__ array of the library,
// BLM_ARGMAX_STATIC_MAX_ROWS rows large (256 KiB per GPU, held until the process ends).  The
// caller passes only logits and out.  More rows than that are refused with an error; nothing is
// allocated or freed, by HIP or by any library.
//
// Every call on a GPU shares that GPU's array.  Nothing in it has to start at zero (the first
// kernel writes every place the second one reads, for exactly the rows of this call), so no
// clearing is queued; what the last call left behind is never read.  Calls that overlap on one GPU
// (two streams, two threads) race on the array: order them, or use blm_argmax with workspaces of
// their own.
//
// blm_static_scratch_init looks the array's device address up for the current device (once per
// device; the entry point does the same at its first call on a device).  Callers that capture
// graphs call it before the capture opens.
#pragma once
#include <hip/hip_runtime.h>

#define BLM_ARGMAX_STATIC_MAX_ROWS 1024

extern "C" int blm_static_scratch_init();
extern "C" int blm_argmax_static(const float* logits, int* out, int R, int V, int ld, hipStream_t stream);
