// An entry point that allocates nothing.
//
// It has no counterpart in the reference, whose sampler runs torch operations that allocate their own
// temporaries (pico_vllm/sampler.py:4-37).  It is for callers that cannot allocate device memory: code
// under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.
//
// pico_argmax_noalloc is pico_argmax (the index of the first maximum of every row of float32 logits,
// PICO_ARGMAX_CHUNKS workgroups a row and a second launch that picks among their results) with the
// per-chunk maxima kept in a fixed array in device memory that belongs to this library instead of a
// workspace that the caller brings.  The array holds PICO_NOALLOC_MAX_ROWS rows (256 KiB; every GPU
// that the library runs on holds its own copy until the process ends); more rows are refused with an error.
// The call makes no hipMalloc, hipFree or other allocating call; the caller passes logits and out.
//
// Every call on a GPU shares that GPU's array, which keeps the last call's contents.  Nothing in it has
// to start at zero: a call writes every entry it later reads.  Calls that overlap on one GPU (different
// streams without an order between them) race on the array and must not be made.
//
// pico_noalloc_init looks up the array's address on the current device; the entry point does the same
// at its first call on a device.  A caller that records a graph calls it once before the capture begins.
#pragma once
#include <hip/hip_runtime.h>

#define PICO_NOALLOC_MAX_ROWS 1024

extern "C" int pico_noalloc_max_rows();
extern "C" int pico_noalloc_init();
extern "C" int pico_argmax_noalloc(const float* logits, int ld, int R, int V, int* out, hipStream_t stream);
