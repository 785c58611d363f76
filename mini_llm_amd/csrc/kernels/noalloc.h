// An entry point that allocates nothing.
//
// It has no counterpart in the reference. It is for callers that cannot allocate device memory:
// code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc. The ordinary
// entry point `mllm_argmax` takes its scratch (the first stage's partial results) from the caller,
// who has to allocate it; this one keeps the scratch in a fixed array inside the library.
#pragma once

#include <hip/hip_runtime.h>

extern "C" {

// The most (row, chunk) pairs the fixed scratch holds: rows * mllm_argmax_chunks(V) must not exceed it
// (for a vocabulary of 50,257, 25 chunks a row: 655 rows). The array takes 8 bytes a pair, 128 KiB,
// on every GPU the library runs on, until the process ends.
#define MLLM_ARGMAX_NOALLOC_MAX_PAIRS 16384
int mllm_argmax_noalloc_max_pairs(void);

// out[i] = index of the largest logits[i*ld + 0..V), the lowest index on ties: the same kernels and
// the same result as `mllm_argmax`, with the partial results in the library's own fixed array on the
// current device. It calls no hipMalloc, hipFree or other allocating routine; the caller passes inputs
// and outputs (device memory) and a stream, and may capture the launches in a graph.
//
// Returns 0; -1 for V <= 0; -3 when n * mllm_argmax_chunks(V) exceeds the limit above (nothing is
// launched); a positive HIP error code if the array's address cannot be found or a launch fails.
//
// Every call on one GPU shares that GPU's array: calls that overlap on one GPU (different streams,
// or threads) race on it and must be ordered by the caller. Nothing in the array has to start at
// zero: every entry that the second stage reads has been written by the first stage of the same call.
int mllm_argmax_noalloc(const float* logits, int ld, int n, int V, int* out, hipStream_t stream);

}  // extern "C"
