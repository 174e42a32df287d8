// Entry points of the library that allocate nothing.
//
// gl3_argmax_static has no counterpart in the reference (its greedy pick runs on the host,
// J/inference/sampler/Sampler.java:144-157). It is for callers that cannot allocate device
// memory: code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.
// It is gl3_argmax (every row's first greatest logit, the same two kernels) with the partial
// results of the row slices kept in a file-scope device array of the library instead of a
// workspace that the caller brings: the call itself neither allocates nor frees, and calls no
// routine that does.
//
// Limits and rules:
//  * at most GL3_ARGMAX_STATIC_ROWS rows a call (128 KiB of device memory per GPU that the library
//    runs on, held until the process ends); more rows are refused with a message;
//  * every call on a GPU uses that GPU's one array, which keeps the last call's contents. Nothing
//    in it has to start at zero (each call writes every partial result it reads), but two calls
//    that overlap in time on one GPU (different streams, different threads) race: keep them on one
//    stream or order them yourself;
//  * the device that is current at the call must be the one whose memory `logits` and `out` are in.
#pragma once
#include <hip/hip_runtime.h>

#define GL3_ARGMAX_STATIC_ROWS 256

// out[r] = index of the first greatest of logits[r * ld .. r * ld + V - 1] (float), r < n_rows.
// Returns 0, or a negative code with a message that gl3_last_error() returns.
extern "C" int gl3_argmax_static(const float* logits, long ld, int* out, int n_rows, int V, hipStream_t stream);
