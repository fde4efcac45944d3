// An entry point of the sampling module that allocates nothing.
//
// It has no counterpart in the reference, whose sampler is torch code.  It is for callers that
// cannot allocate device memory: code under HIP graph capture, tight serving loops, harnesses
// that forbid hipMalloc.  kvf_sample (sampling.hip) reads a greedy row of a large vocabulary with
// several workgroups and needs device memory beyond its inputs and outputs for that: a ticket per
// row and the best value and index of every chunk, which its caller brings in as `work`.
// kvf_sample_static does the same work with that memory in an array that is part of the
// library's image, so the caller passes inputs and outputs only.
//
// Limits: at most KVF_SAMPLE_STATIC_MAX_ROWS rows a call; more is refused with
// hipErrorInvalidValue and a line on stderr.  The array holds
// KVF_SAMPLE_STATIC_MAX_ROWS * (1 + 2 * KVF_SAMPLE_STATIC_MAX_SPLITS) int32 (132 KB) on every
// GPU the library runs on, until the process ends.
//
// Every call on a GPU uses that GPU's one array, which keeps what the last call left: the call
// clears the tickets it is going to use with a small kernel of its own (no memset node, so the
// launches may be captured in a graph) before the sampling kernel runs, in stream order.  Calls
// that overlap on one GPU (two streams, or two graphs replayed side by side) race on the array
// and give wrong tokens; calls in one stream's order are safe.
//
// The first call on a device looks the array's device address up (hipGetSymbolAddress, with that
// device current) and keeps it per device; nothing is allocated then either.
#pragma once
#include <hip/hip_runtime.h>

#define KVF_SAMPLE_STATIC_MAX_ROWS 1024
#define KVF_SAMPLE_STATIC_MAX_SPLITS 16

// One token per row of fp32 logits [rows, V] (row stride ld), as kvf_sample gives it: argmax
// where temperature[row] == 0 (lowest index among equal maxima), otherwise the inverse CDF of the
// processed distribution at u.  top_k, top_p and u_step may be null.  Returns a hipError_t code
// (0 = success).
extern "C" __attribute__((visibility("default")))
int kvf_sample_static(const float* logits, int ld, int rows, int V, const float* temperature,
                      const int* top_k, const float* top_p, const float* u, const int* u_step,
                      int u_stride, int* tokens, hipStream_t stream);
