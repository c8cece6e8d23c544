// Entry points of the sampler (sample.hip), for callers in C or through ctypes.
// Every entry point returns 0, or a negative code with the text in tk_last_error().
#pragma once

#include <hip/hip_runtime.h>

#ifdef __cplusplus
extern "C" {
#endif

#define TK_SAMPLE_EXPORT __attribute__((visibility("default")))

// Chunks a row of `vocab` logits is cut into: the sampler keeps three partial results
// (maximum, sum of exponentials, first index of the maximum) per (row, chunk).
TK_SAMPLE_EXPORT int tk_sample_chunks(int vocab);

// Greedy / temperature sampling of every row of logits [rows, vocab] (rows ld floats apart).
// part_max, part_sum (float) and part_arg (int) are the caller's workspace of
// rows * tk_sample_chunks(vocab) entries each.
TK_SAMPLE_EXPORT int tk_sample(const float* logits, int ld, int rows, int vocab, const float* temperature,
              const float* uniform, const int* slots, int* last_token, int* out_ids,
              float* out_logprobs, float* part_max, float* part_sum, int* part_arg,
              hipStream_t stream);

// The most (row, chunk) pairs tk_sample_static takes: rows * tk_sample_chunks(vocab) may not
// exceed it (256 rows of a 128 256-token vocabulary are 16 128).
#define TK_SAMPLE_STATIC_ITEMS 16384

// tk_sample for callers that cannot allocate device memory: code under HIP graph capture, tight
// serving loops, harnesses that forbid hipMalloc.  It has no counterpart in the reference, whose
// sampler allocates through torch on every call.  Same inputs, outputs and results as tk_sample;
// the partial results live in a file-scope device array of 3 * TK_SAMPLE_STATIC_ITEMS 32-bit
// words (192 KB) that every GPU the library runs on holds until the process ends.  Larger
// inputs are refused with an error.  The call allocates and frees nothing.  Nothing in the
// array has to start at zero: every entry a call reads it has written before.  All calls on
// one GPU share that GPU's array: calls that overlap there (two streams, two threads) race.
TK_SAMPLE_EXPORT int tk_sample_static(const float* logits, int ld, int rows, int vocab, const float* temperature,
                     const float* uniform, const int* slots, int* last_token, int* out_ids,
                     float* out_logprobs, hipStream_t stream);

#ifdef __cplusplus
}
#endif
