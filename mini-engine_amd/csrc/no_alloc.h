// An entry point that allocates nothing. It has no counterpart in the reference (whose sampling is
// a handful of library calls that allocate as they go); it is here for callers that cannot allocate
// device memory around a call: code under HIP graph capture, tight serving loops, harnesses that
// forbid hipMalloc.
//
// me_sample_static does what me_sample does (one token per row of float32 logits [num_rows, vocab]:
// argmax where the row's temperature is 0 or `temperatures` is null, else a draw from
// softmax(logits / temperature) keyed by keys[row]) but takes no workspace: the per-slice
// (value, index) pairs between its two kernels live in a file-scope device array of
// ME_SAMPLE_STATIC_SCRATCH_BYTES, which every GPU this library runs on holds until the process
// ends. The caller still passes the logits, the temperatures and keys, and the output. It calls no
// hipMalloc, hipFree or allocating library routine.
//
//  * Sizes: num_rows * me_sample_chunks(vocab) must not exceed me_sample_static_max_pairs()
//    (16,384 pairs: 215 rows at a vocabulary of 151,936); beyond that it returns non-zero with a
//    message in me_last_error() and launches nothing.
//  * Every call on one GPU uses that GPU's one array, on whatever stream. Calls whose kernels may
//    overlap on a GPU (different streams without an order between them, several host threads) race
//    on it: order them. Nothing in the array has to start at zero, so calls in stream order need no
//    clearing between them.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#define ME_SAMPLE_STATIC_SCRATCH_BYTES (128 * 1024)

extern "C" int me_sample_static_max_pairs();
extern "C" int me_sample_static(const float* logits, int num_rows, int vocab, const float* temperatures,
                                const uint64_t* keys, int* out, hipStream_t stream);
