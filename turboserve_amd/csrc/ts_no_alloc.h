// The one entry point of this library that allocates nothing.
//
// It has no counterpart in the reference, whose sampler calls torch.argmax and leaves memory to
// torch's allocator (src/turboserve/engine/core/sampler.py:216-238).  It is for callers that
// cannot allocate device memory: code under HIP graph capture, tight serving loops, harnesses
// that forbid hipMalloc.  `ts_argmax` needs a scratch buffer from its caller (64 partial
// results per row); this variant keeps that buffer in a file-scope device array of fixed size
// inside the library, so a call needs only its input and its output.
//
// Limits and rules:
//   * at most TS_ARGMAX_STATIC_MAX_ROWS rows a call; more is refused with TS_ERR_SHAPE (2) and
//     nothing is launched;
//   * the array (TS_ARGMAX_STATIC_MAX_ROWS * 64 * 8 bytes = 512 KiB) lives on every GPU the
//     library runs on until the process ends; its address on a device is looked up once, at the
//     first call with that device current;
//   * every call on a GPU uses that GPU's one array: calls that overlap on one GPU (two streams,
//     two threads) race, and the caller must order them.  Nothing in the array has to start at
//     zero: the first kernel writes every element the second one reads;
//   * it calls no hipMalloc, hipFree or allocating library routine.
#pragma once

#include <hip/hip_runtime.h>

#define TS_ARGMAX_STATIC_MAX_ROWS 1024

#ifdef __cplusplus
extern "C" {
#endif

// tokens[r] = index of the largest of logits[r * vocab .. (r + 1) * vocab), the lowest index on
// ties (what ts_argmax computes).  `tokens` (int32 [rows]) and `logits` (float32 [rows, vocab])
// are device memory of the current device; the kernels run on `stream`.  Returns 0, or 4 for a
// null pointer or vocab < 1, 2 for rows above the limit, 3 if a launch or the address look-up failed.
int ts_argmax_static(int* tokens, const float* logits, int rows, int vocab, hipStream_t stream);

#ifdef __cplusplus
}
#endif
