// The one entry point of the library that allocates nothing. It has no counterpart in the
// reference (mojothon/alofa has no GPU code and no such call): it exists for callers that cannot
// allocate device memory at the time of the call: code under HIP graph capture, tight serving
// loops, and harnesses that forbid hipMalloc.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

// Most rows one call takes. The scratch is rows * 64 partial maxima (a float and an int32 each):
// 128 KiB of device memory per GPU, held from the library's load until the process ends.
#define ALOFA_ARGMAX_NO_ALLOC_MAX_ROWS 256

#ifdef __cplusplus
extern "C" {
#endif

// out[r] = first index of the maximum of logits[r * stride .. r * stride + vocab), the lowest index
// on ties: the two-stage form of alofa_argmax (64 blocks per row, then one wave per row) with the
// partial maxima in a file-scope device array of the library instead of a buffer from the caller.
// `out` (int32, rows) and `logits` (float, rows x stride) are device memory of the current device;
// the kernels go to `stream`. Returns 0, or 1 with the reason in alofa_last_error(): rows beyond
// ALOFA_ARGMAX_NO_ALLOC_MAX_ROWS, sizes that do not fit, or a failed launch. It calls no
// hipMalloc, hipFree or allocating library routine; the first call on a device looks the array's
// address up (hipGetSymbolAddress), later calls reuse it.
// Every call on a GPU shares that GPU's array, which keeps the last call's contents: each call
// overwrites the cells it reads, so nothing needs clearing, but two calls that overlap in time on
// one GPU (different streams, different threads) race on it and must be serialised by the caller.
int alofa_argmax_no_alloc(int32_t* out, const float* logits, int64_t stride, int rows, int vocab, hipStream_t stream);

#ifdef __cplusplus
}
#endif
