// An entry point that allocates nothing.
//
// It has no counterpart in the reference, whose kernels take their workspaces from the tensor library's
// allocator. It is for callers that cannot allocate device memory: code that runs under HIP graph capture,
// tight serving loops, harnesses that forbid hipMalloc. The caller passes inputs and outputs only; the
// partial results of the search live in a file-scope device array inside the library.
#pragma once

#include <hip/hip_runtime.h>

#ifdef __cplusplus
extern "C" {
#endif

// Most rows one call takes. The device array holds LMSF_GREEDY_STATIC_MAX_ROWS * 32 (value, index) pairs:
// 256 KiB on every GPU the library runs on, held until the process ends.
#define LMSF_GREEDY_STATIC_MAX_ROWS 1024

// out[r] = index of the first maximum of row r of float32 logits [R, V] (row stride ld, in elements), the
// same tokens as lmsf_sample gives for greedy rows with a scratch buffer, for any V > 0 and 0 <= R <=
// LMSF_GREEDY_STATIC_MAX_ROWS; more rows are refused with an error and nothing is launched.
//
// Calls no hipMalloc, hipFree or allocating library routine. Every call on a GPU uses that GPU's one array,
// which keeps the last call's contents; the kernels write every entry they later read, so nothing has to be
// cleared between calls. Two calls that overlap on one GPU (different streams, or different threads) race on
// the array: the caller orders them. The array's address is asked for once per device, at the first call on
// that device with that device current.
//
// Returns 0 on success; otherwise non-zero, and lmsf_last_error() gives the reason.
int lmsf_greedy_tokens_static(const float* logits, long ld, int R, int V, int* out, hipStream_t stream);

#ifdef __cplusplus
}
#endif
