// Entry points of the next-token sampler (sampling.hip).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

// Bytes of scratch `tw_sample_rows` needs for ROWS logits rows.
long tw_sample_workspace_bytes(int rows);

// out[r] = greedy (temperature null or 0) or sampled token of logits[r][0..vocab); the caller brings the
// scratch memory (`workspace`, at least tw_sample_workspace_bytes(rows) bytes, 16-byte aligned).
int tw_sample_rows(const float* logits, long ld, int rows, int vocab, const float* temperature,
                   const uint64_t* seeds, const int* counters, int* out, void* workspace,
                   long workspace_bytes, hipStream_t stream);

// The same result as tw_sample_rows, from the same kernels, for callers that CANNOT ALLOCATE device memory
// and therefore cannot bring a workspace: code under HIP graph capture, tight serving loops, harnesses that
// forbid hipMalloc. It has no counterpart in the reference engine. The per-chunk partial results live in
// an array that is part of the library's device image (TW_SAMPLE_STATIC_MAX_ROWS rows, 256 KiB, held by
// every GPU the library runs on until the process ends); this call allocates and frees nothing and calls
// no routine that does. More than TW_SAMPLE_STATIC_MAX_ROWS rows are refused with TW_ERR_TOO_LARGE.
// All calls on one GPU share that array: two calls whose kernels overlap there (other streams, other
// threads) race; calls on one stream are ordered and safe. Nothing in the array has to start at zero:
// every entry a call reads it has written first. The first call on a device looks the array's address
// up there (hipGetSymbolAddress, no allocation) and keeps it: a caller that captures graphs makes one
// call on the device before its first capture.
#define TW_SAMPLE_STATIC_MAX_ROWS 256
int tw_sample_rows_static(const float* logits, long ld, int rows, int vocab, const float* temperature,
                          const uint64_t* seeds, const int* counters, int* out, hipStream_t stream);

#ifdef __cplusplus
}
#endif
