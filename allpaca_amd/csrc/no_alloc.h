// The one entry point of the `plain` library that allocates nothing.
//
// It has no counterpart in the reference.  It is for callers that cannot allocate device memory: code under HIP
// graph capture, tight serving loops, harnesses that forbid hipMalloc.  apc_argmax_rows cuts a wide row into 64 pieces
// and needs room for every piece's (value, index), which its caller brings in as a workspace; here that room is a
// file-scope array in device memory (512 KiB, held by every GPU the library runs on until the process ends), so the
// call needs no workspace, and it calls no hipMalloc, hipFree or allocating library routine.
#pragma once
#include <hip/hip_runtime.h>

// Rows of logits one call takes at most: 1024 rows x 64 pieces x (float value + int index) = 512 KiB.
#define APC_ARGMAX_NO_ALLOC_MAX_ROWS 1024
// Returned when n_rows exceeds APC_ARGMAX_NO_ALLOC_MAX_ROWS (nothing is launched).
#define APC_ERR_TOO_LARGE (-3)

// out[r] = index of the first maximum of logits[r, 0..V) (token 0 when nothing exceeds -inf), the same result as
// apc_argmax_rows.  logits: float32 [n_rows, ldl] on the current device, ldl >= V; out: int32 [n_rows].
// Returns 0, APC_ERR_BAD_ARG (-1) for V <= 0 or ldl < V, APC_ERR_TOO_LARGE (-3) for more than
// APC_ARGMAX_NO_ALLOC_MAX_ROWS rows, or a hipError_t (> 0).
// Every call on a GPU uses that GPU's one array: calls that overlap on one GPU (two streams, two threads) race; calls
// in one stream do not.  Nothing in the array has to start at zero: a call writes every entry before it reads it.
extern "C" __attribute__((visibility("default"))) int apc_argmax_rows_no_alloc(const float* logits, int ldl,
                                                                              int n_rows, int V, int* out,
                                                                              hipStream_t stream);
