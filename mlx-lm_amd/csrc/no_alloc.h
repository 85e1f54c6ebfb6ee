// Entry points that allocate nothing.
//
// They have no counterpart in the reference (ml-explore/mlx-lm has no device code and lets its
// array library allocate as it likes).  They are for callers that cannot call hipMalloc:
// code under HIP graph capture, tight serving loops, harnesses that forbid it.  Such a caller
// passes inputs and outputs as before; memory that the kernels need beyond those lies in an
// array that the library holds on every GPU it runs on, from the library's load to the
// process's end.
#pragma once

#include <hip/hip_runtime.h>

#ifdef __cplusplus
extern "C" {
#endif

// Most floats of partial sums that gemm_bf16_decode_split_static can hold: n_splits * M * N
// has to stay within it (4 MiB on each GPU).
#define GEMM_BF16_DECODE_STATIC_FLOATS (1u << 20)

// Looks up, once per device, where the current device holds its copy of the array.  The entry
// point below does the same at its first call on a device; a caller that must not meet that
// look-up later (under graph capture) calls this at set-up, with the device current.
// Returns 0, or 1 with the text in mlxlm_last_error().
int gemm_bf16_decode_static_init(void);

// out = epilogue(A @ W^T + bias) for 1 to 16 rows of bfloat16, K split over n_splits blocks a
// feature group: gemm_bf16_decode's partial sums followed by sum_partials, with the partial sums
// in the library's own array instead of a workspace of the caller's.
//   A    [M, K] bfloat16, row stride lda (a multiple of 8), 16-byte aligned
//   W    [N, K] bfloat16, row stride ldw; or the packed layout of 16 x 64 tiles with ldw = 0
//   bias [N] float32 or null
//   out  [M, N], row stride ldo: bfloat16; float32 with flag 4 (GEMM_OUT_F32) or with
//        flag 2 (GEMM_ACCUMULATE, out += ...); flag 1 adds the tanh-GELU
// n_splits * M * N must not exceed GEMM_BF16_DECODE_STATIC_FLOATS: refused with an error,
// as every size is that gemm_bf16_decode refuses.  Calls hipMalloc, hipFree or any other
// allocating routine never.  All calls on one GPU share that GPU's array, which keeps the last
// call's partial sums: nothing in it has to start at zero (a call writes every partial sum
// that it reads), but two calls that overlap on one GPU (two streams, two threads) race.
// Returns 0, or 1 with the text in mlxlm_last_error().
int gemm_bf16_decode_split_static(void* out, const void* A, int lda, const void* W, const float* bias,
                                  int M, int N, int K, int ldw, int ldo, int flags, int n_splits,
                                  hipStream_t stream);

#ifdef __cplusplus
}
#endif
