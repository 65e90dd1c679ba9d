// The product for many rows that loads its weights straight into registers (gemm_direct_bf16.hip), called from the
// tiled product's launch code.
#pragma once
#include "common.h"

// Fewer rows than this stay with the 128 x 128 tile and its K slices (too few blocks of 128 rows for the chip).
constexpr int GEMM_DIRECT_MIN_ROWS = 1024;

// mode: 0 store bfloat16, 1 store float32, 2 add into float32, 3 SwiGLU (W = gate, W2 = up, N = the width of each).
// True if launch_gemm_direct runs this shape (K a multiple of 128, N and ldc of 4, 16-byte aligned A and C, ...).
bool gemm_direct_takes(int mode, const void* A, int lda, const void* C, int ldc, int M, int N, int K);
// W, W2 in the tiled layout.  APC_ERR_UNSUPPORTED for a shape that gemm_direct_takes refuses.
int launch_gemm_direct(int mode, const bf16_t* A, int lda, const bf16_t* W, const bf16_t* W2, void* C, int ldc, int M,
                       int N, int K, hipStream_t stream);
// Products on rows that a product into the residual left for the RMS norm (A = the rows times the norm's weight, ss =
// [M][ss_parts] sums of x^2): the sums are scaled by 1 / sqrt(sum(ss[m]) / K + eps), before the activation where there
// is one.  mode 0 (store bfloat16) or 3 (SwiGLU).  SwiGLU from GEMM_DIRECT_PRE_MIN_ROWS rows on: the 28,672 weight
// rows of an 8B model's gate and up give 128-row tiles a full round of blocks already at 512 rows, where the 128 x 128
// tile takes 153 us and this 117; the others from GEMM_DIRECT_MIN_ROWS on.
constexpr int GEMM_DIRECT_PRE_MIN_ROWS = 384;
bool gemm_direct_pre_takes(int mode, const void* A, int lda, const void* C, int ldc, int M, int N, int K, int ss_parts);
int launch_gemm_direct_pre(int mode, const bf16_t* A, int lda, const float* ss, int ss_parts, float eps, const bf16_t* W,
                           const bf16_t* W2, void* C, int ldc, int M, int N, int K, hipStream_t stream);
// The product into the float32 residual C that also leaves the row for the RMS norm that reads the residual next:
// raw [M][ldr] = bfloat16(C g) and ss [M][parts] = sums of C^2 over parts of the columns.  gemm_direct_emit_parts says
// how many parts these sizes give (0: not taken; which depends on whether K goes in slices and on the tiles chosen);
// workspace: room for gemm_direct_k_split(M, N, K) * M * N floats where that is more than 1.
int gemm_direct_emit_parts(const void* A, int lda, const void* C, int ldc, int M, int N, int K);
int launch_gemm_direct_emit(const bf16_t* A, int lda, const bf16_t* W, float* C, int ldc, int M, int N, int K,
                            const float* g, bf16_t* raw, int ldr, float* ss, int ss_parts, float* workspace,
                            hipStream_t stream);
// Slices of K that a product of M rows into N columns should be cut into (1: none).  With more than one:
// launch_gemm_direct_slices leaves float32 sums in partials[slice][M][N], K a multiple of k_split * 128.
int gemm_direct_k_split(int M, int N, int K);
int launch_gemm_direct_slices(const bf16_t* A, int lda, const bf16_t* W, float* partials, int M, int N, int K,
                              int k_split, hipStream_t stream);
