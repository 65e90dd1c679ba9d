// The SwiGLU product on the 256-row tile (gemm_wide_bf16.hip), called from the tiled product's launch code.
#pragma once
#include "common.h"

// C[m, f] = silu(A[m] . Wg[f]) * (A[m] . Wu[f]) for all M rows and F columns; Wg, Wu in the tiled layout; K a multiple
// of 64.  With pre_ss the sums are scaled by 1 / sqrt(sum(pre_ss[m][0 .. pre_parts)) / K + pre_eps) (the folded norm).
int launch_swiglu_wide(const bf16_t* A, int lda, const bf16_t* Wg, const bf16_t* Wu, bf16_t* C, int ldc, int M, int F,
                       int K, const float* pre_ss, int pre_parts, float pre_eps, hipStream_t stream);
