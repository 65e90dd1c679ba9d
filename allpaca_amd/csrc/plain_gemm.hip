// Plain matrix product  C[M,N] = A[M,K] . W[N,K]^T  in true 32-bit arithmetic.
//
// Every output element is one chain  acc = fma(a[k], w[k], acc)  over k = 0..K-1
// in order, whatever M, N or the tile a row falls into: a row of a batch equals
// that row computed alone bit for bit (the property the reference asks of its
// host product, crates/allpaca-cpu/src/kernels.rs:2506-2525, and enforces on the
// GPU with `ExactRows`, crates/allpaca-core/src/model.rs:10851-10863).
// Operands may be float32 or bfloat16 (widened exactly); no matrix-core mode.
// Reference for the product itself: matmul_nt, crates/allpaca-cpu/src/kernels.rs:97-128.
#include "common.h"

constexpr int TM = 64, TN = 64, TK = 16;

// mode 0: C = acc (C of c_dtype)   mode 1: C += acc (C float32)
__global__ __launch_bounds__(256) void gemm_plain_kernel(const void* __restrict__ A, int a_dtype, int lda,
                                                         const void* __restrict__ W, int w_dtype, int ldw,
                                                         void* __restrict__ C, int c_dtype, int ldc, int M, int N,
                                                         int K, int mode) {
  __shared__ float As[TK][TM + 4];
  __shared__ float Ws[TK][TN + 4];
  const int tid = threadIdx.x;
  const int tx = tid % 16, ty = tid / 16;
  const int m0 = blockIdx.y * TM, n0 = blockIdx.x * TN;
  float acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;

  for (int k0 = 0; k0 < K; k0 += TK) {
    // 64 rows x 16 k = 1024 elements per operand, 4 per thread; consecutive threads read consecutive k
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int idx = tid + e * 256;
      const int r = idx / TK, kk = idx % TK;
      const int k = k0 + kk;
      float a = 0.f, w = 0.f;
      if (k < K) {
        if (m0 + r < M) a = load_f(A, a_dtype, (size_t)(m0 + r) * lda + k);
        if (n0 + r < N) w = load_f(W, w_dtype, (size_t)(n0 + r) * ldw + k);
      }
      As[kk][r] = a;
      Ws[kk][r] = w;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < TK; ++kk) {
      float a[4], w[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) a[i] = As[kk][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) w[j] = Ws[kk][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], w[j], acc[i][j]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int m = m0 + ty * 4 + i;
    if (m >= M) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + tx * 4 + j;
      if (n >= N) continue;
      const size_t o = (size_t)m * ldc + n;
      if (mode == 1) ((float*)C)[o] += acc[i][j];
      else store_f(C, c_dtype, o, acc[i][j]);
    }
  }
}

APC_EXPORT int apc_gemm_plain(const void* A, int a_dtype, int lda, const void* W, int w_dtype, int ldw, void* C,
                              int c_dtype, int ldc, int M, int N, int K, int mode, hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (K <= 0 || lda < K || ldw < K || ldc < N) return APC_ERR_BAD_ARG;
  if (mode == 1 && c_dtype != APC_F32) return APC_ERR_BAD_ARG;
  const int gy = ceil_div(M, TM);
  if (gy > 65535) return APC_ERR_BAD_ARG;
  hipLaunchKernelGGL(gemm_plain_kernel, dim3(ceil_div(N, TN), gy), dim3(256), 0, stream, A, a_dtype, lda, W, w_dtype,
                     ldw, C, c_dtype, ldc, M, N, K, mode);
  APC_LAUNCH_CHECK();
  return 0;
}
