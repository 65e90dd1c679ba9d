// Matrix product for few rows (decode):  C[M,N] = A[M,K] . W[N,K]^T,  M <= 64, bfloat16 in, float32 sums.
//
// The step is bound by reading W once from HBM, so the kernel is a stream over W:
//  * a block owns 16 output columns (16 rows of W) and all of K; its WPB waves split K in
//    interleaved chunks of 128 elements, so one pass of the block reads 16 rows x WPB*256 bytes;
//  * every lane loads 16 bytes of W straight into the A operand of v_mfma_f32_16x16x32_bf16
//    (row = lane%16, k = (lane/16)*8..+7) and 16 bytes of the activations into the B operand
//    (row m = lane%16): D[n][m], so a lane ends with 4 consecutive n of one row m;
//  * the waves' partial sums are added in wave order through LDS, then the epilogue runs:
//    store (bfloat16 or float32), add into a float32 residual, or SwiGLU of a gate and an up tile.
// The order of additions for an output depends on N and K only (never on M or on which
// other rows are in the batch): a decoded row is the same alone and in any batch.
// Reference counterpart: gemv_nt_bf16_{wide,wide_rows,splitk}_kernel, hip/src/kernels.cpp:3555-3700
// (no matrix cores there); the product is matmul_nt, crates/allpaca-cpu/src/kernels.rs:97-128.
#include "mfma.h"

constexpr int SK_U = 4;                 // MFMAs (32 k each) per wave per pass
constexpr int SK_CHUNK = 32 * SK_U;     // 128 elements of k per wave per pass

enum { SK_STORE_BF16 = 0, SK_STORE_F32 = 1, SK_ACC_F32 = 2, SK_SWIGLU = 3 };

template <int MT, int MODE>
__global__ __launch_bounds__(1024) void skinny_gemm_kernel(const bf16_t* __restrict__ A, int lda,
                                                           const bf16_t* __restrict__ W,
                                                           const bf16_t* __restrict__ W2, int ldw,
                                                           void* __restrict__ C, int ldc, int M, int N, int K) {
  extern __shared__ float red[];  // [waves][SETS * MT][64][4]
  constexpr int SETS = MODE == SK_SWIGLU ? 2 : 1;
  const int lane = threadIdx.x % WAVE, wave = threadIdx.x / WAVE, wpb = blockDim.x / WAVE;
  const int i = lane % 16, c = lane / 16;
  const int n0 = blockIdx.x * 16;
  const int n_row = min(n0 + i, N - 1);
  const bf16_t* wrow = W + (size_t)n_row * ldw;
  const bf16_t* wrow2 = MODE == SK_SWIGLU ? W2 + (size_t)n_row * ldw : nullptr;

  floatx4 acc[SETS][MT];
#pragma unroll
  for (int s = 0; s < SETS; ++s)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[s][mt] = floatx4{0.f, 0.f, 0.f, 0.f};

  const bf16_t* arow[MT];
  bool avalid[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int m = mt * 16 + i;
    avalid[mt] = m < M;
    arow[mt] = A + (size_t)min(m, M - 1) * lda;
  }

  for (int kb = wave * SK_CHUNK; kb < K; kb += wpb * SK_CHUNK) {
    Frag wf[SETS][SK_U];
    Frag af[MT][SK_U];
    const bool full = kb + SK_CHUNK <= K;
#pragma unroll
    for (int u = 0; u < SK_U; ++u) {
      const int k = kb + u * 32 + c * 8;
      const bool in = full || k < K;
      wf[0][u] = in ? load_frag(wrow + k) : zero_frag();
      if (MODE == SK_SWIGLU) wf[SETS - 1][u] = in ? load_frag(wrow2 + k) : zero_frag();
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) af[mt][u] = (in && avalid[mt]) ? load_frag(arow[mt] + k) : zero_frag();
    }
#pragma unroll
    for (int u = 0; u < SK_U; ++u)
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        acc[0][mt] = mfma16(wf[0][u], af[mt][u], acc[0][mt]);
        if (MODE == SK_SWIGLU) acc[SETS - 1][mt] = mfma16(wf[SETS - 1][u], af[mt][u], acc[SETS - 1][mt]);
      }
  }

  // partial sums of the waves, added in wave order
  float* mine = red + ((size_t)wave * SETS * MT) * 256;
#pragma unroll
  for (int s = 0; s < SETS; ++s)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int r = 0; r < 4; ++r) mine[((s * MT + mt) * 64 + lane) * 4 + r] = acc[s][mt][r];
  __syncthreads();

  for (int mt = wave; mt < MT; mt += wpb) {
    float sum[SETS][4];
#pragma unroll
    for (int s = 0; s < SETS; ++s)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        float t = 0.f;
        for (int w = 0; w < wpb; ++w) t += red[(((size_t)w * SETS * MT) + s * MT + mt) * 256 + lane * 4 + r];
        sum[s][r] = t;
      }
    const int m = mt * 16 + i;        // D[n][m]: this lane holds row m = lane%16 of the tile ...
    if (m >= M) continue;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int n = n0 + c * 4 + r;   // ... and columns n0 + (lane/16)*4 + r
      if (n >= N) continue;
      const size_t o = (size_t)m * ldc + n;
      if (MODE == SK_STORE_BF16) ((bf16_t*)C)[o] = float_to_bf16(sum[0][r]);
      else if (MODE == SK_STORE_F32) ((float*)C)[o] = sum[0][r];
      else if (MODE == SK_ACC_F32) ((float*)C)[o] += sum[0][r];
      else ((bf16_t*)C)[o] = float_to_bf16(silu_f(sum[0][r]) * sum[SETS - 1][r]);
    }
  }
}

// waves per block: enough waves on the chip to keep HBM busy, never more than K can feed
static int pick_wpb(int N, int K) {
  const int tiles = ceil_div(N, 16);
  int wpb = 4;
  while (wpb < 16 && (long)tiles * wpb < 4096 && wpb * 2 * SK_CHUNK <= K) wpb *= 2;
  return wpb;
}

template <int MODE>
static int launch_skinny(const bf16_t* A, int lda, const bf16_t* W, const bf16_t* W2, int ldw, void* C, int ldc, int M,
                         int N, int K, hipStream_t stream) {
  const int wpb = pick_wpb(N, K);
  const int mt = ceil_div(M, 16);
  const int sets = MODE == SK_SWIGLU ? 2 : 1;
  const size_t smem = (size_t)wpb * sets * mt * 256 * sizeof(float);
  dim3 grid(ceil_div(N, 16)), block(wpb * WAVE);
#define SK_LAUNCH(MT_)                                                                                              \
  hipLaunchKernelGGL((skinny_gemm_kernel<MT_, MODE>), grid, block, smem, stream, A, lda, W, W2, ldw, C, ldc, M, N, K)
  switch (mt) {
    case 1: SK_LAUNCH(1); break;
    case 2: SK_LAUNCH(2); break;
    case 3: SK_LAUNCH(3); break;
    case 4: SK_LAUNCH(4); break;
    default: return APC_ERR_UNSUPPORTED;
  }
#undef SK_LAUNCH
  APC_LAUNCH_CHECK();
  return 0;
}

static bool aligned16(const void* p) { return ((uintptr_t)p & 15u) == 0; }

// mode: 0 store bfloat16, 1 store float32, 2 add into float32
APC_EXPORT int apc_skinny_gemm_bf16(const void* A, int lda, const void* W, int ldw, void* C, int ldc, int M, int N,
                                    int K, int mode, hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (K <= 0 || lda < K || ldw < K || ldc < N) return APC_ERR_BAD_ARG;
  if (M > 64 || K % 8 || lda % 8 || ldw % 8 || !aligned16(A) || !aligned16(W)) return APC_ERR_UNSUPPORTED;
  const bf16_t* a = (const bf16_t*)A;
  const bf16_t* w = (const bf16_t*)W;
  switch (mode) {
    case SK_STORE_BF16: return launch_skinny<SK_STORE_BF16>(a, lda, w, nullptr, ldw, C, ldc, M, N, K, stream);
    case SK_STORE_F32: return launch_skinny<SK_STORE_F32>(a, lda, w, nullptr, ldw, C, ldc, M, N, K, stream);
    case SK_ACC_F32: return launch_skinny<SK_ACC_F32>(a, lda, w, nullptr, ldw, C, ldc, M, N, K, stream);
    default: return APC_ERR_BAD_ARG;
  }
}

// out[m, f] = silu(A[m] . Wg[f]) * (A[m] . Wu[f]);  Wg, Wu: [F, K] with the same row stride
APC_EXPORT int apc_skinny_swiglu_bf16(const void* A, int lda, const void* Wg, const void* Wu, int ldw, void* C, int ldc,
                                      int M, int F, int K, hipStream_t stream) {
  if (M <= 0 || F <= 0) return 0;
  if (K <= 0 || lda < K || ldw < K || ldc < F) return APC_ERR_BAD_ARG;
  if (M > 64 || K % 8 || lda % 8 || ldw % 8 || !aligned16(A) || !aligned16(Wg) || !aligned16(Wu))
    return APC_ERR_UNSUPPORTED;
  return launch_skinny<SK_SWIGLU>((const bf16_t*)A, lda, (const bf16_t*)Wg, (const bf16_t*)Wu, ldw, C, ldc, M, F, K,
                                  stream);
}
