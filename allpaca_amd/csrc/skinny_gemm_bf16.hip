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
// The order of additions for an output depends on N, K and the number of 16-row tiles of M
// (which bounds the waves per block), never on which other rows are in the batch: a decoded
// row is the same alone and in any batch of up to 16 rows.
// Reference counterpart: gemv_nt_bf16_{wide,wide_rows,splitk}_kernel, hip/src/kernels.cpp:3555-3700
// (no matrix cores there); the product is matmul_nt, crates/allpaca-cpu/src/kernels.rs:97-128.
#include "mfma.h"

constexpr int SK_U = 4;                 // MFMAs (32 k each) per wave per pass
constexpr int SK_CHUNK = 32 * SK_U;     // 128 elements of k per wave per pass

enum { SK_STORE_BF16 = 0, SK_STORE_F32 = 1, SK_ACC_F32 = 2, SK_SWIGLU = 3 };

// (a non-temporal hint on the loads of W was measured slower here: plain loads)
__device__ __forceinline__ Frag load_stream(const bf16_t* p) { return load_frag(p); }

template <int MT, int MODE>
struct SkRegs {
  static constexpr int SETS = MODE == SK_SWIGLU ? 2 : 1;
  Frag w[SETS][SK_U];
  Frag a[MT][SK_U];
};

template <int MT, int MODE, int WPB>
__global__ __launch_bounds__(WPB * 64) void skinny_gemm_kernel(const bf16_t* __restrict__ A, int lda,
                                                               const bf16_t* __restrict__ W,
                                                               const bf16_t* __restrict__ W2, int ldw,
                                                               void* __restrict__ C, int ldc, int M, int N, int K) {
  constexpr int SETS = MODE == SK_SWIGLU ? 2 : 1;
  __shared__ float red[WPB * SETS * MT * 256];
  const int lane = threadIdx.x % WAVE, wave = threadIdx.x / WAVE;
  const int i = lane % 16, c = lane / 16;
  const int n0 = blockIdx.x * 16;
  const int n_row = min(n0 + i, N - 1);
  // rows beyond M or N are clamped to a valid row: what they compute is never stored
  const bf16_t* wrow = W + (size_t)n_row * ldw + c * 8;
  const bf16_t* wrow2 = MODE == SK_SWIGLU ? W2 + (size_t)n_row * ldw + c * 8 : nullptr;
  const bf16_t* arow[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) arow[mt] = A + (size_t)min(mt * 16 + i, M - 1) * lda + c * 8;

  floatx4 acc[SETS][MT];
#pragma unroll
  for (int s = 0; s < SETS; ++s)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[s][mt] = floatx4{0.f, 0.f, 0.f, 0.f};

  auto load_full = [&](SkRegs<MT, MODE>& r, int kb) {
#pragma unroll
    for (int u = 0; u < SK_U; ++u) {
      r.w[0][u] = load_stream(wrow + kb + u * 32);
      if (MODE == SK_SWIGLU) r.w[SETS - 1][u] = load_stream(wrow2 + kb + u * 32);
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) r.a[mt][u] = load_frag(arow[mt] + kb + u * 32);
    }
  };
  auto compute = [&](const SkRegs<MT, MODE>& r) {
#pragma unroll
    for (int u = 0; u < SK_U; ++u)
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        acc[0][mt] = mfma16(r.w[0][u], r.a[mt][u], acc[0][mt]);
        if (MODE == SK_SWIGLU) acc[SETS - 1][mt] = mfma16(r.w[SETS - 1][u], r.a[mt][u], acc[SETS - 1][mt]);
      }
  };

  // full chunks: the loads of the next chunk are in flight while the current one is multiplied.  Two register
  // sets swap roles, and the steady-state loop has no branch around a load, so the wait before a
  // multiplication counts exactly the loads issued after its operands.
  const int step = WPB * SK_CHUNK;
  const int first = wave * SK_CHUNK;
  const int nfull = K - first >= SK_CHUNK ? (K - SK_CHUNK - first) / step + 1 : 0;
  int kb = first + nfull * step;  // where this wave's cut chunk starts, if it has one
  SkRegs<MT, MODE> r0, r1;
  if (nfull > 0) {
    int at = first;
    load_full(r0, at);
    int done = 0;
    while (done + 2 < nfull) {
      load_full(r1, at + step);
      compute(r0);
      load_full(r0, at + 2 * step);
      compute(r1);
      at += 2 * step;
      done += 2;
    }
    if (done + 1 < nfull) {
      load_full(r1, at + step);
      compute(r0);
      compute(r1);
    } else {
      compute(r0);
    }
  }
  SkRegs<MT, MODE>& cur = r0;
  // the chunk that K cuts (K is a multiple of 8: a 16-byte piece is inside or outside as a whole)
  if (kb < K) {
#pragma unroll
    for (int u = 0; u < SK_U; ++u) {
      const bool in = kb + u * 32 + c * 8 < K;
      cur.w[0][u] = in ? load_frag(wrow + kb + u * 32) : zero_frag();
      if (MODE == SK_SWIGLU) cur.w[SETS - 1][u] = in ? load_frag(wrow2 + kb + u * 32) : zero_frag();
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) cur.a[mt][u] = in ? load_frag(arow[mt] + kb + u * 32) : zero_frag();
    }
    compute(cur);
  }

  // partial sums of the waves, added in wave order
  float* mine = red + wave * (SETS * MT * 256);
#pragma unroll
  for (int s = 0; s < SETS; ++s)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
      *reinterpret_cast<floatx4*>(&mine[((s * MT + mt) * 64 + lane) * 4]) = acc[s][mt];
  __syncthreads();

  for (int mt = wave; mt < MT; mt += WPB) {
    floatx4 sum[SETS];
#pragma unroll
    for (int s = 0; s < SETS; ++s) {
      sum[s] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int w = 0; w < WPB; ++w)
        sum[s] += *reinterpret_cast<const floatx4*>(&red[w * (SETS * MT * 256) + ((s * MT + mt) * 64 + lane) * 4]);
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

// waves per block: enough waves on the chip to keep HBM busy, never more than K can feed or LDS can hold
static int pick_wpb(int N, int K, int sets_mt) {
  const int tiles = ceil_div(N, 16);
  int wpb = 4;
  while (wpb < 16 && (long)tiles * wpb < 4096 && wpb * 2 * SK_CHUNK <= K && wpb * 2 * sets_mt <= 64) wpb *= 2;
  return wpb;
}

template <int MODE, int MT>
static int launch_skinny_mt(const bf16_t* A, int lda, const bf16_t* W, const bf16_t* W2, int ldw, void* C, int ldc,
                            int M, int N, int K, hipStream_t stream) {
  constexpr int SETS = MODE == SK_SWIGLU ? 2 : 1;
  const int wpb = pick_wpb(N, K, SETS * MT);
  dim3 grid(ceil_div(N, 16));
#define SK_LAUNCH(WPB_)                                                                                       \
  hipLaunchKernelGGL((skinny_gemm_kernel<MT, MODE, WPB_>), grid, dim3(WPB_ * WAVE), 0, stream, A, lda, W, W2, \
                     ldw, C, ldc, M, N, K)
  if (wpb == 4) SK_LAUNCH(4);
  else if (wpb == 8) SK_LAUNCH(8);
  else {
    if constexpr (SETS * MT <= 4) SK_LAUNCH(16);
    else return APC_ERR_UNSUPPORTED;
  }
#undef SK_LAUNCH
  APC_LAUNCH_CHECK();
  return 0;
}

template <int MODE>
static int launch_skinny(const bf16_t* A, int lda, const bf16_t* W, const bf16_t* W2, int ldw, void* C, int ldc, int M,
                         int N, int K, hipStream_t stream) {
  switch (ceil_div(M, 16)) {
    case 1: return launch_skinny_mt<MODE, 1>(A, lda, W, W2, ldw, C, ldc, M, N, K, stream);
    case 2: return launch_skinny_mt<MODE, 2>(A, lda, W, W2, ldw, C, ldc, M, N, K, stream);
    case 3: return launch_skinny_mt<MODE, 3>(A, lda, W, W2, ldw, C, ldc, M, N, K, stream);
    case 4: return launch_skinny_mt<MODE, 4>(A, lda, W, W2, ldw, C, ldc, M, N, K, stream);
    default: return APC_ERR_UNSUPPORTED;
  }
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
