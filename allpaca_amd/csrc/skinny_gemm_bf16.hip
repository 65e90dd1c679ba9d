// Matrix product for few rows (decode):  C[M,N] = A[M,K] . W[N,K]^T,  M <= 64, bfloat16 in, float32 sums.
//
// The step is bound by reading W once from HBM, so the kernel is a stream over W, which is stored in
// tiles of 16 rows x 32 columns laid out as the 64 lanes of a wave hold an operand of
// v_mfma_f32_16x16x32_bf16 (1 KiB a tile, tiles of a 16-row band in K order, bands in N order; rows and
// columns beyond N, K are zero):
//  * a block owns NB bands (16 NB output columns) and all of K; each of its WPB waves takes a contiguous
//    range of K and reads it in steps of 4 tiles per band: every load of W is 1 KiB of consecutive bytes and a
//    wave walks forward through one region of memory;
//  * the activations are the other operand (row m = lane % 16, 16 bytes of k per lane), loaded once per step
//    for all NB bands: D[n][m], so a lane ends with 4 consecutive n of one row m;
//  * the loads of the next step are in flight while the current one is multiplied (two register sets that
//    swap roles; no branch around a load in the steady state);
//  * the waves' partial sums are added in wave order through LDS, then the epilogue runs: store (bfloat16 or
//    float32), add into a float32 residual, or SwiGLU of a gate band and an up band.
// The order of additions for an output depends on N, K and the number of 16-row tiles of M, never on which
// other rows are in the batch: a decoded row is the same alone and in any batch of up to 16 rows.
// Reference counterpart: gemv_nt_bf16_{wide,wide_rows,splitk}_kernel, hip/src/kernels.cpp:3555-3700
// (no matrix cores, row-major weights); the product is matmul_nt, crates/allpaca-cpu/src/kernels.rs:97-128.
#include "mfma.h"

constexpr int SK_U = 4;              // tiles (32 k each) per band per step
constexpr int TILE_ELEMS = 16 * 32;  // elements of a tile

enum { SK_STORE_BF16 = 0, SK_STORE_F32 = 1, SK_ACC_F32 = 2, SK_SWIGLU = 3 };

template <int MT, int NB>
struct SkRegs {
  Frag w[NB][SK_U];
  Frag a[MT][SK_U];
};

// NB: weight bands per block (for SwiGLU: 2 = one gate band and the up band of the same outputs)
template <int MT, int MODE, int NB, int WPB>
__global__ __launch_bounds__(WPB * 64) void skinny_gemm_kernel(const bf16_t* __restrict__ A, int lda,
                                                               const bf16_t* __restrict__ W,
                                                               const bf16_t* __restrict__ W2, int chunks,
                                                               void* __restrict__ C, int ldc, int M, int N, int K) {
  __shared__ float red[WPB * NB * MT * 256];
  const int lane = threadIdx.x % WAVE, wave = threadIdx.x / WAVE;
  const int i = lane % 16, c = lane / 16;
  constexpr int OUT_BANDS = MODE == SK_SWIGLU ? 1 : NB;
  const int band0 = blockIdx.x * OUT_BANDS;
  const int bands = (N + 15) / 16;

  // band pointers (bands beyond the matrix are clamped to the last: what they compute is never stored)
  const bf16_t* wb[NB];
#pragma unroll
  for (int b = 0; b < NB; ++b) {
    if (MODE == SK_SWIGLU) wb[b] = (b == 0 ? W : W2) + (size_t)band0 * chunks * TILE_ELEMS + lane * 8;
    else wb[b] = W + (size_t)min(band0 + b, bands - 1) * chunks * TILE_ELEMS + lane * 8;
  }
  const bf16_t* arow[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) arow[mt] = A + (size_t)min(mt * 16 + i, M - 1) * lda + c * 8;

  floatx4 acc[NB][MT];
#pragma unroll
  for (int b = 0; b < NB; ++b)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[b][mt] = floatx4{0.f, 0.f, 0.f, 0.f};

  auto load_step = [&](SkRegs<MT, NB>& r, int ch) {  // tiles ch .. ch+3, all inside K
#pragma unroll
    for (int u = 0; u < SK_U; ++u) {
#pragma unroll
      for (int b = 0; b < NB; ++b) r.w[b][u] = load_frag(wb[b] + (size_t)(ch + u) * TILE_ELEMS);
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) r.a[mt][u] = load_frag(arow[mt] + (ch + u) * 32);
    }
  };
  auto compute = [&](const SkRegs<MT, NB>& r) {
#pragma unroll
    for (int u = 0; u < SK_U; ++u)
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int b = 0; b < NB; ++b) acc[b][mt] = mfma16(r.w[b][u], r.a[mt][u], acc[b][mt]);
  };

  // this wave's range of tiles along K: [c_lo, c_hi); steps of 4 whole tiles, then single tiles
  const int full_chunks = K / 32;                       // tiles that lie wholly inside K (for the activations)
  const int per_wave = ((chunks + WPB - 1) / WPB + SK_U - 1) / SK_U * SK_U;
  const int c_lo = min(wave * per_wave, chunks), c_hi = min(c_lo + per_wave, chunks);
  const int c_full_hi = min(c_hi, full_chunks);
  const int nsteps = c_full_hi > c_lo ? (c_full_hi - c_lo) / SK_U : 0;
  SkRegs<MT, NB> r0, r1;
  if (nsteps > 0) {
    int at = c_lo;
    load_step(r0, at);
    int done = 0;
    while (done + 2 < nsteps) {
      load_step(r1, at + SK_U);
      compute(r0);
      load_step(r0, at + 2 * SK_U);
      compute(r1);
      at += 2 * SK_U;
      done += 2;
    }
    if (done + 1 < nsteps) {
      load_step(r1, at + SK_U);
      compute(r0);
      compute(r1);
    } else {
      compute(r0);
    }
  }
  // what is left of the range: single tiles; the last one may be cut by K (K is a multiple of 8, so a lane's
  // 16 bytes of activations are inside or outside as a whole; W is zero beyond K)
  for (int ch = c_lo + nsteps * SK_U; ch < c_hi; ++ch) {
    const bool in = ch * 32 + c * 8 < K;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      const Frag af = in ? load_frag(arow[mt] + ch * 32) : zero_frag();
#pragma unroll
      for (int b = 0; b < NB; ++b) acc[b][mt] = mfma16(load_frag(wb[b] + (size_t)ch * TILE_ELEMS), af, acc[b][mt]);
    }
  }

  // partial sums of the waves, added in wave order
  float* mine = red + wave * (NB * MT * 256);
#pragma unroll
  for (int b = 0; b < NB; ++b)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) *reinterpret_cast<floatx4*>(&mine[((b * MT + mt) * 64 + lane) * 4]) = acc[b][mt];
  __syncthreads();

  constexpr int ITEMS = OUT_BANDS * MT;  // (band, m-tile) pairs to finish, spread over the waves
  constexpr int NSUM = MODE == SK_SWIGLU ? 2 : 1;
  for (int item = wave; item < ITEMS; item += WPB) {
    const int b = item / MT, mt = item % MT;
    floatx4 sum[NSUM];
#pragma unroll
    for (int s = 0; s < NSUM; ++s) {
      const int bb = MODE == SK_SWIGLU ? s : b;
      sum[s] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int w = 0; w < WPB; ++w)
        sum[s] += *reinterpret_cast<const floatx4*>(&red[w * (NB * MT * 256) + ((bb * MT + mt) * 64 + lane) * 4]);
    }
    const int m = mt * 16 + i;  // D[n][m]: this lane holds row m = lane % 16 of the tile ...
    if (m >= M) continue;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int n = (band0 + b) * 16 + c * 4 + r;  // ... and columns (lane / 16) * 4 + r of the band
      if (n >= N) continue;
      const size_t o = (size_t)m * ldc + n;
      if (MODE == SK_STORE_BF16) ((bf16_t*)C)[o] = float_to_bf16(sum[0][r]);
      else if (MODE == SK_STORE_F32) ((float*)C)[o] = sum[0][r];
      else if (MODE == SK_ACC_F32) ((float*)C)[o] += sum[0][r];
      else ((bf16_t*)C)[o] = float_to_bf16(silu_f(sum[0][r]) * sum[NSUM - 1][r]);
    }
  }
}

// bands per block and waves per block: enough blocks and waves to keep HBM busy, never more waves than K
// can feed with whole steps or LDS can hold
static void pick_shape(int N, int K, int mt, bool swiglu, int* nb, int* wpb) {
  const int bands = ceil_div(N, 16), chunks = ceil_div(K, 32);
  *nb = (!swiglu && bands >= 2048 && mt <= 2) ? 2 : 1;
  const int blocks = ceil_div(bands, *nb);
  const int sets = swiglu ? 2 : *nb;
  int w = 4;
  while (w < 16 && (long)blocks * w < 4096 && chunks >= w * 2 * SK_U && w * 2 * sets * mt <= 64) w *= 2;
  *wpb = w;
}

template <int MODE, int MT>
static int launch_skinny_mt(const bf16_t* A, int lda, const bf16_t* W, const bf16_t* W2, void* C, int ldc, int M,
                            int N, int K, hipStream_t stream) {
  int nb, wpb;
  pick_shape(N, K, MT, MODE == SK_SWIGLU, &nb, &wpb);
  const int chunks = ceil_div(K, 32), bands = ceil_div(N, 16);
#define SK_LAUNCH(NB_, WPB_)                                                                                        \
  hipLaunchKernelGGL((skinny_gemm_kernel<MT, MODE, NB_, WPB_>), dim3(ceil_div(bands, MODE == SK_SWIGLU ? 1 : NB_)), \
                     dim3(WPB_ * WAVE), 0, stream, A, lda, W, W2, chunks, C, ldc, M, N, K)
  if constexpr (MODE == SK_SWIGLU) {
    if (wpb == 4) SK_LAUNCH(2, 4);
    else if (wpb == 8 || MT > 2) SK_LAUNCH(2, 8);
    else if constexpr (MT <= 2) SK_LAUNCH(2, 16);
  } else if (nb == 2) {
    if constexpr (MT <= 2) {
      if (wpb == 4) SK_LAUNCH(2, 4);
      else SK_LAUNCH(2, 8);
    }
  } else {
    if (wpb == 4) SK_LAUNCH(1, 4);
    else if (wpb == 8) SK_LAUNCH(1, 8);
    else SK_LAUNCH(1, 16);
  }
#undef SK_LAUNCH
  APC_LAUNCH_CHECK();
  return 0;
}

template <int MODE>
static int launch_skinny(const bf16_t* A, int lda, const bf16_t* W, const bf16_t* W2, void* C, int ldc, int M, int N,
                         int K, hipStream_t stream) {
  switch (ceil_div(M, 16)) {
    case 1: return launch_skinny_mt<MODE, 1>(A, lda, W, W2, C, ldc, M, N, K, stream);
    case 2: return launch_skinny_mt<MODE, 2>(A, lda, W, W2, C, ldc, M, N, K, stream);
    case 3: return launch_skinny_mt<MODE, 3>(A, lda, W, W2, C, ldc, M, N, K, stream);
    case 4: return launch_skinny_mt<MODE, 4>(A, lda, W, W2, C, ldc, M, N, K, stream);
    default: return APC_ERR_UNSUPPORTED;
  }
}

static bool aligned16(const void* p) { return ((uintptr_t)p & 15u) == 0; }

// W: tiled layout of an [N, K] matrix.  mode: 0 store bfloat16, 1 store float32, 2 add into float32
APC_EXPORT int apc_skinny_gemm_bf16(const void* A, int lda, const void* W, void* C, int ldc, int M, int N, int K,
                                    int mode, hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (K <= 0 || lda < K || ldc < N) return APC_ERR_BAD_ARG;
  if (M > 64 || K % 8 || lda % 8 || !aligned16(A) || !aligned16(W)) return APC_ERR_UNSUPPORTED;
  const bf16_t* a = (const bf16_t*)A;
  const bf16_t* w = (const bf16_t*)W;
  switch (mode) {
    case SK_STORE_BF16: return launch_skinny<SK_STORE_BF16>(a, lda, w, nullptr, C, ldc, M, N, K, stream);
    case SK_STORE_F32: return launch_skinny<SK_STORE_F32>(a, lda, w, nullptr, C, ldc, M, N, K, stream);
    case SK_ACC_F32: return launch_skinny<SK_ACC_F32>(a, lda, w, nullptr, C, ldc, M, N, K, stream);
    default: return APC_ERR_BAD_ARG;
  }
}

// out[m, f] = silu(A[m] . Wg[f]) * (A[m] . Wu[f]);  Wg, Wu: tiled layouts of two [F, K] matrices
APC_EXPORT int apc_skinny_swiglu_bf16(const void* A, int lda, const void* Wg, const void* Wu, void* C, int ldc, int M,
                                      int F, int K, hipStream_t stream) {
  if (M <= 0 || F <= 0) return 0;
  if (K <= 0 || lda < K || ldc < F) return APC_ERR_BAD_ARG;
  if (M > 64 || K % 8 || lda % 8 || !aligned16(A) || !aligned16(Wg) || !aligned16(Wu)) return APC_ERR_UNSUPPORTED;
  return launch_skinny<SK_SWIGLU>((const bf16_t*)A, lda, (const bf16_t*)Wg, (const bf16_t*)Wu, C, ldc, M, F, K,
                                  stream);
}
