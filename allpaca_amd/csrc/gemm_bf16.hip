// Matrix product for many rows (prefill):  C[M,N] = A[M,K] . W[N,K]^T, bfloat16 in, float32 sums on MFMA.
//
// W is stored in tiles of 16 rows x 32 columns in the lane order of an MFMA operand (see
// skinny_gemm_bf16.hip; the decode kernel streams that layout); here a wave copies such a tile with one
// contiguous 1 KiB load into a row-major LDS tile.
// A block of 256 threads (4 waves, 2 x 2) computes a 128 x 128 tile of C; K runs in steps of 64
// through a double-buffered LDS tile of A and of W (rows padded by 16 bytes so that the 16-byte
// operand reads of 8 consecutive rows fall into different banks).  Each wave owns 64 x 64 of the tile
// as 2 x 2 v_mfma_f32_32x32x16_bf16 accumulators.  Global loads of the next K step are issued before
// the MFMAs of the current one and stored to the other LDS buffer after them.
// Epilogues: store bfloat16 / float32, add into a float32 residual, or SwiGLU: then the W tile is
// 64 gate rows and the matching 64 up rows, each wave computes gate and up of the same 64 x 32 outputs,
// and the block writes a 128 x 64 tile of silu(gate) * up.
// The K order of every output is fixed (k = 0, 16, 32, ... inside one accumulator), whatever M.
// Reference counterpart: gemm_nt_bf16_tiled_kernel, hip/src/kernels.cpp:634 (no matrix cores there).
#include "mfma.h"

constexpr int BM = 128, BN = 128, BK = 64;
constexpr int LDS_ROW = BK + 8;  // bfloat16 elements per LDS row (144 bytes)

enum { G_STORE_BF16 = 0, G_STORE_F32 = 1, G_ACC_F32 = 2, G_SWIGLU = 3 };

template <int MODE>
__global__ __launch_bounds__(256) void gemm_bf16_kernel(const bf16_t* __restrict__ A, int lda,
                                                        const bf16_t* __restrict__ W,
                                                        const bf16_t* __restrict__ W2, int chunks,
                                                        void* __restrict__ C, int ldc, int M, int N, int K) {
  __shared__ __attribute__((aligned(16))) bf16_t As[2][BM * LDS_ROW];
  __shared__ __attribute__((aligned(16))) bf16_t Ws[2][BN * LDS_ROW];
  const int tid = threadIdx.x, lane = tid % WAVE, wave = tid / WAVE;
  const int wm = wave / 2, wn = wave % 2;
  const int m0 = blockIdx.y * BM;
  // N per block: 128 output columns, or 64 (gate and up) in SwiGLU mode
  constexpr int NB = MODE == G_SWIGLU ? BN / 2 : BN;
  const int n0 = blockIdx.x * NB;

  // global -> registers: 128 rows x 64 k per operand = 1024 pieces of 16 bytes, 4 per thread and operand.
  // A (row-major): thread -> (row within a group of 32, piece within the 128-byte row).
  // W (tiled): a wave copies one 16 x 32 tile per pass: thread -> (row in band, 8-column piece, which of the
  // two tiles along K, which of two bands); 4 passes cover the 8 bands of the block tile.
  const int lrow = tid / 8, lchunk = tid % 8;
  const int wi = tid % 16, wc = (tid / 16) % 4, wkc = (tid / 64) % 2, wbl = tid / 128;
  const int bands = (N + 15) / 16;
  const bf16_t* aptr[4];
  const bf16_t* wptr[4];
#pragma unroll
  for (int p = 0; p < 4; ++p) {
    aptr[p] = A + (size_t)min(m0 + p * 32 + lrow, M - 1) * lda + lchunk * 8;
    const int bl = p * 2 + wbl;  // band of the block tile, 0..7
    int band;
    const bf16_t* base = W;
    if (MODE == G_SWIGLU) {
      band = n0 / 16 + (bl % 4);
      base = bl < 4 ? W : W2;
    } else {
      band = n0 / 16 + bl;
    }
    wptr[p] = base + ((size_t)min(band, bands - 1) * chunks + wkc) * 512 + (wc * 16 + wi) * 8;
  }

  floatx16 acc[2][2];
#pragma unroll
  for (int a = 0; a < 2; ++a)
#pragma unroll
    for (int b = 0; b < 2; ++b)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[a][b][r] = 0.f;

  Frag ra[4], rw[4];
  auto load_global = [&](int k0) {
    const bool in = k0 + lchunk * 8 < K;  // K is a multiple of 8: a piece is inside or outside as a whole
    const bool win = k0 / 32 + wkc < chunks;  // W is zero-padded up to whole tiles
#pragma unroll
    for (int p = 0; p < 4; ++p) {
      ra[p] = in ? load_frag(aptr[p] + k0) : zero_frag();
      rw[p] = win ? load_frag(wptr[p] + (size_t)(k0 / 32) * 512) : zero_frag();
    }
  };
  auto store_lds = [&](int buf) {
#pragma unroll
    for (int p = 0; p < 4; ++p) {
      *reinterpret_cast<Frag*>(&As[buf][(p * 32 + lrow) * LDS_ROW + lchunk * 8]) = ra[p];
      *reinterpret_cast<Frag*>(&Ws[buf][((p * 2 + wbl) * 16 + wi) * LDS_ROW + wkc * 32 + wc * 8]) = rw[p];
    }
  };

  const int ktiles = ceil_div(K, BK);
  load_global(0);
  store_lds(0);
  __syncthreads();
  const int li = lane % 32, lc = lane / 32;
  for (int kt = 0; kt < ktiles; ++kt) {
    const int buf = kt & 1;
    if (kt + 1 < ktiles) load_global((kt + 1) * BK);
#pragma unroll
    for (int kk = 0; kk < BK / 16; ++kk) {
      Frag fa[2], fw[2];
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        fa[t] = *reinterpret_cast<const Frag*>(&As[buf][(wm * 64 + t * 32 + li) * LDS_ROW + kk * 16 + lc * 8]);
        // SwiGLU: tile 0 = gate rows wn*32.., tile 1 = the up rows of the same outputs
        const int wrow = MODE == G_SWIGLU ? t * 64 + wn * 32 + li : wn * 64 + t * 32 + li;
        fw[t] = *reinterpret_cast<const Frag*>(&Ws[buf][wrow * LDS_ROW + kk * 16 + lc * 8]);
      }
#pragma unroll
      for (int a = 0; a < 2; ++a)
#pragma unroll
        for (int b = 0; b < 2; ++b) acc[a][b] = mfma32(fa[a], fw[b], acc[a][b]);
    }
    if (kt + 1 < ktiles) store_lds(buf ^ 1);
    __syncthreads();
  }

  // D[i][j]: i = row of A (m), j = row of W (n); lane holds column j = lane%32 and rows (r/4)*8 + (lane/32)*4 + r%4
#pragma unroll
  for (int a = 0; a < 2; ++a) {
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int m = m0 + wm * 64 + a * 32 + (r / 4) * 8 + lc * 4 + (r % 4);
      if (m >= M) continue;
      if (MODE == G_SWIGLU) {
        const int n = n0 + wn * 32 + li;
        if (n < N) ((bf16_t*)C)[(size_t)m * ldc + n] = float_to_bf16(silu_f(acc[a][0][r]) * acc[a][1][r]);
      } else {
#pragma unroll
        for (int b = 0; b < 2; ++b) {
          const int n = n0 + wn * 64 + b * 32 + li;
          if (n >= N) continue;
          const size_t o = (size_t)m * ldc + n;
          if (MODE == G_STORE_BF16) ((bf16_t*)C)[o] = float_to_bf16(acc[a][b][r]);
          else if (MODE == G_STORE_F32) ((float*)C)[o] = acc[a][b][r];
          else ((float*)C)[o] += acc[a][b][r];
        }
      }
    }
  }
}

static bool aligned16(const void* p) { return ((uintptr_t)p & 15u) == 0; }

template <int MODE>
static int launch_gemm(const bf16_t* A, int lda, const bf16_t* W, const bf16_t* W2, void* C, int ldc, int M, int N,
                       int K, hipStream_t stream) {
  constexpr int NB = MODE == G_SWIGLU ? BN / 2 : BN;
  const int gy = ceil_div(M, BM);
  if (gy > 65535) return APC_ERR_BAD_ARG;
  hipLaunchKernelGGL((gemm_bf16_kernel<MODE>), dim3(ceil_div(N, NB), gy), dim3(256), 0, stream, A, lda, W, W2,
                     ceil_div(K, 32), C, ldc, M, N, K);
  APC_LAUNCH_CHECK();
  return 0;
}

// W: tiled layout of an [N, K] matrix.  mode: 0 store bfloat16, 1 store float32, 2 add into float32
APC_EXPORT int apc_gemm_bf16(const void* A, int lda, const void* W, void* C, int ldc, int M, int N, int K, int mode,
                             hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (K <= 0 || lda < K || ldc < N) return APC_ERR_BAD_ARG;
  if (K % 8 || lda % 8 || !aligned16(A) || !aligned16(W)) return APC_ERR_UNSUPPORTED;
  const bf16_t* a = (const bf16_t*)A;
  const bf16_t* w = (const bf16_t*)W;
  switch (mode) {
    case G_STORE_BF16: return launch_gemm<G_STORE_BF16>(a, lda, w, nullptr, C, ldc, M, N, K, stream);
    case G_STORE_F32: return launch_gemm<G_STORE_F32>(a, lda, w, nullptr, C, ldc, M, N, K, stream);
    case G_ACC_F32: return launch_gemm<G_ACC_F32>(a, lda, w, nullptr, C, ldc, M, N, K, stream);
    default: return APC_ERR_BAD_ARG;
  }
}

APC_EXPORT int apc_gemm_swiglu_bf16(const void* A, int lda, const void* Wg, const void* Wu, void* C, int ldc, int M,
                                    int F, int K, hipStream_t stream) {
  if (M <= 0 || F <= 0) return 0;
  if (K <= 0 || lda < K || ldc < F) return APC_ERR_BAD_ARG;
  if (K % 8 || lda % 8 || !aligned16(A) || !aligned16(Wg) || !aligned16(Wu)) return APC_ERR_UNSUPPORTED;
  return launch_gemm<G_SWIGLU>((const bf16_t*)A, lda, (const bf16_t*)Wg, (const bf16_t*)Wu, C, ldc, M, F, K, stream);
}
