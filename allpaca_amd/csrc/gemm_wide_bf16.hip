// SwiGLU of many rows on a tile of 256 rows x (128 gate + 128 up) columns: 4 waves (2 along the rows x 2 along the
// columns), a wave computes gate and up of 128 rows x 64 outputs as 4 x 4 accumulators of v_mfma_f32_32x32x16_bf16
// (256 registers, which is why this file is compiled with the accumulators in the accumulation registers: see
// kernels/build.py).  Against the 128 x 128 tile of gemm_bf16.hip an operand read from LDS feeds twice the arithmetic
// (8 reads for 16 MFMAs instead of 4 for 4) and a tile of the weights is stored into LDS once for 256 rows instead of
// 128: LDS traffic per MFMA falls from 1.5 KiB to 0.75 KiB, and LDS bandwidth is what bounds the smaller tile.
// One block a compute unit (144 KiB of LDS), one wave a SIMD, so the wave overlaps its own work: the operands of a
// group of 16 MFMAs are read from LDS while the group before is multiplied, the next K step's pieces are asked for
// during the first two groups and stored into the other LDS buffer during the last two, and the instructions of a
// group are laid out by hand (two memory instructions, four MFMAs, and so on).  Loads go through buffer descriptors
// (base and K offset in scalar registers, a constant byte offset per lane).  K must be a multiple of 64.
// The loop over K keeps everything in registers (256 vector + 256 accumulation registers); the code of the last one or
// two steps and of the epilogue, which runs once a block, spills some values to scratch memory.
// 8B shapes, 4,096 rows: 847 us against 914 us of the 128 x 128 tile (1.14 PFLOP/s); an 8-wave version of this tile
// (128 rows x 32 outputs a wave, two waves a SIMD) was slower (925 us).
// Reference counterpart: gemm_nt_bf16_tiled_kernel, hip/src/kernels.cpp:634 (no matrix cores there).
#include <type_traits>

#include "gemm_wide.h"
#include "mfma.h"

constexpr int BK = 64;
constexpr int LDS_ROW = BK + 8;  // bfloat16 elements per LDS row (144 bytes: operand reads of 8 rows fall into different banks)
struct WideRegs {  // one K step of a thread's pieces of the tile: 8 of A, 8 of W
  Frag a[8], w[8];
};
template <bool PRE>
__global__ __launch_bounds__(256) void swiglu_wide_kernel(const bf16_t* __restrict__ A, int lda, const bf16_t* __restrict__ Wg,
                                                          const bf16_t* __restrict__ Wu, int chunks, bf16_t* __restrict__ C,
                                                          int ldc, int M, int F, int K, const float* __restrict__ pre_ss,
                                                          int pre_parts, float pre_eps) {
  __shared__ float rstd_s[PRE ? 256 : 1];
  __shared__ __attribute__((aligned(16))) bf16_t As[2][256 * LDS_ROW];
  __shared__ __attribute__((aligned(16))) bf16_t Ws[2][256 * LDS_ROW];
  const int tid = threadIdx.x, lane = tid % WAVE, wave = tid / WAVE;
  const int wm = wave / 2, wn = wave % 2;
  int mt, nt;
  {
    const int MT = ceil_div(M, 256), NT = ceil_div(F, 128), NL = ceil_div(NT, 8);
    constexpr int GM = 8;
    const int xcd = blockIdx.x % 8, j = blockIdx.x / 8;
    const int first_m = j / (GM * NL) * GM, gsz = min(MT - first_m, GM), jj = j % (GM * NL);
    mt = first_m + jj % gsz;
    nt = jj / gsz * 8 + xcd;
    if (nt >= NT || mt >= MT) return;
  }
  const int m0 = mt * 256, n0 = nt * 128;
  const int lrow = tid / 8, lchunk = tid % 8;
  const int wi = tid % 16, wc = (tid / 16) % 4, wkc = (tid / 64) % 2, wbl = tid / 128;
  const int bands = (F + 15) / 16, band0 = n0 / 16;
  const BufferRsrc abuf = make_rsrc(A + (size_t)m0 * lda);
  const BufferRsrc gbuf = make_rsrc(Wg + (size_t)band0 * chunks * 512);
  const BufferRsrc ubuf = make_rsrc(Wu + (size_t)band0 * chunks * 512);
  int aoff[8], woff[8];
#pragma unroll
  for (int p = 0; p < 8; ++p) {
    aoff[p] = ((min(m0 + p * 32 + lrow, M - 1) - m0) * lda + lchunk * 8) * 2;
    const int rel = (p % 4) * 2 + wbl;
    woff[p] = ((min(band0 + rel, bands - 1) - band0) * chunks * 512 + wkc * 512 + (wc * 16 + wi) * 8) * 2;
  }
  floatx16 acc[4][4];
#pragma unroll
  for (int a = 0; a < 4; ++a)
#pragma unroll
    for (int b = 0; b < 4; ++b)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[a][b][r] = 0.f;
  auto load_piece = [&](WideRegs& g, int kt, int j) {
    if (j < 8) g.a[j] = load_frag_buffer(abuf, aoff[j], kt * (BK * 2));
    else g.w[j - 8] = load_frag_buffer(j - 8 < 4 ? gbuf : ubuf, woff[j - 8], kt * 2048);
  };
  auto store_piece = [&](const WideRegs& g, int buf, int j) {
    if (j < 8) *reinterpret_cast<Frag*>(&As[buf][(j * 32 + lrow) * LDS_ROW + lchunk * 8]) = g.a[j];
    else {
      const int p = j - 8;
      *reinterpret_cast<Frag*>(&Ws[buf][((p * 2 + wbl) * 16 + wi) * LDS_ROW + wkc * 32 + wc * 8]) = g.w[p];
    }
  };
  const int li = lane % 32, lc = lane / 32;
  WideRegs regs;
  Frag fa[2][4], fw[2][4];
  auto read_group = [&](int set, int buf, int kk) {
#pragma unroll
    for (int t = 0; t < 4; ++t)  // 0, 1: gate columns wn*64 + t*32; 2, 3: the up columns of the same outputs
      fw[set][t] = *reinterpret_cast<const Frag*>(&Ws[buf][((t / 2) * 128 + wn * 64 + (t % 2) * 32 + li) * LDS_ROW + kk * 16 + lc * 8]);
#pragma unroll
    for (int a = 0; a < 4; ++a)
      fa[set][a] = *reinterpret_cast<const Frag*>(&As[buf][(wm * 128 + a * 32 + li) * LDS_ROW + kk * 16 + lc * 8]);
  };
  auto step = [&](auto NEXT, int buf, int kt_next) {
    read_group(0, buf, 0);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int kk = 0; kk < 4; ++kk) {
      if constexpr (decltype(NEXT)::value) {
        if (kk < 2) {
#pragma unroll
          for (int j = kk * 8; j < kk * 8 + 8; ++j) load_piece(regs, kt_next, j);
        }
      }
      if (kk < 3) read_group((kk + 1) % 2, buf, kk + 1);
#pragma unroll
      for (int a = 0; a < 4; ++a)
#pragma unroll
        for (int b = 0; b < 4; ++b) acc[a][b] = mfma32(fa[kk % 2][a], fw[kk % 2][b], acc[a][b]);
      if constexpr (decltype(NEXT)::value) {
        if (kk >= 2) {
#pragma unroll
          for (int j = (kk - 2) * 8; j < (kk - 2) * 8 + 8; ++j) store_piece(regs, buf ^ 1, j);
        }
      }
      // the order inside the group: a few memory instructions, four MFMAs, and so on
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        if (decltype(NEXT)::value && kk < 2) __builtin_amdgcn_sched_group_barrier(0x020, 2, 0);   // 2 global loads
        if (kk < 3) __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);                            // 2 LDS reads
        if (decltype(NEXT)::value && kk >= 2) __builtin_amdgcn_sched_group_barrier(0x200, 2, 0);  // 2 LDS writes
        __builtin_amdgcn_sched_group_barrier(0x008, 4, 0);                                        // 4 MFMAs
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  constexpr std::true_type yes{};
  constexpr std::false_type no{};
  const int ktiles = K / BK;
  if (ktiles > 0) {
#pragma unroll
    for (int j = 0; j < 16; ++j) load_piece(regs, 0, j);
#pragma unroll
    for (int j = 0; j < 16; ++j) store_piece(regs, 0, j);
    if constexpr (PRE) {  // one row a thread, its parts added in order, 8 loads at a time
      const float* row = pre_ss + (size_t)min(m0 + tid, M - 1) * pre_parts;
      float sum = 0.f;
      for (int p0 = 0; p0 < pre_parts; p0 += 8) {
        float v[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) v[j] = p0 + j < pre_parts ? row[p0 + j] : 0.f;
#pragma unroll
        for (int j = 0; j < 8; ++j) sum += v[j];
      }
      rstd_s[tid] = 1.0f / sqrtf(sum / (float)K + pre_eps);
    }
    __syncthreads();
    int kt = 0;
    while (kt + 2 < ktiles) {
      step(yes, 0, kt + 1);
      __syncthreads();
      step(yes, 1, kt + 2);
      __syncthreads();
      kt += 2;
    }
    if (kt + 1 < ktiles) {
      step(yes, 0, kt + 1);
      __syncthreads();
      step(no, 1, 0);
    } else {
      step(no, 0, 0);
    }
  }
#pragma unroll
  for (int a = 0; a < 4; ++a)
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      const int n = n0 + wn * 64 + t * 32 + li;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int m = m0 + wm * 128 + a * 32 + (r / 4) * 8 + lc * 4 + (r % 4);
        if (m >= M || n >= F) continue;
        float g = acc[a][t][r], u = acc[a][2 + t][r];
        if constexpr (PRE) {
          const float rs = rstd_s[m - m0];
          g *= rs;
          u *= rs;
        }
        C[(size_t)m * ldc + n] = float_to_bf16(silu_f(g) * u);
      }
    }
}
int launch_swiglu_wide(const bf16_t* A, int lda, const bf16_t* Wg, const bf16_t* Wu, bf16_t* C, int ldc, int M, int F,
                       int K, const float* pre_ss, int pre_parts, float pre_eps, hipStream_t stream) {
  if (M <= 0 || F <= 0) return 0;
  if (K <= 0 || K % BK || lda < K || ldc < F) return APC_ERR_BAD_ARG;
  // the lanes' byte offsets into the tile's rows of A and bands of W are 32-bit
  if ((long)256 * lda * 2 >= 0x7fffffffL || (long)8 * ceil_div(K, 32) * 1024 >= 0x7fffffffL) return APC_ERR_UNSUPPORTED;
  const long blocks = 8L * ceil_div(ceil_div(F, 128), 8) * ceil_div(M, 256);
  if (blocks > 0x7fffffffL) return APC_ERR_BAD_ARG;
  if (pre_ss)
    hipLaunchKernelGGL((swiglu_wide_kernel<true>), dim3((unsigned)blocks), dim3(256), 0, stream, A, lda, Wg, Wu,
                       ceil_div(K, 32), C, ldc, M, F, K, pre_ss, pre_parts, pre_eps);
  else
    hipLaunchKernelGGL((swiglu_wide_kernel<false>), dim3((unsigned)blocks), dim3(256), 0, stream, A, lda, Wg, Wu,
                       ceil_div(K, 32), C, ldc, M, F, K, nullptr, 0, 0.f);
  APC_LAUNCH_CHECK();
  return 0;
}
