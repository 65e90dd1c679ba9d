// Matrix product for many rows (prefill):  C[M,N] = A[M,K] . W[N,K]^T, bfloat16 in, float32 sums on MFMA.
//
// W is stored in tiles of 16 rows x 32 columns in the lane order of an MFMA operand (see
// skinny_gemm_bf16.hip; the decode kernel streams that layout); here a wave copies such a tile with one
// contiguous 1 KiB load into a row-major LDS tile.
// A block of 256 threads (4 waves, 2 x 2) computes a 128 x 128 tile of C; K runs in steps of 64
// through a double-buffered LDS tile of A and of W (rows padded by 16 bytes so that the 16-byte
// operand reads of 8 consecutive rows fall into different banks).  Each wave owns a quarter of the tile
// as 2 x 2 v_mfma_f32_32x32x16_bf16 accumulators.  Global loads run two K steps ahead of the MFMAs, and
// loads and LDS stores are spread between the MFMAs of a step: LDS bandwidth (reads of operands plus stores of
// the next step) and the load path are each about as busy as the matrix cores, so none of them may wait for another.
// Epilogues: store bfloat16 / float32, add into a float32 residual, or SwiGLU: then the W tile is
// 64 gate rows and the matching 64 up rows, each wave computes gate and up of the same 64 x 32 outputs,
// and the block writes a 128 x 64 tile of silu(gate) * up.
// With 17..128 rows and a long K, K is cut into slices for different blocks and a second kernel adds the slices in
// order.  The order of additions for an output depends on N, K and on whether the step has up to 128 rows or more,
// never on which other rows are in the batch.
// Reference counterpart: gemm_nt_bf16_tiled_kernel, hip/src/kernels.cpp:634 (no matrix cores there).
#include <type_traits>

#include "gemm_direct.h"
#include "gemm_wide.h"
#include "mfma.h"

constexpr int BN = 128, BK = 64;
// Rows of the block tile (the split path also uses 64).  256 rows (4 x 2 accumulators a wave, one block a compute
// unit) were tried on the shapes of an 8B model with 2,048 rows: no faster than two 128-row blocks sharing a unit.
constexpr int BM_ROWS = 128;
constexpr int LDS_ROW = BK + 8;  // bfloat16 elements per LDS row (144 bytes)

enum { G_STORE_BF16 = 0, G_STORE_F32 = 1, G_ACC_F32 = 2, G_SWIGLU = 3, G_PARTIAL = 4 };

template <int BM>
struct GemmRegs {
  Frag a[BM / 32], w[4];
};

// PRE (storing modes): A is the row bfloat16(x * g) that a product into the residual left for the RMS norm, and
// ss[m][parts] are its sums of x^2 per row and block of columns; the sums of this product are scaled by
// 1 / sqrt(sum(ss[m]) / K + eps): the product of the normalised row without a kernel for the norm.
struct TiledPre {
  const float* ss;
  int parts;
  float eps;
};

// EVEN_K: K is a multiple of 64, so no load needs a bound check.  BM: rows of the block tile, 64 or 128.
// DEPTH (even): how many K steps the global loads run ahead of the MFMAs, one register set a step.  2 where two blocks
// share a compute unit (many rows); 4 for the steps of up to 128 rows, whose blocks have a unit each and stream the
// weights once: what they have in flight sets their pace (a block of 64 rows x 64 SwiGLU outputs with 2 steps in
// flight took 0.8 us a step of 16 KiB of weights).
template <int MODE, bool EVEN_K, int BM, bool PRE = false, int DEPTH = 2>
__global__ __launch_bounds__(256) void gemm_bf16_kernel(const bf16_t* __restrict__ A, int lda,
                                                        const bf16_t* __restrict__ W,
                                                        const bf16_t* __restrict__ W2, int chunks,
                                                        void* __restrict__ C, int ldc, int M, int N, int K,
                                                        int k_split, TiledPre pre = TiledPre{}) {
  static_assert(!PRE || MODE == G_STORE_BF16 || MODE == G_STORE_F32 || MODE == G_SWIGLU,
                "a product that reads a normalised row stores its result");
  __shared__ float rstd_s[PRE ? BM : 1];
  constexpr int AP = BM / 32;          // 16-byte pieces of A per thread and K step
  constexpr int WM = BM / 64;          // 32-row accumulators of a wave along M
  constexpr int PIECES = AP + 4;       // pieces of A and W per thread and K step
  constexpr int PER_GROUP = (PIECES + 3) / 4;
  __shared__ __attribute__((aligned(16))) bf16_t As[2][BM * LDS_ROW];
  __shared__ __attribute__((aligned(16))) bf16_t Ws[2][BN * LDS_ROW];
  const int tid = threadIdx.x, lane = tid % WAVE, wave = tid / WAVE;
  const int wm = wave / 2, wn = wave % 2;
  // N per block: 128 output columns, or 64 (gate and up) in SwiGLU mode
  constexpr int NB = MODE == G_SWIGLU ? BN / 2 : BN;
  int mt, nt;
  if (MODE == G_PARTIAL) {
    mt = blockIdx.y;
    nt = blockIdx.x;
  } else {
    // Order of the blocks: consecutive block ids go to the 8 XCDs in turn, each with an L2 of its own.  XCD x takes
    // the column tiles x, x+8, ..; inside it, groups of up to 8 row tiles sweep those columns, row tile fastest, so
    // the blocks that run on an XCD at one time share a few tiles of W and of A.
    const int MT = ceil_div(M, BM), NT = ceil_div(N, NB), NL = ceil_div(NT, 8);
    constexpr int GM = 8;
    const int xcd = blockIdx.x % 8, j = blockIdx.x / 8;
    const int first_m = j / (GM * NL) * GM, gsz = min(MT - first_m, GM), jj = j % (GM * NL);
    mt = first_m + jj % gsz;
    nt = jj / gsz * 8 + xcd;
    if (nt >= NT || mt >= MT) return;
  }
  const int m0 = mt * BM, n0 = nt * NB;
  // G_PARTIAL: blockIdx.z = which * k_split + slice; the block multiplies slice `slice` of K with matrix `which`
  // (0: W, 1: W2) and leaves its float32 sums in C[which][slice][M][N]
  const int slice = MODE == G_PARTIAL ? blockIdx.z % k_split : 0;
  const int which = MODE == G_PARTIAL ? blockIdx.z / k_split : 0;
  if (MODE == G_PARTIAL && which) W = W2;

  // global -> registers: BM rows of A and 128 rows of W x 64 k = pieces of 16 bytes, BM/32 + 4 per thread.
  // A (row-major): thread -> (row within a group of 32, piece within the 128-byte row).
  // W (tiled): a wave copies one 16 x 32 tile per pass: thread -> (row in band, 8-column piece, which of the
  // two tiles along K, which of two bands); 4 passes cover the 8 bands of the block tile.
  // Addresses are a base that is the same for the whole block (it moves along K) plus a small offset per thread.
  const int lrow = tid / 8, lchunk = tid % 8;
  const int wi = tid % 16, wc = (tid / 16) % 4, wkc = (tid / 64) % 2, wbl = tid / 128;
  const int bands = (N + 15) / 16;
  const int band0 = n0 / 16;
  const bf16_t* abase = A + (size_t)m0 * lda;
  const bf16_t* wbase0 = W + (size_t)band0 * chunks * 512;
  const bf16_t* wbase1 = (MODE == G_SWIGLU ? W2 : W) + (size_t)band0 * chunks * 512;  // passes 2, 3
  unsigned aoff[AP], woff[4];
#pragma unroll
  for (int p = 0; p < AP; ++p) aoff[p] = (unsigned)(min(m0 + p * 32 + lrow, M - 1) - m0) * lda + lchunk * 8;
#pragma unroll
  for (int p = 0; p < 4; ++p) {
    const int bl = p * 2 + wbl;                               // band of the block tile, 0..7
    const int rel = MODE == G_SWIGLU ? bl % 4 : bl;           // SwiGLU: 4 gate bands, then the same 4 up bands
    woff[p] = (unsigned)(min(band0 + rel, bands - 1) - band0) * chunks * 512 + wkc * 512 + (wc * 16 + wi) * 8;
  }

  floatx16 acc[WM][2];
#pragma unroll
  for (int a = 0; a < WM; ++a)
#pragma unroll
    for (int b = 0; b < 2; ++b)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[a][b][r] = 0.f;

  // piece j of K step kt (64 columns): j < AP a piece of A, else of W
  auto load_piece = [&](GemmRegs<BM>& g, int kt, int j) {
    if (j < AP) {
      const bf16_t* src = abase + kt * BK + aoff[j];
      // K is a multiple of 8: a piece is inside or outside as a whole
      g.a[j] = (EVEN_K || kt * BK + lchunk * 8 < K) ? load_frag(src) : zero_frag();
    } else {
      const int p = j - AP;
      const bf16_t* src = (p < 2 ? wbase0 : wbase1) + (size_t)kt * 1024 + woff[p];
      // W is zero-padded to whole tiles.  With up to 128 rows a weight is read once, by this block: a load that the
      // caches do not keep, where the block walks all of K (SwiGLU of 64 rows at 8B shapes 45.2 -> 42.5 us; with K in
      // slices the short runs of a slice were slower that way, o_proj of 64 rows 15.9 -> 17.9 us)
      constexpr bool ONCE = DEPTH > 2 && MODE != G_PARTIAL;
      g.w[p] = (EVEN_K || kt * 2 + wkc < chunks) ? (ONCE ? load_frag_once(src) : load_frag(src)) : zero_frag();
    }
  };
  auto store_piece = [&](const GemmRegs<BM>& g, int buf, int j) {
    if (j < AP) {
      *reinterpret_cast<Frag*>(&As[buf][(j * 32 + lrow) * LDS_ROW + lchunk * 8]) = g.a[j];
    } else {
      const int p = j - AP;
      *reinterpret_cast<Frag*>(&Ws[buf][((p * 2 + wbl) * 16 + wi) * LDS_ROW + wkc * 32 + wc * 8]) = g.w[p];
    }
  };
  const int li = lane % 32, lc = lane / 32;
  // One K step out of LDS buffer `buf` in four groups of MFMAs.  Between the groups the loads of step `kt_load` go
  // out into `ld` (if LD) and the pieces of `st`, loaded a step earlier, go into the other LDS buffer (if ST): the
  // memory pipeline and LDS work while the matrix cores do, instead of in a burst around the barrier.
  auto step = [&](auto LD, auto ST, int buf, GemmRegs<BM>& ld, int kt_load, const GemmRegs<BM>& st) {
#pragma unroll
    for (int kk = 0; kk < BK / 16; ++kk) {
      if constexpr (decltype(LD)::value) {
#pragma unroll
        for (int j = kk * PER_GROUP; j < (kk + 1) * PER_GROUP; ++j)
          if (j < PIECES) load_piece(ld, kt_load, j);
      }
      Frag fa[WM], fw[2];
#pragma unroll
      for (int t = 0; t < WM; ++t)
        fa[t] = *reinterpret_cast<const Frag*>(&As[buf][(wm * (BM / 2) + t * 32 + li) * LDS_ROW + kk * 16 + lc * 8]);
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        // SwiGLU: tile 0 = gate rows wn*32.., tile 1 = the up rows of the same outputs
        const int wrow = MODE == G_SWIGLU ? t * 64 + wn * 32 + li : wn * 64 + t * 32 + li;
        fw[t] = *reinterpret_cast<const Frag*>(&Ws[buf][wrow * LDS_ROW + kk * 16 + lc * 8]);
      }
#pragma unroll
      for (int a = 0; a < WM; ++a)
#pragma unroll
        for (int b = 0; b < 2; ++b) acc[a][b] = mfma32(fa[a], fw[b], acc[a][b]);
      if constexpr (decltype(ST)::value) {
#pragma unroll
        for (int j = kk * PER_GROUP; j < (kk + 1) * PER_GROUP; ++j)
          if (j < PIECES) store_piece(st, buf ^ 1, j);
      }
      __builtin_amdgcn_sched_barrier(0);  // keeps each group's memory work in its group
    }
  };
  constexpr std::true_type yes{};
  constexpr std::false_type no{};

  const int all_tiles = ceil_div(K, BK);
  const int per_slice = MODE == G_PARTIAL ? ceil_div(all_tiles, k_split) : all_tiles;
  const int kt0 = slice * per_slice;
  const int ktiles = max(0, min(all_tiles, kt0 + per_slice) - kt0);
  // K steps are loaded DEPTH ahead: while step t is multiplied out of one LDS buffer, step t+1 moves from registers
  // into the other and the loads of step t+DEPTH go out (register set t % DEPTH, whose step went into LDS a step
  // ago).  The steady loop has no branch around a load, so the waits for one set never wait for another: near the end
  // of K it loads the last step again instead.
  static_assert(DEPTH >= 2 && DEPTH % 2 == 0, "the LDS buffer of a step is its register set's parity");
  if (ktiles > 0) {
    GemmRegs<BM> s[DEPTH];
    const int last = kt0 + ktiles - 1;
#pragma unroll
    for (int j = 0; j < PIECES; ++j) load_piece(s[0], kt0, j);
#pragma unroll
    for (int dd = 1; dd < DEPTH; ++dd)
#pragma unroll
      for (int j = 0; j < PIECES; ++j) load_piece(s[dd], min(kt0 + dd, last), j);
#pragma unroll
    for (int j = 0; j < PIECES; ++j) store_piece(s[0], 0, j);
    if constexpr (PRE) {  // behind the first loads of the tiles: one row a thread, its parts added in order, 8 loads
      if (tid < BM) {     // at a time; read after the barriers of the K loop
        const float* row = pre.ss + (size_t)min(m0 + tid, M - 1) * pre.parts;
        float sum = 0.f;
        for (int p0 = 0; p0 < pre.parts; p0 += 8) {
          float v[8];
#pragma unroll
          for (int j = 0; j < 8; ++j) v[j] = p0 + j < pre.parts ? row[p0 + j] : 0.f;
#pragma unroll
          for (int j = 0; j < 8; ++j) sum += v[j];
        }
        rstd_s[tid] = 1.0f / sqrtf(sum / (float)K + pre.eps);
      }
    }
    __syncthreads();
    int kt = 0;
    for (; kt + DEPTH < ktiles; kt += DEPTH) {  // whole rounds of the register sets with a step behind them
#pragma unroll
      for (int dd = 0; dd < DEPTH; ++dd) {
        step(yes, yes, dd & 1, s[dd], min(kt0 + kt + dd + DEPTH, last), s[(dd + 1) % DEPTH]);
        __syncthreads();
      }
    }
    // 1..DEPTH steps left, all loaded: step kt in LDS buffer 0, the others in their sets
#pragma unroll
    for (int dd = 0; dd < DEPTH; ++dd) {
      if (kt + dd + 1 < ktiles) {
        step(no, yes, dd & 1, s[dd], 0, s[(dd + 1) % DEPTH]);
        __syncthreads();
      } else if (kt + dd < ktiles) {
        step(no, no, dd & 1, s[dd], 0, s[dd]);
      }
    }
  }

  // D[i][j]: i = row of A (m), j = row of W (n); lane holds column j = lane%32 and rows (r/4)*8 + (lane/32)*4 + r%4
  if constexpr (MODE == G_ACC_F32) {
    // all loads of the residual first, then the sums and the stores: a store between two loads would make the second
    // wait (the compiler cannot tell that the addresses differ); 13 us of 98 on a 2048 x 4096 x 4096 product
    bool n_in[2];
#pragma unroll
    for (int b = 0; b < 2; ++b) n_in[b] = n0 + wn * 64 + b * 32 + li < N;
#pragma unroll
    for (int a = 0; a < WM; ++a) {
      float cv[16][2];
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int m = m0 + wm * (BM / 2) + a * 32 + (r / 4) * 8 + lc * 4 + (r % 4);
#pragma unroll
        for (int b = 0; b < 2; ++b)
          cv[r][b] = (m < M && n_in[b]) ? ((const float*)C)[(size_t)m * ldc + n0 + wn * 64 + b * 32 + li] : 0.f;
      }
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int m = m0 + wm * (BM / 2) + a * 32 + (r / 4) * 8 + lc * 4 + (r % 4);
#pragma unroll
        for (int b = 0; b < 2; ++b)
          if (m < M && n_in[b]) ((float*)C)[(size_t)m * ldc + n0 + wn * 64 + b * 32 + li] = cv[r][b] + acc[a][b][r];
      }
    }
    return;
  }
#pragma unroll
  for (int a = 0; a < WM; ++a) {
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int m = m0 + wm * (BM / 2) + a * 32 + (r / 4) * 8 + lc * 4 + (r % 4);
      if (m >= M) continue;
      if constexpr (PRE) {
        const float rs = rstd_s[m - m0];
        acc[a][0][r] *= rs;
        acc[a][1][r] *= rs;
      }
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
          else if (MODE == G_ACC_F32) ((float*)C)[o] += acc[a][b][r];
          else ((float*)C)[((size_t)blockIdx.z * M + m) * N + n] = acc[a][b][r];
        }
      }
    }
  }
}

static bool aligned16(const void* p) { return ((uintptr_t)p & 15u) == 0; }

template <int MODE, bool PRE = false>
static int launch_gemm(const bf16_t* A, int lda, const bf16_t* W, const bf16_t* W2, void* C, int ldc, int M, int N,
                       int K, hipStream_t stream, TiledPre pre = TiledPre{}) {
  constexpr int NB = MODE == G_SWIGLU ? BN / 2 : BN;
  if constexpr (!PRE) {
    // many rows, K a multiple of 128: the kernel that keeps the weights out of LDS (same sums, bit for bit)
    if (gemm_direct_takes(MODE, A, lda, C, ldc, M, N, K)) return launch_gemm_direct(MODE, A, lda, W, W2, C, ldc, M, N, K, stream);
  } else if constexpr (MODE == G_SWIGLU || MODE == G_STORE_BF16) {
    if (gemm_direct_pre_takes(MODE, A, lda, C, ldc, M, N, K, pre.parts))
      return launch_gemm_direct_pre(MODE, A, lda, pre.ss, pre.parts, pre.eps, W, W2, C, ldc, M, N, K, stream);
  }
  if constexpr (MODE == G_SWIGLU) {
    // From 1,024 rows on the tile of 256 rows x 128 outputs takes as many columns as make whole rounds of one tile a
    // compute unit (at least two rounds), and the 128-row tile, two blocks a unit and so finer grained, the rest:
    // 2,048 rows x 14,336 outputs are 3.5 rounds of big tiles, of which 3 run as such (96 of 112 column tiles).
    const int MT = ceil_div(M, 256), NT = ceil_div(N, 128);
    const long rounds = (long)MT * NT / 256;
    if (M >= 1024 && K % BK == 0 && rounds >= 2 && MT <= 256 && (long)256 * lda * 2 < 0x7fffffffL) {
      const int cols_big = (int)((rounds * 256 / MT < NT ? rounds * 256 / MT : NT));  // column tiles of the big kernel
      const int n_big = cols_big * 128 < N ? cols_big * 128 : N;
      const int e = launch_swiglu_wide(A, lda, W, W2, (bf16_t*)C, ldc, M, n_big, K, PRE ? pre.ss : nullptr, pre.parts,
                                       pre.eps, stream);
      if (e) return e;
      if (n_big == N) return 0;
      const size_t w_skip = (size_t)(n_big / 16) * ceil_div(K, 32) * 512;  // whole bands of the tiled layout
      W += w_skip;
      W2 += w_skip;
      C = (bf16_t*)C + n_big;
      N -= n_big;
    }
  }
  // up to 128 rows (a decode step of many requests, a short portion): a block has a compute unit to itself and streams
  // its weights once, so its loads run 4 steps ahead; up to 64 rows on tiles of 64 rows (half the loads of activations
  // and half the MFMAs)
  const int bm = M <= 64 ? 64 : BM_ROWS;
  const long blocks = 8L * ceil_div(ceil_div(N, NB), 8) * ceil_div(M, bm);
  if (blocks > 0x7fffffffL) return APC_ERR_BAD_ARG;
#define TILED_LAUNCH(EVEN_, BM_, DEPTH_)                                                                              \
  hipLaunchKernelGGL((gemm_bf16_kernel<MODE, EVEN_, BM_, PRE, DEPTH_>), dim3((unsigned)blocks), dim3(256), 0, stream, A, \
                     lda, W, W2, ceil_div(K, 32), C, ldc, M, N, K, 1, pre)
#define TILED_BY_K(BM_, DEPTH_)                     \
  if (K % BK == 0) TILED_LAUNCH(true, BM_, DEPTH_); \
  else TILED_LAUNCH(false, BM_, DEPTH_)
  if (M <= 64) { TILED_BY_K(64, 4); }
  else if (M <= 128) { TILED_BY_K(BM_ROWS, 4); }
  else { TILED_BY_K(BM_ROWS, 2); }
#undef TILED_BY_K
#undef TILED_LAUNCH
  APC_LAUNCH_CHECK();
  return 0;
}

// What the folded RMS norm needs in the finishing kernel (see skinny_gemm_bf16.hip for the idea).
// PRE: the activations were the row bfloat16(x * g) that an emitting product left; pre_ss[m][pre_parts] are that
// product's sums of x^2 per row and block of 256 columns; the sums of this product are scaled by
// 1 / sqrt(sum(pre_ss[m]) / K + eps).  EMIT (mode G_ACC_F32): beside C = x the kernel writes raw[m, n] =
// bfloat16(x * g[n]) and emit_ss[m][blocks of 256 columns] = sums of x^2.
struct FinishNorm {
  const float* pre_ss;
  int pre_parts;
  float eps;
  const float* g;
  bf16_t* raw;
  int ld_raw;
  float* emit_ss;
};

// Sums the float32 sums that G_PARTIAL blocks left ([which][slice][M][N], slices in order) and finishes:
// store bfloat16 / float32, add into a float32 residual, or SwiGLU of the two matrices' sums.
template <bool PRE, bool EMIT>
__global__ __launch_bounds__(256) void gemm_finish_kernel(const float* __restrict__ partials, int k_split, int M, int N,
                                                          int K, int mode, void* __restrict__ C, int ldc,
                                                          FinishNorm norm) {
  __shared__ float red[4];
  const int n = blockIdx.x * 256 + threadIdx.x, m = blockIdx.y;
  const bool on = n < N;
  float rstd = 1.f;
  if constexpr (PRE) {  // pre_parts <= 256: one value a thread, added in a fixed order
    const float v = threadIdx.x < norm.pre_parts ? norm.pre_ss[(size_t)m * norm.pre_parts + threadIdx.x] : 0.f;
    rstd = 1.0f / sqrtf(block_sum<256>(v, red) / (float)K + norm.eps);
  }
  const size_t plane = (size_t)M * N;
  const float* src = partials + (size_t)m * N + (on ? n : 0);
  float g = 0.f;
  for (int s = 0; s < k_split; ++s) g += src[s * plane];
  g *= rstd;
  const size_t o = (size_t)m * ldc + n;
  float sq = 0.f;
  if (on) {
    if (mode == G_STORE_BF16) ((bf16_t*)C)[o] = float_to_bf16(g);
    else if (mode == G_STORE_F32) ((float*)C)[o] = g;
    else if (mode == G_ACC_F32) {
      const float x = ((float*)C)[o] + g;
      ((float*)C)[o] = x;
      if constexpr (EMIT) {
        norm.raw[(size_t)m * norm.ld_raw + n] = float_to_bf16(x * norm.g[n]);
        sq = x * x;
      }
    } else {
      float u = 0.f;
      for (int s = 0; s < k_split; ++s) u += src[(k_split + s) * plane];
      ((bf16_t*)C)[o] = float_to_bf16(silu_f(g) * (u * rstd));
    }
  }
  if constexpr (EMIT) {
    const float total = block_sum<256>(sq, red);
    if (threadIdx.x == 0) norm.emit_ss[(size_t)m * gridDim.x + blockIdx.x] = total;
  }
}

// The first half of a product with K in slices: G_PARTIAL blocks leave float32 sums in workspace[which][slice][M][N].
static int launch_partials(const void* A, int lda, const void* W, const void* Wu, int M, int N, int K, int k_split,
                           float* workspace, hipStream_t stream) {
  if (K <= 0 || lda < K || k_split < 1 || !workspace || M > 65535) return APC_ERR_BAD_ARG;
  if (K % 8 || lda % 8 || !aligned16(A) || !aligned16(W) || (Wu && !aligned16(Wu))) return APC_ERR_UNSUPPORTED;
  const int n_mats = Wu ? 2 : 1;
  if (k_split * n_mats > 65535) return APC_ERR_BAD_ARG;
  if (!Wu) {  // many rows: the slices on the kernel that keeps the weights out of LDS, where it takes them
    const int e = launch_gemm_direct_slices((const bf16_t*)A, lda, (const bf16_t*)W, workspace, M, N, K, k_split, stream);
    if (e != APC_ERR_UNSUPPORTED) return e;
  }
  // up to 64 rows: tiles of 64 rows (half the loads of activations and half the MFMAs of a 128-row tile)
#define PARTIAL_LAUNCH(EVEN_, BM_, DEPTH_)                                                                          \
  hipLaunchKernelGGL((gemm_bf16_kernel<G_PARTIAL, EVEN_, BM_, false, DEPTH_>),                                      \
                     dim3(ceil_div(N, BN), ceil_div(M, BM_), k_split * n_mats), dim3(256), 0, stream, (const bf16_t*)A, \
                     lda, (const bf16_t*)W, (const bf16_t*)Wu, ceil_div(K, 32), workspace, N, M, N, K, k_split,      \
                     TiledPre{})
  if (M <= 64) {
    if (K % BK == 0) PARTIAL_LAUNCH(true, 64, 4);
    else PARTIAL_LAUNCH(false, 64, 4);
  } else if (M <= 128) {
    if (K % BK == 0) PARTIAL_LAUNCH(true, BM_ROWS, 4);
    else PARTIAL_LAUNCH(false, BM_ROWS, 4);
  } else {
    if (K % BK == 0) PARTIAL_LAUNCH(true, BM_ROWS, 2);
    else PARTIAL_LAUNCH(false, BM_ROWS, 2);
  }
#undef PARTIAL_LAUNCH
  APC_LAUNCH_CHECK();
  return 0;
}

// The plain finishing steps (no folded norm, no SwiGLU) four outputs a thread: the slices added in order, then stored
// or added into the residual.  N and ldc multiples of 4, 16-byte aligned rows.  (One output a thread takes 34 us for
// 2,048 x 4,096 outputs in two slices, this 13.)
__global__ __launch_bounds__(256) void gemm_finish4_kernel(const float* __restrict__ partials, int k_split, int M, int N,
                                                           int mode, void* __restrict__ C, int ldc) {
  const int n4 = N / 4;
  const size_t total = (size_t)M * n4, plane = (size_t)M * N;
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (size_t)gridDim.x * 256) {
    const int m = (int)(i / n4), n = (int)(i % n4) * 4;
    const float* src = partials + (size_t)m * N + n;
    floatx4 g = *reinterpret_cast<const floatx4*>(src);
    for (int s = 1; s < k_split; ++s) g += *reinterpret_cast<const floatx4*>(src + s * plane);
    const size_t o = (size_t)m * ldc + n;
    if (mode == G_STORE_BF16) {
      uint2 pk;
      pk.x = pack_bf16x2(g[0], g[1]);
      pk.y = pack_bf16x2(g[2], g[3]);
      *reinterpret_cast<uint2*>((bf16_t*)C + o) = pk;
    } else if (mode == G_STORE_F32) {
      *reinterpret_cast<floatx4*>((float*)C + o) = g;
    } else {
      floatx4* dst = reinterpret_cast<floatx4*>((float*)C + o);
      *dst = *dst + g;
    }
  }
}

static int launch_splitk(const void* A, int lda, const void* W, const void* Wu, void* C, int ldc, int M, int N, int K,
                         int mode, int k_split, float* workspace, int pre, int emit, FinishNorm norm,
                         hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (ldc < N) return APC_ERR_BAD_ARG;
  if (mode < 0 || mode > G_SWIGLU || (mode == G_SWIGLU) != (Wu != nullptr)) return APC_ERR_BAD_ARG;
  const int e = launch_partials(A, lda, W, Wu, M, N, K, k_split, workspace, stream);
  if (e) return e;
  if (!pre && !emit && mode != G_SWIGLU && N % 4 == 0 && ldc % 4 == 0 && aligned16(C) && (long)M * N >= (1L << 20)) {
    const long want = ((long)M * (N / 4) + 255) / 256;
    hipLaunchKernelGGL(gemm_finish4_kernel, dim3((unsigned)(want < 8192 ? want : 8192)), dim3(256), 0, stream, workspace,
                       k_split, M, N, mode, C, ldc);
    APC_LAUNCH_CHECK();
    return 0;
  }
  const dim3 grid(ceil_div(N, 256), M);
#define FINISH(PRE_, EMIT_)                                                                                     \
  hipLaunchKernelGGL((gemm_finish_kernel<PRE_, EMIT_>), grid, dim3(256), 0, stream, workspace, k_split, M, N, K, mode, \
                     C, ldc, norm)
  if (pre) FINISH(true, false);
  else if (emit) FINISH(false, true);
  else FINISH(false, false);
#undef FINISH
  APC_LAUNCH_CHECK();
  return 0;
}

// Finishing kernel of the product for q, k and v (K in slices): it adds the slices, scales them if the row came from
// a product that left the norm's row (PRE), rounds to bfloat16 as a stored result would be, rotates q and k by the
// row's position (whole heads, pairs (e, e + d/2)) and writes k and v into the paged cache: what the product's
// finishing kernel and the kernel for rotation and cache write would do one after the other.  A block has 256
// columns of one row, which are whole heads (256 is a multiple of d): a value meets its partner through LDS.
struct FinishRope {
  const float* cos_sin;    // [positions][2][d / 2]
  const int* positions;    // [M]
  const int* row_seg;      // [M]
  const int* block_table;  // [segments][max_blocks]
  int max_blocks;
  bf16_t* cache;           // pages of [2][Hk][P * d]: keys [kv head][slot][d], values [kv head][d][slot]
  int P, H, Hk, d;
};

template <bool PRE>
__global__ __launch_bounds__(256) void gemm_finish_qkv_rope_kernel(const float* __restrict__ partials, int k_split, int M,
                                                                   int N, int K, bf16_t* __restrict__ q_out, int ldq,
                                                                   FinishNorm norm, FinishRope rope) {
  __shared__ float red[4];
  __shared__ float vals[256];
  const int n = blockIdx.x * 256 + threadIdx.x, m = blockIdx.y;
  const bool on = n < N;
  float rstd = 1.f;
  if constexpr (PRE) {
    const float v = threadIdx.x < norm.pre_parts ? norm.pre_ss[(size_t)m * norm.pre_parts + threadIdx.x] : 0.f;
    rstd = 1.0f / sqrtf(block_sum<256>(v, red) / (float)K + norm.eps);
  }
  const size_t plane = (size_t)M * N;
  const float* src = partials + (size_t)m * N + (on ? n : 0);
  float g = 0.f;
  for (int s = 0; s < k_split; ++s) g += src[s * plane];
  const float x = bf16_to_float(float_to_bf16(g * rstd));
  vals[threadIdx.x] = x;
  __syncthreads();
  if (!on) return;
  const int d = rope.d, half = d / 2, head = n / d, e = n % d;
  const int pos = rope.positions[m];
  bf16_t* page = rope.cache + (size_t)rope.block_table[(size_t)rope.row_seg[m] * rope.max_blocks + pos / rope.P] *
                                  ((size_t)2 * rope.Hk * rope.P * d);
  const int slot = pos % rope.P;
  if (head < rope.H + rope.Hk) {
    const float* cs = rope.cos_sin + (size_t)pos * d;
    float y;
    if (e < half) {
      const float av = x, bv = vals[threadIdx.x + half], c = cs[e], sn = cs[half + e];
      y = av * c - bv * sn;
    } else {
      const float av = vals[threadIdx.x - half], bv = x, c = cs[e - half], sn = cs[e];
      y = av * sn + bv * c;
    }
    if (head < rope.H) q_out[(size_t)m * ldq + n] = float_to_bf16(y);
    else page[((size_t)(head - rope.H) * rope.P + slot) * d + e] = float_to_bf16(y);
  } else {
    page[(size_t)rope.Hk * rope.P * d + ((size_t)(head - rope.H - rope.Hk) * d + e) * rope.P + slot] = float_to_bf16(x);
  }
}

// Product for 17..128 rows: K is cut into `k_split` slices that different blocks multiply, so that matrices with
// few output columns still give the chip enough blocks; `workspace` holds (Wu ? 2 : 1) * k_split * M * N floats.
// mode as below, or 3 for SwiGLU (W = gate, Wu = up).
// How many slices of K the product of many rows (gemm_direct_bf16.hip) wants for this shape: 1, or 2 when narrow
// tiles would be needed to fill the chip otherwise.  The caller brings the workspace for apc_gemm_splitk_bf16.
APC_EXPORT int apc_gemm_direct_k_split(int M, int N, int K) { return gemm_direct_k_split(M, N, K); }

// residual += A . W^T for more than 1,024 rows, leaving the row for the RMS norm (weight g) that reads the residual
// next: raw [M][N] bfloat16 and ss [M][parts] (see gemm_direct.h).  apc_gemm_direct_emit_parts: the parts these sizes
// give, 0 if this entry point does not take them.
APC_EXPORT int apc_gemm_direct_emit_parts(const void* A, int lda, const void* residual, int ldc, int M, int N, int K) {
  return gemm_direct_emit_parts(A, lda, residual, ldc, M, N, K);
}
APC_EXPORT int apc_gemm_direct_emit_bf16(const void* A, int lda, const void* W, float* residual, int ldc, int M, int N,
                                         int K, const float* g, void* raw, int ldr, float* ss, int parts,
                                         float* workspace, hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (!aligned16(W)) return APC_ERR_UNSUPPORTED;
  return launch_gemm_direct_emit((const bf16_t*)A, lda, (const bf16_t*)W, residual, ldc, M, N, K, g, (bf16_t*)raw, ldr, ss,
                                 parts, workspace, stream);
}

APC_EXPORT int apc_gemm_splitk_bf16(const void* A, int lda, const void* W, const void* Wu, void* C, int ldc, int M,
                                    int N, int K, int mode, int k_split, float* workspace, hipStream_t stream) {
  return launch_splitk(A, lda, W, Wu, C, ldc, M, N, K, mode, k_split, workspace, 0, 0, FinishNorm{}, stream);
}

// C += A . W^T into the float32 residual, and for the RMS norm (weight g) that reads C next: raw[m, n] =
// bfloat16(C[m, n] * g[n]) and ss[m][ceil(N / 256)] = sums of C^2 per row and block of 256 columns.
APC_EXPORT int apc_gemm_splitk_emit_bf16(const void* A, int lda, const void* W, void* C, int ldc, int M, int N, int K,
                                         int k_split, float* workspace, const float* g, void* raw, int ld_raw,
                                         float* ss, hipStream_t stream) {
  if (!g || !raw || !ss || ld_raw < N) return APC_ERR_BAD_ARG;
  const FinishNorm norm{nullptr, 0, 0.f, g, (bf16_t*)raw, ld_raw, ss};
  return launch_splitk(A, lda, W, nullptr, C, ldc, M, N, K, G_ACC_F32, k_split, workspace, 0, 1, norm, stream);
}

// The storing products (mode 0, 1 or 3) on a row that apc_gemm_splitk_emit_bf16 left: A = raw [M, K],
// ss = [M][ss_parts] sums of x^2 (ss_parts <= 256); the sums are scaled by 1 / sqrt(sum(ss[m]) / K + eps).
APC_EXPORT int apc_gemm_splitk_pre_bf16(const void* A, int lda, const float* ss, int ss_parts, float eps,
                                        const void* W, const void* Wu, void* C, int ldc, int M, int N, int K, int mode,
                                        int k_split, float* workspace, hipStream_t stream) {
  if (!ss || ss_parts <= 0 || mode == G_ACC_F32) return APC_ERR_BAD_ARG;
  if (ss_parts > 256) return APC_ERR_UNSUPPORTED;
  const FinishNorm norm{ss, ss_parts, eps, nullptr, nullptr, 0, nullptr};
  return launch_splitk(A, lda, W, Wu, C, ldc, M, N, K, mode, k_split, workspace, 1, 0, norm, stream);
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

// The storing products on a row that a product into the residual left for the RMS norm, K in one piece:
// A = raw [M, K], ss = [M][ss_parts] sums of x^2; out = (A . W^T) / sqrt(sum(ss[m]) / K + eps).
// mode 0 store bfloat16, 1 store float32, 3 SwiGLU (W = gate, Wu = up; C is [M, N] with N = the width of each).
APC_EXPORT int apc_gemm_pre_bf16(const void* A, int lda, const float* ss, int ss_parts, float eps, const void* W,
                                 const void* Wu, void* C, int ldc, int M, int N, int K, int mode, hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (K <= 0 || lda < K || ldc < N || !ss || ss_parts <= 0) return APC_ERR_BAD_ARG;
  if ((mode == G_SWIGLU) != (Wu != nullptr)) return APC_ERR_BAD_ARG;
  if (K % 8 || lda % 8 || !aligned16(A) || !aligned16(W) || (Wu && !aligned16(Wu))) return APC_ERR_UNSUPPORTED;
  const bf16_t* a = (const bf16_t*)A;
  const bf16_t* w = (const bf16_t*)W;
  const TiledPre pre{ss, ss_parts, eps};
  switch (mode) {
    case G_STORE_BF16: return launch_gemm<G_STORE_BF16, true>(a, lda, w, nullptr, C, ldc, M, N, K, stream, pre);
    case G_STORE_F32: return launch_gemm<G_STORE_F32, true>(a, lda, w, nullptr, C, ldc, M, N, K, stream, pre);
    case G_SWIGLU: return launch_gemm<G_SWIGLU, true>(a, lda, w, (const bf16_t*)Wu, C, ldc, M, N, K, stream, pre);
    default: return APC_ERR_BAD_ARG;
  }
}

// q, k and v of 17 or more rows with K in slices, q and k rotated, k and v written into the paged cache (see
// gemm_finish_qkv_rope_kernel).  W: tiled layout of [(H + 2 Hk) d, K]; q_out [M, ldq] takes the rotated q heads in its
// first H d columns; 256 must be a multiple of d.  With ss: A is a row that a product into the residual left and the
// sums are scaled as in apc_gemm_splitk_pre_bf16.  workspace: k_split * M * (H + 2 Hk) d floats.
APC_EXPORT int apc_gemm_splitk_qkv_rope_bf16(const void* A, int lda, const float* ss, int ss_parts, float eps,
                                             const void* W, void* q_out, int ldq, int M, int K, int H, int Hk, int d,
                                             const float* cos_sin, const int* positions, const int* row_seg,
                                             const int* block_table, int max_blocks, void* cache, int page_tokens,
                                             int k_split, float* workspace, hipStream_t stream) {
  if (M <= 0) return 0;
  if (H <= 0 || Hk <= 0 || d <= 0 || ldq < H * d || !cos_sin || !positions || !row_seg || !block_table ||
      max_blocks <= 0 || !cache || page_tokens <= 0 || !q_out || (ss && ss_parts <= 0))
    return APC_ERR_BAD_ARG;
  if (d % 2 || 256 % d || (ss && ss_parts > 256)) return APC_ERR_UNSUPPORTED;
  const int N = (H + 2 * Hk) * d;
  const int e = launch_partials(A, lda, W, nullptr, M, N, K, k_split, workspace, stream);
  if (e) return e;
  const FinishNorm norm{ss, ss_parts, eps, nullptr, nullptr, 0, nullptr};
  const FinishRope rope{cos_sin, positions, row_seg, block_table, max_blocks, (bf16_t*)cache, page_tokens, H, Hk, d};
  const dim3 grid(ceil_div(N, 256), M);
  if (ss)
    hipLaunchKernelGGL((gemm_finish_qkv_rope_kernel<true>), grid, dim3(256), 0, stream, workspace, k_split, M, N, K,
                       (bf16_t*)q_out, ldq, norm, rope);
  else
    hipLaunchKernelGGL((gemm_finish_qkv_rope_kernel<false>), grid, dim3(256), 0, stream, workspace, k_split, M, N, K,
                       (bf16_t*)q_out, ldq, norm, rope);
  APC_LAUNCH_CHECK();
  return 0;
}
