// Matrix product for few rows (decode):  C[M,N] = A[M,K] . W[N,K]^T,  M <= 16, bfloat16 in, float32 sums.
//
// The step is bound by reading W once from HBM, so the kernel is a stream over W, which is stored in
// tiles of 16 rows x 32 columns laid out as the 64 lanes of a wave hold an operand of
// v_mfma_f32_16x16x32_bf16 (1 KiB a tile, tiles of a 16-row band in K order, bands in N order; rows and
// columns beyond N, K are zero):
//  * a block owns NB bands (16 NB output columns) and all of K; each of its WPB waves takes a contiguous
//    range of K and reads it in steps of 4 tiles per band: every load of W is 1 KiB of consecutive bytes and a
//    wave walks forward through one region of memory;
//  * the activations are the other operand (row m = lane % 16, 16 bytes of k per lane), loaded once per step
//    for all NB bands: D[n][m], so a lane ends with 4 consecutive n of one row m (SwiGLU: steps of 2 tiles);
//  * the loads of the next step are in flight while the current one is multiplied (two register sets that
//    swap roles; no branch around a load in the steady state);
//  * the waves' partial sums are added in wave order through LDS, then the epilogue runs: store (bfloat16 or
//    float32), add into a float32 residual, SwiGLU of a gate band and an up band, or rotation of q and k and the
//    write of k and v into the paged cache (SK_QKV_ROPE, see SkRope).
//  * the RMS norm between a product that adds into the residual x and the product that reads the normalised row
//    is folded into the two (EMIT and PRE): the first writes, beside x, the row bfloat16(x[m,n] * g[n]) (g: the
//    norm's weight) and, per band of 16 columns, the sum of x^2 of each row; the second multiplies with that row
//    as it is and scales its sums by 1 / sqrt(mean(x^2) + eps), which it gets by adding the bands' sums in band
//    order.  That is the product of the normalised row up to where the rounding to bfloat16 falls, without a
//    kernel of its own for the norm.
// The order of additions for an output depends on N and K, never on which other rows are in the batch: a
// decoded row is the same alone and in any batch of up to 16 rows.
// Reference counterpart: gemv_nt_bf16_{wide,wide_rows,splitk}_kernel, hip/src/kernels.cpp:3555-3700
// (no matrix cores, row-major weights); the product is matmul_nt, crates/allpaca-cpu/src/kernels.rs:97-128.
#include "mfma.h"

constexpr int SK_U = 4;              // tiles (32 k each) per band per step
constexpr int TILE_ELEMS = 16 * 32;  // elements of a tile

enum { SK_STORE_BF16 = 0, SK_STORE_F32 = 1, SK_ACC_F32 = 2, SK_SWIGLU = 3, SK_QKV_ROPE = 4 };

template <int MT, int NB, int U>
struct SkRegs {
  Frag w[NB][U];
  Frag a[MT][U];
};

// NB: weight bands per block (for SwiGLU: 2 = one gate band and the up band of the same outputs)
// What the folded norm needs.  ss: sums of x^2 per row and band, [16 rows][ld_ss] floats, ld_ss = n_ss rounded up
// to a multiple of 4.  PRE (this product reads a row that an EMIT product left): ss, n_ss, eps.  EMIT (SK_ACC_F32
// only): g = the next norm's weight [N], raw = where the row bfloat16(x * g) goes [M, ld_raw], ss = where this
// product's n_ss = ceil(N / 16) bands leave their sums.
constexpr int SS_LOADS = 8;  // 16-byte loads of sums a lane may have to make (PRE): n_ss <= 4 * 4 * WPB * SS_LOADS
struct SkNorm {
  float* ss;
  int n_ss;
  int ld_ss;
  float eps;
  const float* g;
  bf16_t* raw;
  int ld_raw;
};

// SK_QKV_ROPE: the product that gives q, k and v of a row also turns q and k by the row's position and writes k
// and v into the paged cache, so no kernel of its own does that.  W is [(H + 2 Hk) d, K], heads in the order q, k, v;
// the whole head is rotated (pairs (e, e + d/2)); d is a multiple of 32.  A block takes the bands j and j + d/32 of
// one head, so a lane of the finishing wave holds both elements of 4 pairs.  Rotated q goes to C; k to
// cache[page][0][kv head][slot][:], v to cache[page][1][kv head][:][slot], page = block_table[row_seg][pos / P],
// slot = pos % P.  The sums are rounded to bfloat16 before the rotation, as a product that stores them would.
struct SkRope {
  const float* cos_sin;    // [positions][2][d / 2]
  const int* positions;    // [M]
  const int* row_seg;      // [M]
  const int* block_table;  // [segments][max_blocks]
  int max_blocks;
  bf16_t* cache;
  int P, H, Hk, d;
};

// Tiles per band and step, and blocks that share a compute unit.  SwiGLU on a wide layer has more blocks than
// compute units and each block streams 2 bands: with steps of 2 tiles a block of 8 waves needs under 128 registers
// a lane, two blocks share a unit, and one block's first loads and final reduction hide behind the other's stream
// (8B shapes, 8 rows: 48.0 -> 44.4 us; the bytes in flight per unit stay the same).
constexpr int sk_step(int mode) { return mode == SK_SWIGLU ? 2 : SK_U; }
constexpr int sk_blocks(int mode, int wpb) { return (mode == SK_SWIGLU && wpb == 8) ? 2 : 1; }

template <int MT, int MODE, int NB, int WPB, bool PRE, bool EMIT>
__global__ __launch_bounds__(WPB * 64, sk_blocks(MODE, WPB)) void skinny_gemm_kernel(const bf16_t* __restrict__ A, int lda,
                                                               const bf16_t* __restrict__ W,
                                                               const bf16_t* __restrict__ W2, int chunks,
                                                               void* __restrict__ C, int ldc, int M, int N, int K,
                                                               SkNorm norm, int vec_c, SkRope rope) {
  static_assert(MODE != SK_QKV_ROPE || NB == 2, "the two bands of a block hold the two halves of the pairs");
  static_assert(!EMIT || MODE == SK_ACC_F32, "only a product that adds into the residual emits the next norm's row");
  static_assert(!PRE || MODE != SK_ACC_F32, "a product that reads a normalised row stores its result");
  constexpr int U = sk_step(MODE);
  static_assert(MT == 1, "written for one tile of rows (the finishing wave's early loads, the folded norm)");
  __shared__ float red[WPB * NB * MT * 256];
  __shared__ float row_ss[WPB * MT * 16];
  const int lane = threadIdx.x % WAVE, wave = threadIdx.x / WAVE;
  const int i = lane % 16, c = lane / 16;
  constexpr int OUT_BANDS = (MODE == SK_SWIGLU || MODE == SK_QKV_ROPE) ? 1 : NB;
  const int band0 = blockIdx.x * OUT_BANDS;
  const int bands = (N + 15) / 16;
  // SK_QKV_ROPE: head and first element of this lane's 4 pairs; position and segment of the finishing wave's row
  // are asked for before the stream starts, what depends on them behind its first loads
  int qkv_head = 0, qkv_e = 0, qkv_pos = 0, qkv_seg = 0;
  if constexpr (MODE == SK_QKV_ROPE) {
    const int hb = rope.d / 32;
    qkv_head = blockIdx.x / hb;
    qkv_e = (blockIdx.x % hb) * 16 + c * 4;
    if (wave == 0 && i < M) {
      qkv_pos = rope.positions[i];
      qkv_seg = rope.row_seg[i];
    }
  }

  // band pointers (bands beyond the matrix are clamped to the last: what they compute is never stored)
  const bf16_t* wb[NB];
#pragma unroll
  for (int b = 0; b < NB; ++b) {
    if (MODE == SK_SWIGLU) wb[b] = (b == 0 ? W : W2) + (size_t)band0 * chunks * TILE_ELEMS + lane * 8;
    else if (MODE == SK_QKV_ROPE)
      wb[b] = W + (size_t)(qkv_head * (rope.d / 16) + blockIdx.x % (rope.d / 32) + b * (rope.d / 32)) * chunks * TILE_ELEMS + lane * 8;
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
  auto load_step = [&](SkRegs<MT, NB, U>& r, int ch) {  // tiles ch .. ch+3, all inside K
#pragma unroll
    for (int u = 0; u < U; ++u) {
#pragma unroll
      for (int b = 0; b < NB; ++b) r.w[b][u] = load_frag_once(wb[b] + (size_t)(ch + u) * TILE_ELEMS);
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) r.a[mt][u] = load_frag(arow[mt] + (ch + u) * 32);
    }
  };
  auto compute = [&](const SkRegs<MT, NB, U>& r) {
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int b = 0; b < NB; ++b) acc[b][mt] = mfma16(r.w[b][u], r.a[mt][u], acc[b][mt]);
  };

  // this wave's range of tiles along K: [c_lo, c_hi); steps of 4 whole tiles, then single tiles
  const int full_chunks = K / 32;                       // tiles that lie wholly inside K (for the activations)
  const int per_wave = ((chunks + WPB - 1) / WPB + U - 1) / U * U;
  const int c_lo = min(wave * per_wave, chunks), c_hi = min(c_lo + per_wave, chunks);
  const int c_full_hi = min(c_hi, full_chunks);
  const int nsteps = c_full_hi > c_lo ? (c_full_hi - c_lo) / U : 0;
  // Steps are loaded two ahead (register sets r0, r1 take turns); no branch lies around a load in the steady loop,
  // so the waits for one set never wait for the other.
  SkRegs<MT, NB, U> r0, r1;
  if (nsteps > 0) load_step(r0, c_lo);
  if (nsteps > 1) load_step(r1, c_lo + U);
  // Behind the first loads of the stream, and needed only at the end: the sums of x^2 that the emitting product
  // left (PRE; the 4 * WPB (wave, c) pairs of the block take groups of 4 bands in turn, the pieces meet in LDS with
  // the partial sums of the product), and what the finishing wave of an output band adds to (residual, EMIT: g).
  float ss_piece = 0.f;
  if constexpr (PRE) {
    const int groups = norm.ld_ss / 4;
    floatx4 v[SS_LOADS];
#pragma unroll
    for (int j = 0; j < SS_LOADS; ++j) {
      const int q = wave * 4 + c + j * WPB * 4;
      v[j] = q < groups ? *reinterpret_cast<const floatx4*>(norm.ss + (size_t)i * norm.ld_ss + q * 4)
                        : floatx4{0.f, 0.f, 0.f, 0.f};
    }
#pragma unroll
    for (int j = 0; j < SS_LOADS; ++j) {
      const int q = wave * 4 + c + j * WPB * 4;
#pragma unroll
      for (int e = 0; e < 4; ++e)
        if (q * 4 + e < norm.n_ss) ss_piece += v[j][e];
    }
  }
  constexpr int ITEMS = OUT_BANDS * MT;  // (band, m-tile) pairs to finish: wave w finishes pair w
  const int fin_n = (band0 + wave) * 16 + c * 4;  // first of this lane's 4 columns if this wave finishes a band
  const bool fin_vec = vec_c && wave < ITEMS && i < M && fin_n + 3 < N;
  floatx4 c_old = floatx4{0.f, 0.f, 0.f, 0.f}, g_next = floatx4{0.f, 0.f, 0.f, 0.f};
  if (MODE == SK_ACC_F32 && fin_vec) {
    c_old = *reinterpret_cast<const floatx4*>((const float*)C + (size_t)i * ldc + fin_n);
    if constexpr (EMIT) g_next = *reinterpret_cast<const floatx4*>(norm.g + fin_n);
  }
  floatx4 cosv = floatx4{0.f, 0.f, 0.f, 0.f}, sinv = floatx4{0.f, 0.f, 0.f, 0.f};
  int qkv_page = 0;
  if constexpr (MODE == SK_QKV_ROPE) {
    if (wave == 0 && i < M) {
      if (qkv_head < rope.H + rope.Hk) {
        const float* cs = rope.cos_sin + (size_t)qkv_pos * rope.d;
        cosv = *reinterpret_cast<const floatx4*>(cs + qkv_e);
        sinv = *reinterpret_cast<const floatx4*>(cs + rope.d / 2 + qkv_e);
      }
      if (qkv_head >= rope.H) qkv_page = rope.block_table[(size_t)qkv_seg * rope.max_blocks + qkv_pos / rope.P];
    }
  }
  if (nsteps > 0) {
    int at = c_lo, done = 0;
    while (done + 3 < nsteps) {  // steps done, done+1 are loaded; done+2, done+3 exist
      compute(r0);
      load_step(r0, at + 2 * U);
      compute(r1);
      load_step(r1, at + 3 * U);
      at += 2 * U;
      done += 2;
    }
    const int rem = nsteps - done;  // 1..3
    compute(r0);
    if (rem == 3) load_step(r0, at + 2 * U);
    if (rem >= 2) compute(r1);
    if (rem == 3) compute(r0);
  }
  // what is left of the range: single tiles; the last one may be cut by K (K is a multiple of 8, so a lane's
  // 16 bytes of activations are inside or outside as a whole; W is zero beyond K)
  for (int ch = c_lo + nsteps * U; ch < c_hi; ++ch) {
    const bool in = ch * 32 + c * 8 < K;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      const Frag af = in ? load_frag(arow[mt] + ch * 32) : zero_frag();
#pragma unroll
      for (int b = 0; b < NB; ++b) acc[b][mt] = mfma16(load_frag_once(wb[b] + (size_t)ch * TILE_ELEMS), af, acc[b][mt]);
    }
  }

  if constexpr (PRE) {
    ss_piece += __shfl_xor(ss_piece, 16);
    ss_piece += __shfl_xor(ss_piece, 32);
    if (c == 0) row_ss[wave * 16 + i] = ss_piece;
  }
  // partial sums of the waves, added in wave order
  float* mine = red + wave * (NB * MT * 256);
#pragma unroll
  for (int b = 0; b < NB; ++b)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) *reinterpret_cast<floatx4*>(&mine[((b * MT + mt) * 64 + lane) * 4]) = acc[b][mt];
  __syncthreads();

  constexpr int NSUM = (MODE == SK_SWIGLU || MODE == SK_QKV_ROPE) ? 2 : 1;
  if (wave < ITEMS) {
    const int b = wave;
    floatx4 sum[NSUM];
#pragma unroll
    for (int s = 0; s < NSUM; ++s) {
      const int bb = NSUM == 2 ? s : b;
      sum[s] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int w = 0; w < WPB; ++w)
        sum[s] += *reinterpret_cast<const floatx4*>(&red[w * (NB * MT * 256) + (bb * MT * 64 + lane) * 4]);
    }
    const int m = i;  // D[n][m]: this lane holds row m = lane % 16 of the tile and columns fin_n .. fin_n + 3
    if constexpr (PRE) {
      float total = 0.f;
#pragma unroll
      for (int w = 0; w < WPB; ++w) total += row_ss[w * 16 + i];
      const float rstd = 1.0f / sqrtf(total / (float)K + norm.eps);
#pragma unroll
      for (int s2 = 0; s2 < NSUM; ++s2) sum[s2] *= rstd;
    }
    if constexpr (MODE == SK_QKV_ROPE) {
      if (m < M) {
        float lo[4], hi[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          lo[r] = bf16_to_float(float_to_bf16(sum[0][r]));
          hi[r] = bf16_to_float(float_to_bf16(sum[1][r]));
        }
        const int half = rope.d / 2, slot = qkv_pos % rope.P;
        bf16_t* page = rope.cache + (size_t)qkv_page * ((size_t)2 * rope.Hk * rope.P * rope.d);
        if (qkv_head < rope.H + rope.Hk) {
          float ya[4], yb[4];
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            const float av = lo[r], bv = hi[r], cc = cosv[r], sn = sinv[r];
            ya[r] = av * cc - bv * sn;
            yb[r] = av * sn + bv * cc;
          }
          bf16_t* dst = qkv_head < rope.H ? (bf16_t*)C + (size_t)m * ldc + (size_t)qkv_head * rope.d
                                          : page + ((size_t)(qkv_head - rope.H) * rope.P + slot) * rope.d;
          uint2 pa, pb;
          pa.x = pack_bf16x2(ya[0], ya[1]);
          pa.y = pack_bf16x2(ya[2], ya[3]);
          pb.x = pack_bf16x2(yb[0], yb[1]);
          pb.y = pack_bf16x2(yb[2], yb[3]);
          *reinterpret_cast<uint2*>(dst + qkv_e) = pa;
          *reinterpret_cast<uint2*>(dst + qkv_e + half) = pb;
        } else {
          bf16_t* col = page + (size_t)rope.Hk * rope.P * rope.d +
                        ((size_t)(qkv_head - rope.H - rope.Hk) * rope.d + qkv_e) * rope.P + slot;
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            col[(size_t)r * rope.P] = float_to_bf16(sum[0][r]);
            col[(size_t)(half + r) * rope.P] = float_to_bf16(sum[1][r]);
          }
        }
      }
      return;
    }
    float sq = 0.f;  // EMIT: x^2 over this lane's columns
    if (fin_vec) {
      if (MODE == SK_STORE_BF16 || MODE == SK_SWIGLU) {
        floatx4 y = sum[0];
        if (MODE == SK_SWIGLU) {
#pragma unroll
          for (int r = 0; r < 4; ++r) y[r] = silu_f(sum[0][r]) * sum[NSUM - 1][r];
        }
        uint2 packed;
        packed.x = pack_bf16x2(y[0], y[1]);
        packed.y = pack_bf16x2(y[2], y[3]);
        *reinterpret_cast<uint2*>((bf16_t*)C + (size_t)m * ldc + fin_n) = packed;
      } else if (MODE == SK_STORE_F32) {
        *reinterpret_cast<floatx4*>((float*)C + (size_t)m * ldc + fin_n) = sum[0];
      } else {
        const floatx4 x = c_old + sum[0];
        *reinterpret_cast<floatx4*>((float*)C + (size_t)m * ldc + fin_n) = x;
        if constexpr (EMIT) {
          uint2 packed;
          packed.x = pack_bf16x2(x[0] * g_next[0], x[1] * g_next[1]);
          packed.y = pack_bf16x2(x[2] * g_next[2], x[3] * g_next[3]);
          *reinterpret_cast<uint2*>(norm.raw + (size_t)m * norm.ld_raw + fin_n) = packed;
#pragma unroll
          for (int r = 0; r < 4; ++r) sq = fmaf(x[r], x[r], sq);
        }
      }
    } else if (m < M) {
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int n = fin_n + r;
        if (n >= N) continue;
        const size_t o = (size_t)m * ldc + n;
        if (MODE == SK_STORE_BF16) ((bf16_t*)C)[o] = float_to_bf16(sum[0][r]);
        else if (MODE == SK_STORE_F32) ((float*)C)[o] = sum[0][r];
        else if (MODE == SK_ACC_F32) {
          const float x = ((float*)C)[o] + sum[0][r];
          ((float*)C)[o] = x;
          if constexpr (EMIT) {
            norm.raw[(size_t)m * norm.ld_raw + n] = float_to_bf16(x * norm.g[n]);
            sq = fmaf(x, x, sq);
          }
        } else ((bf16_t*)C)[o] = float_to_bf16(silu_f(sum[0][r]) * sum[NSUM - 1][r]);
      }
    }
    if constexpr (EMIT) {  // the four lanes with pieces of row i add up (all lanes of the wave take part)
      sq += __shfl_xor(sq, 16);
      sq += __shfl_xor(sq, 32);
      if (c == 0 && band0 + b < bands) norm.ss[(size_t)i * norm.ld_ss + band0 + b] = sq;
    }
  }
}

// bands per block and waves per block: enough blocks and waves to keep HBM busy, never more waves than K
// can feed with whole steps or LDS can hold
static void pick_shape(int N, int K, bool swiglu, int* nb, int* wpb) {
  const int bands = ceil_div(N, 16), chunks = ceil_div(K, 32);
  *nb = (!swiglu && bands >= 2048) ? 2 : 1;
  const int blocks = ceil_div(bands, *nb);
  const int sets = swiglu ? 2 : *nb;
  int w = 4;
  while (w < 16 && (long)blocks * w < 4096 && chunks >= w * 2 * SK_U && w * 2 * sets <= 64) w *= 2;
  *wpb = w;
}

static bool aligned16(const void* p) { return ((uintptr_t)p & 15u) == 0; }

template <int MODE, bool PRE, bool EMIT>
static int launch_skinny(const bf16_t* A, int lda, const bf16_t* W, const bf16_t* W2, void* C, int ldc, int M, int N,
                         int K, SkNorm norm, hipStream_t stream, SkRope rope = SkRope{}) {
  int nb, wpb;
  pick_shape(MODE == SK_QKV_ROPE ? N / 2 : N, K, MODE == SK_SWIGLU || MODE == SK_QKV_ROPE, &nb, &wpb);
  const int chunks = ceil_div(K, 32), bands = ceil_div(N, 16);
  if ((MODE == SK_SWIGLU || MODE == SK_QKV_ROPE) && wpb > 8) wpb = 8;
  if (PRE && norm.ld_ss > 4 * 4 * wpb * SS_LOADS) return APC_ERR_UNSUPPORTED;
  // whole 16-byte (float32) or 8-byte (bfloat16) accesses to C and to the emitted row where everything is aligned
  const int elem = (MODE == SK_STORE_BF16 || MODE == SK_SWIGLU) ? 2 : 4;
  int vec_c = ldc % 4 == 0 && ((uintptr_t)C % (4 * elem)) == 0;
  if (EMIT) vec_c = vec_c && norm.ld_raw % 4 == 0 && ((uintptr_t)norm.raw % 8) == 0 && aligned16(norm.g);
#define SK_LAUNCH(NB_, WPB_)                                                                                  \
  hipLaunchKernelGGL((skinny_gemm_kernel<1, MODE, NB_, WPB_, PRE, EMIT>),                                     \
                     dim3(ceil_div(bands, MODE == SK_SWIGLU ? 1 : NB_)), dim3(WPB_ * WAVE), 0, stream, A, lda, W, \
                     W2, chunks, C, ldc, M, N, K, norm, vec_c, rope)
  if constexpr (MODE == SK_SWIGLU || MODE == SK_QKV_ROPE) {
    // two bands a wave: with 16 waves a block the two register sets of loads would not fit the 128 registers a
    // wave has then
    if (wpb == 4) SK_LAUNCH(2, 4);
    else SK_LAUNCH(2, 8);
  } else if (nb == 2) {
    if (wpb == 4) SK_LAUNCH(2, 4);
    else SK_LAUNCH(2, 8);
  } else {
    if (wpb == 4) SK_LAUNCH(1, 4);
    else if (wpb == 8) SK_LAUNCH(1, 8);
    else SK_LAUNCH(1, 16);
  }
#undef SK_LAUNCH
  APC_LAUNCH_CHECK();
  return 0;
}

static bool operands_ok(const void* A, int lda, const void* W, int M, int K) {
  return M <= 16 && K % 8 == 0 && lda % 8 == 0 && aligned16(A) && aligned16(W);
}

// W: tiled layout of an [N, K] matrix.  mode: 0 store bfloat16, 1 store float32, 2 add into float32
APC_EXPORT int apc_skinny_gemm_bf16(const void* A, int lda, const void* W, void* C, int ldc, int M, int N, int K,
                                    int mode, hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (K <= 0 || lda < K || ldc < N) return APC_ERR_BAD_ARG;
  if (!operands_ok(A, lda, W, M, K)) return APC_ERR_UNSUPPORTED;
  const bf16_t* a = (const bf16_t*)A;
  const bf16_t* w = (const bf16_t*)W;
  const SkNorm none{};
  switch (mode) {
    case SK_STORE_BF16: return launch_skinny<SK_STORE_BF16, false, false>(a, lda, w, nullptr, C, ldc, M, N, K, none, stream);
    case SK_STORE_F32: return launch_skinny<SK_STORE_F32, false, false>(a, lda, w, nullptr, C, ldc, M, N, K, none, stream);
    case SK_ACC_F32: return launch_skinny<SK_ACC_F32, false, false>(a, lda, w, nullptr, C, ldc, M, N, K, none, stream);
    default: return APC_ERR_BAD_ARG;
  }
}

// out[m, f] = silu(A[m] . Wg[f]) * (A[m] . Wu[f]);  Wg, Wu: tiled layouts of two [F, K] matrices
APC_EXPORT int apc_skinny_swiglu_bf16(const void* A, int lda, const void* Wg, const void* Wu, void* C, int ldc, int M,
                                      int F, int K, hipStream_t stream) {
  if (M <= 0 || F <= 0) return 0;
  if (K <= 0 || lda < K || ldc < F) return APC_ERR_BAD_ARG;
  if (!operands_ok(A, lda, Wg, M, K) || !aligned16(Wu)) return APC_ERR_UNSUPPORTED;
  return launch_skinny<SK_SWIGLU, false, false>((const bf16_t*)A, lda, (const bf16_t*)Wg, (const bf16_t*)Wu, C, ldc, M,
                                                F, K, SkNorm{}, stream);
}

// C += A . W^T into the float32 residual C [M, N], and for the RMS norm that reads C next: raw[m, n] =
// bfloat16(C[m, n] * g[n]) and ss[row][band] = the sum of C^2 over the band's 16 columns (ss: 16 rows of
// ceil(N / 16) floats rounded up to a multiple of 4).
APC_EXPORT int apc_skinny_gemm_emit_bf16(const void* A, int lda, const void* W, void* C, int ldc, int M, int N, int K,
                                         const float* g, void* raw, int ld_raw, float* ss, hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (K <= 0 || lda < K || ldc < N || ld_raw < N || !g || !raw || !ss) return APC_ERR_BAD_ARG;
  if (!operands_ok(A, lda, W, M, K)) return APC_ERR_UNSUPPORTED;
  const SkNorm norm{ss, ceil_div(N, 16), ceil_div(ceil_div(N, 16), 4) * 4, 0.f, g, (bf16_t*)raw, ld_raw};
  return launch_skinny<SK_ACC_F32, false, true>((const bf16_t*)A, lda, (const bf16_t*)W, nullptr, C, ldc, M, N, K, norm,
                                                stream);
}

// The two storing products on a row that apc_skinny_gemm_emit_bf16 left: A = raw [M, K], ss = [16][n_ss rounded up
// to 4] sums of x^2 (n_ss = ceil(K / 16)); out = (A . W^T) / sqrt(sum(ss) / K + eps).  mode: 0 store bfloat16, 1 store float32.
APC_EXPORT int apc_skinny_gemm_pre_bf16(const void* A, int lda, const float* ss, int n_ss, float eps, const void* W,
                                        void* C, int ldc, int M, int N, int K, int mode, hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (K <= 0 || lda < K || ldc < N || !ss || n_ss <= 0 || !aligned16(ss)) return APC_ERR_BAD_ARG;
  if (!operands_ok(A, lda, W, M, K)) return APC_ERR_UNSUPPORTED;
  const SkNorm norm{const_cast<float*>(ss), n_ss, ceil_div(n_ss, 4) * 4, eps, nullptr, nullptr, 0};
  const bf16_t* a = (const bf16_t*)A;
  const bf16_t* w = (const bf16_t*)W;
  switch (mode) {
    case SK_STORE_BF16: return launch_skinny<SK_STORE_BF16, true, false>(a, lda, w, nullptr, C, ldc, M, N, K, norm, stream);
    case SK_STORE_F32: return launch_skinny<SK_STORE_F32, true, false>(a, lda, w, nullptr, C, ldc, M, N, K, norm, stream);
    default: return APC_ERR_BAD_ARG;
  }
}

APC_EXPORT int apc_skinny_swiglu_pre_bf16(const void* A, int lda, const float* ss, int n_ss, float eps, const void* Wg,
                                          const void* Wu, void* C, int ldc, int M, int F, int K, hipStream_t stream) {
  if (M <= 0 || F <= 0) return 0;
  if (K <= 0 || lda < K || ldc < F || !ss || n_ss <= 0 || !aligned16(ss)) return APC_ERR_BAD_ARG;
  if (!operands_ok(A, lda, Wg, M, K) || !aligned16(Wu)) return APC_ERR_UNSUPPORTED;
  const SkNorm norm{const_cast<float*>(ss), n_ss, ceil_div(n_ss, 4) * 4, eps, nullptr, nullptr, 0};
  return launch_skinny<SK_SWIGLU, true, false>((const bf16_t*)A, lda, (const bf16_t*)Wg, (const bf16_t*)Wu, C, ldc, M, F,
                                               K, norm, stream);
}

// q, k, v of M <= 16 rows in one product, q and k rotated, k and v written into the paged cache (see SkRope).
// W: tiled layout of [(H + 2 Hk) d, K]; q_out [M, ldq] takes the rotated q heads in its first H d columns.  With ss:
// A is a row that apc_skinny_gemm_emit_bf16 left and the sums are scaled as in apc_skinny_gemm_pre_bf16.
APC_EXPORT int apc_skinny_qkv_rope_bf16(const void* A, int lda, const float* ss, int n_ss, float eps, const void* W,
                                        void* q_out, int ldq, int M, int K, int H, int Hk, int d,
                                        const float* cos_sin, const int* positions, const int* row_seg,
                                        const int* block_table, int max_blocks, void* cache, int page_tokens,
                                        hipStream_t stream) {
  if (M <= 0) return 0;
  if (H <= 0 || Hk <= 0 || d <= 0 || K <= 0 || lda < K || ldq < H * d || !cos_sin || !positions || !row_seg ||
      !block_table || max_blocks <= 0 || !cache || page_tokens <= 0 || (ss && n_ss <= 0))
    return APC_ERR_BAD_ARG;
  if (!operands_ok(A, lda, W, M, K) || d % 32 || ldq % 4 || ((uintptr_t)q_out & 7u) || !aligned16(cos_sin) ||
      ((uintptr_t)cache & 7u) || (ss && !aligned16(ss)))
    return APC_ERR_UNSUPPORTED;
  const SkRope rope{cos_sin, positions, row_seg, block_table, max_blocks, (bf16_t*)cache, page_tokens, H, Hk, d};
  const int N = (H + 2 * Hk) * d;
  if (ss) {
    const SkNorm norm{const_cast<float*>(ss), n_ss, ceil_div(n_ss, 4) * 4, eps, nullptr, nullptr, 0};
    return launch_skinny<SK_QKV_ROPE, true, false>((const bf16_t*)A, lda, (const bf16_t*)W, nullptr, q_out, ldq, M, N, K,
                                                   norm, stream, rope);
  }
  return launch_skinny<SK_QKV_ROPE, false, false>((const bf16_t*)A, lda, (const bf16_t*)W, nullptr, q_out, ldq, M, N, K,
                                                  SkNorm{}, stream, rope);
}
