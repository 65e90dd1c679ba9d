// Attention over the paged cache in bfloat16 on MFMA, float32 softmax.
//
//   prefill kernels  a block takes up to 64 consecutive rows of one request x one head (half of a step's tile of up to
//                    128 rows; tiles that are mostly whole, of heads of 128 or 64, go to attention_wide_bf16.hip, which
//                    takes a whole tile a block); keys in tiles of 64 through LDS; online softmax.  Head sizes up to 128: v_mfma_f32_32x32x16_bf16, a wave takes
//                    32 rows x half of each tile's keys (attn_prefill32_kernel; 98 us for 2,048 rows of 32 heads
//                    of 128, 707 TFLOP/s at 32,768 rows).  Larger heads: v_mfma_f32_16x16x32_bf16, 16 rows a wave
//                    (attn_prefill_kernel, which was 9 % slower at 128).
//   decode kernel    one row x one kv head (the H/Hk query heads of the group are the 16 rows of the MFMA
//                    tile, so keys and values are read once per group); each wave is a "part" that covers
//                    KW consecutive keys straight from global memory; parts are merged by a second kernel
//                    in key order.  (Merging in the same kernel, by the part that arrives last, was tried: the
//                    device-wide fences it needs write back and invalidate the XCDs' L2 caches and cost ten
//                    times what the second launch does.  Turning q and k and writing the row's own key and value
//                    into the cache inside this kernel, instead of in a kernel before it, was tried too: the
//                    dependent loads it puts in front of the stream of keys cost more than that kernel.)
// Cache pages: keys [kv_head][slot][d] (d contiguous), values [kv_head][d][slot] (slots contiguous): both
// MFMA operands want the summed axis contiguous per lane, d for the scores and positions for the values.
// Masking: a row at position p sees keys max(0, p - window + 1) .. p.  Scores are scaled on the finished
// dot product; softmax maxima, sums and exponentials are float32; P is rounded to bfloat16 for the
// value product (as every activation between two matrix products is in this path).
// Formula: crates/allpaca-cpu/src/kernels.rs:293-356.  Reference kernels (contiguous K/V, no matrix
// cores): attention_qtile_kernel hip/src/kernels.cpp:2203, attention_split_gqa_kernel 2276, merges 2479-2516.
#include "attention_wide.h"
#include "mfma.h"
#include <math.h>

constexpr int KT = 64;            // keys per tile in the prefill kernel
constexpr int QT = 64;            // rows per block in the prefill kernels of this file
constexpr int TILE_ROWS = ATTN_WIDE_ROWS;  // rows of a tile as the step packs them: two blocks here, one of the wide kernel
static_assert(TILE_ROWS == 2 * QT, "a tile is two halves");
constexpr int KPAD = 8;

// Both kernels compute the transposed products  S^T = K Q^T  and  O^T = V^T P^T : the MFMA result then holds, per
// lane, 4 consecutive keys (or value elements) of ONE query row (row = lane % 16), so a row's maximum and sum
// are 16 values in registers and two exchanges between the 4 lanes that share the row, P goes to LDS as 8-byte
// pieces in the row-major order the second product reads, and the output leaves as 8-byte pieces.
__device__ __forceinline__ float row4_max(float v) {  // over the 4 lanes that share lane % 16
  v = fmaxf(v, __shfl_xor(v, 16, WAVE));
  return fmaxf(v, __shfl_xor(v, 32, WAVE));
}
__device__ __forceinline__ float row4_sum(float v) {
  v += __shfl_xor(v, 16, WAVE);
  return v + __shfl_xor(v, 32, WAVE);
}
__device__ __forceinline__ uint32_t bf16_pair(float a, float b) { return pack_bf16x2(a, b); }
// A value operand holds 8 consecutive positions of one element.  Positions beyond the row's last key lie in slots
// that nobody has written since the page's last owner, positions in front of a window's first key may lie in the
// spare page that stands in for pages given back.  Their weight in P is 0, but 0 x NaN is NaN, so all but the
// positions lo <= p < hi of the 8 are cleared before the product sees them.
__device__ __forceinline__ void keep_positions(Frag& v, int lo, int hi) {
#pragma unroll
  for (int w = 0; w < 4; ++w) {
    const uint32_t a = (2 * w >= lo && 2 * w < hi) ? 0x0000ffffu : 0u;
    const uint32_t b = (2 * w + 1 >= lo && 2 * w + 1 < hi) ? 0xffff0000u : 0u;
    v.w[w] &= a | b;
  }
}
// 2^x for x <= 0 (or -inf): the bare instruction, without the range handling that large arguments need
__device__ __forceinline__ float exp2_neg(float x) { return __builtin_amdgcn_exp2f(x); }
constexpr float LOG2E = 1.4426950408889634f;
constexpr float RISE = 8.f;  // by how much (in powers of 2) a score may exceed the running reference in attn_prefill32_kernel

// ------------------------------------------------------------------------------------------ prefill
// A block of 4 waves works on up to 64 consecutive rows of one request and one head, 16 rows a wave.
template <int DP>  // head_dim rounded up to a multiple of 32
__global__ __launch_bounds__(256) void attn_prefill_kernel(
    const bf16_t* __restrict__ q, int ldq, int q_off, bf16_t* __restrict__ out, int ldo, int H, int Hk, int d,
    const bf16_t* __restrict__ cache, int P, const int* __restrict__ block_table, int max_blocks,
    const int* __restrict__ positions, const int* __restrict__ row_seg, const int* __restrict__ tile_row0,
    const int* __restrict__ tile_rows, int n_tiles, int window, float scale) {
  // elements of a row of K in LDS: a stride of 36 banks modulo 64 (as the rows of V and P have), so that the 16-byte
  // operand reads of 16 consecutive rows and of neighbouring pieces fall into different banks
  constexpr int KROW = DP + (DP % 128 == 0 ? 72 : DP % 128 == 64 ? 8 : DP % 128 == 32 ? 40 : 104);
  __shared__ __attribute__((aligned(16))) bf16_t Ks[KT * KROW];
  __shared__ __attribute__((aligned(16))) bf16_t Vs[DP * (KT + KPAD)];
  __shared__ __attribute__((aligned(16))) bf16_t Ps[4 * 16 * (KT + KPAD)];
  const int tid = threadIdx.x, lane = tid % WAVE, wave = tid / WAVE;
  const int li = lane % 16, lc = lane / 16;
  // Workgroups go to the 8 XCDs in turn (id % 8) and each XCD has an L2 of its own: all heads that read one kv
  // head run on one XCD, so its keys and values stay in that L2 for every query tile and head of the group.
  // Tiles are taken from the last (longest under the causal mask) to the first.
  int tile, h;
  {
    const int id = blockIdx.x, G = H / Hk;
    if (Hk % 8 == 0) {
      const int xcd = id % 8, slot = id / 8;
      const int lh = slot / n_tiles;                 // head among the H/8 heads of this XCD
      tile = n_tiles - 1 - slot % n_tiles;
      h = (xcd + 8 * (lh / G)) * G + lh % G;
    } else {
      tile = n_tiles - 1 - id % n_tiles;
      h = id / n_tiles;
    }
  }
  // the step's tiles have up to TILE_ROWS rows; this kernel takes them in halves of QT rows (n_tiles counts halves)
  const int nrows = min(tile_rows[tile / 2] - (tile % 2) * QT, QT);
  if (nrows <= 0) return;
  const int row0 = tile_row0[tile / 2] + (tile % 2) * QT;
  const int kvh = h / (H / Hk);
  const int pos0 = positions[row0];
  const int* bt = block_table + (size_t)row_seg[row0] * max_blocks;
  const int last = pos0 + nrows - 1;
  const int first = (window > 0 && pos0 - window + 1 > 0) ? pos0 - window + 1 : 0;
  const size_t page_stride = (size_t)2 * Hk * P * d;
  const int dchunks = d / 8;

  // K and V are zero where nothing is ever stored: the padding columns of K (a padded q column is zero as well,
  // but 0 * NaN is NaN) and the rows of V beyond d
  for (int idx = tid; idx < KT * KROW; idx += 256) Ks[idx] = 0;
  for (int idx = tid; idx < DP * (KT + KPAD); idx += 256) Vs[idx] = 0;

  // this wave's 16 query rows as an MFMA operand (row = lane % 16, 8 elements of d per lane and step)
  const int my_row = wave * 16 + li;
  Frag qf[DP / 32];
  {
    const bf16_t* qrow = q + (size_t)(row0 + min(my_row, nrows - 1)) * ldq + q_off + (size_t)h * d;
#pragma unroll
    for (int ks = 0; ks < DP / 32; ++ks) {
      const int e = ks * 32 + lc * 8;
      qf[ks] = (my_row < nrows && e < d) ? load_frag(qrow + e) : zero_frag();
    }
  }
  const int my_pos = pos0 + my_row;
  const int my_lo = (window > 0 && my_pos - window + 1 > 0) ? my_pos - window + 1 : 0;
  // the wave's rows see every key of a tile [t0, t0 + 64) when it lies inside [wave_lo, wave_hi]
  const int wave_hi = pos0 + wave * 16;  // smallest position of the wave's rows
  const int wave_top = wave_hi + 15;
  const int wave_lo = (window > 0 && wave_top - window + 1 > 0) ? wave_top - window + 1 : 0;
  const float sc2 = scale * LOG2E;  // exponentials are taken in base 2
  floatx4 o[DP / 16];               // O^T: element dt*16 + lc*4 + r of row li
#pragma unroll
  for (int dt = 0; dt < DP / 16; ++dt) o[dt] = floatx4{0.f, 0.f, 0.f, 0.f};
  float m_run = -INFINITY, l_run = 0.f;
  bf16_t* pw = Ps + wave * 16 * (KT + KPAD) + li * (KT + KPAD);  // this lane's row of P
  const bf16_t* krd = Ks + li * KROW + lc * 8;            // this lane's place in a K operand
  const bf16_t* vrd = Vs + li * (KT + KPAD) + lc * 8;            // ... and in a V operand

  // A tile of 64 keys and values goes global -> registers -> LDS; the loads of the next tile are issued before
  // the work on the current one and stored after it.  The tile is 8 groups of 8 consecutive keys, and a group lies
  // in one page (page sizes are multiples of 8): the 32 threads of group tid / 32 copy its keys (8 slots x d
  // elements, one run of consecutive bytes in the page) and its values (d rows of 8 slots, 16 bytes each).  So a
  // thread looks up one page per tile, one tile ahead, and its addresses are that page's base plus constants.
  // No load is conditional: a group beyond the last key is read from the last key's group (scores are masked, P is
  // 0 there), a piece beyond d from piece 0 (it is not stored).
  constexpr int PIECES = DP / 32;  // 16-byte pieces of K and of V per thread and tile
  const int grp = tid / 32, gl = tid % 32;
  const int last_group = (last / 8) * 8;
  int k_ldst[PIECES], v_ldst[PIECES];  // where this thread's pieces go in LDS (elements)
  bool on[PIECES];                     // piece j exists: gl + 32 j < d
#pragma unroll
  for (int j = 0; j < PIECES; ++j) {
    const int idx = gl + 32 * j;       // K: piece idx of the group's 8 x d elements; V: element idx of the head
    on[j] = idx < d;
    const int key = on[j] ? idx / dchunks : 0, ch = on[j] ? idx % dchunks : 0;
    k_ldst[j] = (grp * 8 + key) * KROW + ch * 8;
    v_ldst[j] = (on[j] ? idx : 0) * (KT + KPAD) + grp * 8;
  }
  const bf16_t* k_head = cache + (size_t)kvh * P * d;
  const bf16_t* v_head = cache + (size_t)(Hk + kvh) * P * d;
  int page_next = 0;  // page of this thread's group in the tile that is loaded next
  auto lookup_tile = [&](int t0) { page_next = bt[min(t0 + grp * 8, last_group) / P]; };
  Frag kreg[PIECES], vreg[PIECES];
  int v_lo = 0, v_hi = 8;
  auto load_tile = [&](int t0) {  // uses the page found by the last lookup_tile, which was for this t0
    const int tg = min(t0 + grp * 8, last_group), slot0 = tg % P;
    v_lo = first - tg;       // the group's positions v_lo <= p < v_hi can be seen by a row of the tile
    v_hi = last - tg + 1;
    const bf16_t* kp = k_head + (size_t)page_next * page_stride + (size_t)slot0 * d;
    const bf16_t* vp = v_head + (size_t)page_next * page_stride + slot0;
#pragma unroll
    for (int j = 0; j < PIECES; ++j) {
      const int idx = on[j] ? gl + 32 * j : 0;
      kreg[j] = load_frag(kp + idx * 8);
      vreg[j] = load_frag(vp + (size_t)idx * P);
    }
  };
  auto store_tile = [&]() {
#pragma unroll
    for (int j = 0; j < PIECES; ++j) {
      if (on[j]) {
        if (v_lo > 0 || v_hi < 8) keep_positions(vreg[j], v_lo, v_hi);
        *reinterpret_cast<Frag*>(Ks + k_ldst[j]) = kreg[j];
        *reinterpret_cast<Frag*>(Vs + v_ldst[j]) = vreg[j];
      }
    }
  };

  const int t_begin = (first / KT) * KT;
  lookup_tile(t_begin);
  load_tile(t_begin);
  lookup_tile(t_begin + KT);
  __syncthreads();  // the zero fills are done
  store_tile();
  __syncthreads();
  for (int t0 = t_begin; t0 <= last; t0 += KT) {
    load_tile(t0 + KT);          // beyond the last key: a harmless copy of the last group
    lookup_tile(t0 + 2 * KT);

    // S^T: lane holds keys t0 + nt*16 + lc*4 + r of row li
    floatx4 s[KT / 16];
#pragma unroll
    for (int nt = 0; nt < KT / 16; ++nt) {
      s[nt] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ks = 0; ks < DP / 32; ++ks) {
        const Frag kf = *reinterpret_cast<const Frag*>(krd + nt * 16 * KROW + ks * 32);
        s[nt] = mfma16(kf, qf[ks], s[nt]);
      }
    }
    // The scale (positive) goes into the exponent: max over the bare scores, one multiply for the maximum, and
    // 2^(s * sc2 - m) with one fused multiply-add a score.
    float mx = -INFINITY;
    if (t0 >= wave_lo && t0 + KT - 1 <= wave_hi) {  // every row of the wave sees the whole tile
#pragma unroll
      for (int nt = 0; nt < KT / 16; ++nt)
#pragma unroll
        for (int r = 0; r < 4; ++r) mx = fmaxf(mx, s[nt][r]);
    } else {
#pragma unroll
      for (int nt = 0; nt < KT / 16; ++nt)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int t = t0 + nt * 16 + lc * 4 + r;
          const float v = (t >= my_lo && t <= my_pos) ? s[nt][r] : -INFINITY;
          s[nt][r] = v;
          mx = fmaxf(mx, v);
        }
    }
    mx = row4_max(mx) * sc2;
    const float m_new = fmaxf(m_run, mx);
    const float m_safe = m_new == -INFINITY ? 0.f : m_new;
    const float alpha = exp2_neg(m_run - m_safe);
    float sum = 0.f;
#pragma unroll
    for (int nt = 0; nt < KT / 16; ++nt) {
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        s[nt][r] = exp2_neg(fmaf(s[nt][r], sc2, -m_safe));
        sum += s[nt][r];
      }
      // P, row-major [row][key], 4 consecutive keys at once (read back below by this wave only)
      uint2 pk;
      pk.x = bf16_pair(s[nt][0], s[nt][1]);
      pk.y = bf16_pair(s[nt][2], s[nt][3]);
      *reinterpret_cast<uint2*>(pw + nt * 16 + lc * 4) = pk;
    }
    l_run = l_run * alpha + row4_sum(sum);
    m_run = m_new;
    if (__builtin_amdgcn_ballot_w64(alpha != 1.0f)) {  // some row's maximum rose: O shrinks (else every factor is 1)
#pragma unroll
      for (int dt = 0; dt < DP / 16; ++dt)
#pragma unroll
        for (int r = 0; r < 4; ++r) o[dt][r] *= alpha;
    }
    wave_lds_order();
    // O^T += V^T P^T
#pragma unroll
    for (int kstep = 0; kstep < KT / 32; ++kstep) {
      const Frag pf = *reinterpret_cast<const Frag*>(pw + kstep * 32 + lc * 8);
#pragma unroll
      for (int dt = 0; dt < DP / 16; ++dt) {
        const Frag vf = *reinterpret_cast<const Frag*>(vrd + dt * 16 * (KT + KPAD) + kstep * 32);
        o[dt] = mfma16(vf, pf, o[dt]);
      }
    }
    __syncthreads();  // every wave is done with this tile's K and V
    store_tile();
    __syncthreads();
  }
  if (my_row < nrows) {
    const float inv = 1.0f / l_run;
    bf16_t* orow = out + (size_t)(row0 + my_row) * ldo + (size_t)h * d;
#pragma unroll
    for (int dt = 0; dt < DP / 16; ++dt) {
      const int e = dt * 16 + lc * 4;
      if (e < d) {
        uint2 pk;
        pk.x = bf16_pair(o[dt][0] * inv, o[dt][1] * inv);
        pk.y = bf16_pair(o[dt][2] * inv, o[dt][3] * inv);
        *reinterpret_cast<uint2*>(orow + e) = pk;
      }
    }
  }
}

// The same tile on v_mfma_f32_32x32x16_bf16, for head sizes up to 128.  The 4 waves are 2 halves of the rows x 2
// halves of each tile's 64 keys: a wave computes S^T [32 keys x 32 rows] and O^T [d x 32 rows] for its keys only,
// with a running maximum and sum of its own, and the two waves of a row half merge once at the end through LDS.
// Against the 16-row kernel above an operand read from LDS feeds twice the arithmetic (LDS bandwidth was what
// bound that kernel), P goes from the first product's result registers straight into the second product's operand
// (a lane's 8 results of a 16-key step are keys lh*4+0..3 and 8+lh*4+0..3, lh = lane / 32; V^T lies in LDS with the
// two middle groups of 4 keys of every 16 swapped, so that the matching 8 values of V are one 16-byte read), and a
// row's maximum and sum take one exchange between 2 lanes instead of two between 4.
// (Loading tiles two ahead, with a second set of registers for the pieces on their way, was tried: at a head size
// of 128 the kernel then needs all 256 registers, only one block fits a compute unit, and it runs at 490 instead
// of 720 TFLOP/s on 32,768 rows.)
template <int DP>  // head_dim rounded up to a multiple of 32, at most 128
__global__ __launch_bounds__(256) void attn_prefill32_kernel(
    const bf16_t* __restrict__ q, int ldq, int q_off, bf16_t* __restrict__ out, int ldo, int H, int Hk, int d,
    const bf16_t* __restrict__ cache, int P, const int* __restrict__ block_table, int max_blocks,
    const int* __restrict__ positions, const int* __restrict__ row_seg, const int* __restrict__ tile_row0,
    const int* __restrict__ tile_rows, int n_tiles, int window, float scale) {
  constexpr int KROW = DP + (DP % 128 == 0 ? 72 : DP % 128 == 64 ? 8 : DP % 128 == 32 ? 40 : 104);
  constexpr int VROW = KT + KPAD;
  constexpr int DT = DP / 32;  // 32-row tiles of O^T
  constexpr int LDS_ELEMS = KT * KROW + DP * VROW;
  static_assert((size_t)LDS_ELEMS * 2 >= (size_t)(2 * DT * 16 * 64 + 2 * 2 * 32) * 4, "the merge needs this much LDS");
  __shared__ __attribute__((aligned(16))) bf16_t smem[LDS_ELEMS];
  bf16_t* Ks = smem;
  bf16_t* Vs = smem + KT * KROW;
  const int tid = threadIdx.x, lane = tid % WAVE, wave = tid / WAVE;
  const int li = lane % 32, lh = lane / 32;
  const int rh = wave / 2, kh = wave % 2;  // half of the rows, half of each tile's keys
  int tile, h;
  {
    const int id = blockIdx.x, G = H / Hk;
    if (Hk % 8 == 0) {  // see attn_prefill_kernel
      const int xcd = id % 8, slot = id / 8;
      const int lhd = slot / n_tiles;
      tile = n_tiles - 1 - slot % n_tiles;
      h = (xcd + 8 * (lhd / G)) * G + lhd % G;
    } else {
      tile = n_tiles - 1 - id % n_tiles;
      h = id / n_tiles;
    }
  }
  // the step's tiles have up to TILE_ROWS rows; this kernel takes them in halves of QT rows (n_tiles counts halves)
  const int nrows = min(tile_rows[tile / 2] - (tile % 2) * QT, QT);
  if (nrows <= 0) return;
  const int row0 = tile_row0[tile / 2] + (tile % 2) * QT;
  const int kvh = h / (H / Hk);
  const int pos0 = positions[row0];
  const int* bt = block_table + (size_t)row_seg[row0] * max_blocks;
  const int last = pos0 + nrows - 1;
  const int first = (window > 0 && pos0 - window + 1 > 0) ? pos0 - window + 1 : 0;
  const size_t page_stride = (size_t)2 * Hk * P * d;
  const int dchunks = d / 8;

  for (int idx = tid; idx < LDS_ELEMS; idx += 256) smem[idx] = 0;  // padding columns of K, rows of V beyond d

  // this wave's 32 query rows as the second operand: row = lane % 32, 8 elements of d per lane and step of 16
  const int my_row = rh * 32 + li;
  Frag qf[DP / 16];
  {
    const bf16_t* qrow = q + (size_t)(row0 + min(my_row, nrows - 1)) * ldq + q_off + (size_t)h * d;
#pragma unroll
    for (int ks = 0; ks < DP / 16; ++ks) {
      const int e = ks * 16 + lh * 8;
      qf[ks] = (my_row < nrows && e < d) ? load_frag(qrow + e) : zero_frag();
    }
  }
  const int my_pos = pos0 + my_row;
  const int my_lo = (window > 0 && my_pos - window + 1 > 0) ? my_pos - window + 1 : 0;
  const int wave_hi = pos0 + rh * 32;  // smallest position of the wave's rows
  const int wave_top = wave_hi + 31;
  const int wave_lo = (window > 0 && wave_top - window + 1 > 0) ? wave_top - window + 1 : 0;
  const float sc2 = scale * LOG2E;
  floatx16 o[DT];  // O^T: element dt*32 + (r/4)*8 + lh*4 + r%4 of row li
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
#pragma unroll
    for (int r = 0; r < 16; ++r) o[dt][r] = 0.f;
  float m_run = -INFINITY, l_run = 0.f;
  const bf16_t* krd = Ks + (kh * 32 + li) * KROW + lh * 8;  // key kh*32 + li, d piece lh of a step of 16
  const bf16_t* vrd = Vs + li * VROW + kh * 32 + lh * 8;    // value row li of a group of 32, this half's columns

  // global -> registers -> LDS as in attn_prefill_kernel; the 8 keys of a group go into V^T's columns as two
  // pieces of 4 (the column order described above)
  constexpr int PIECES = DP / 32;
  const int grp = tid / 32, gl = tid % 32;
  const int last_group = (last / 8) * 8;
  int k_ldst[PIECES], v_ldst[PIECES];
  bool on[PIECES];
#pragma unroll
  for (int j = 0; j < PIECES; ++j) {
    const int idx = gl + 32 * j;
    on[j] = idx < d;
    const int key = on[j] ? idx / dchunks : 0, ch = on[j] ? idx % dchunks : 0;
    k_ldst[j] = (grp * 8 + key) * KROW + ch * 8;
    v_ldst[j] = (on[j] ? idx : 0) * VROW + (grp / 2) * 16 + (grp % 2) * 4;
  }
  const bf16_t* k_head = cache + (size_t)kvh * P * d;
  const bf16_t* v_head = cache + (size_t)(Hk + kvh) * P * d;
  int page_next = 0;
  auto lookup_tile = [&](int t0) { page_next = bt[min(t0 + grp * 8, last_group) / P]; };
  Frag kreg[PIECES], vreg[PIECES];
  int v_lo = 0, v_hi = 8;
  auto load_tile = [&](int t0) {
    const int tg = min(t0 + grp * 8, last_group), slot0 = tg % P;
    v_lo = first - tg;       // the group's positions v_lo <= p < v_hi can be seen by a row of the tile
    v_hi = last - tg + 1;
    const bf16_t* kp = k_head + (size_t)page_next * page_stride + (size_t)slot0 * d;
    const bf16_t* vp = v_head + (size_t)page_next * page_stride + slot0;
#pragma unroll
    for (int j = 0; j < PIECES; ++j) {
      const int idx = on[j] ? gl + 32 * j : 0;
      kreg[j] = load_frag(kp + idx * 8);
      vreg[j] = load_frag(vp + (size_t)idx * P);
    }
  };
  auto store_tile = [&]() {
#pragma unroll
    for (int j = 0; j < PIECES; ++j) {
      if (on[j]) {
        if (v_lo > 0 || v_hi < 8) keep_positions(vreg[j], v_lo, v_hi);
        *reinterpret_cast<Frag*>(Ks + k_ldst[j]) = kreg[j];
        uint2 a, b;
        a.x = vreg[j].w[0];
        a.y = vreg[j].w[1];
        b.x = vreg[j].w[2];
        b.y = vreg[j].w[3];
        *reinterpret_cast<uint2*>(Vs + v_ldst[j]) = a;
        *reinterpret_cast<uint2*>(Vs + v_ldst[j] + 8) = b;
      }
    }
  };

  const int t_begin = (first / KT) * KT;
  lookup_tile(t_begin);
  load_tile(t_begin);
  lookup_tile(t_begin + KT);
  __syncthreads();
  store_tile();
  __syncthreads();
  for (int t0 = t_begin; t0 <= last; t0 += KT) {
    load_tile(t0 + KT);
    lookup_tile(t0 + 2 * KT);

    // S^T: lane holds keys tk + (r/4)*8 + lh*4 + r%4 of row li
    const int tk = t0 + kh * 32;
    floatx16 s;
#pragma unroll
    for (int r = 0; r < 16; ++r) s[r] = 0.f;
#pragma unroll
    for (int ks = 0; ks < DP / 16; ++ks) {
      const Frag kf = *reinterpret_cast<const Frag*>(krd + ks * 16);
      s = mfma32(kf, qf[ks], s);
    }
    float mx = -INFINITY;
    if (tk >= wave_lo && tk + 31 <= wave_hi) {  // every row of the wave sees all 32 keys
#pragma unroll
      for (int r = 0; r < 16; ++r) mx = fmaxf(mx, s[r]);
    } else {
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int t = tk + (r / 4) * 8 + lh * 4 + (r % 4);
        const float v = (t >= my_lo && t <= my_pos) ? s[r] : -INFINITY;
        s[r] = v;
        mx = fmaxf(mx, v);
      }
    }
    mx = fmaxf(mx, __shfl_xor(mx, 32, WAVE)) * sc2;
    // The running maximum is only a reference point for the exponents: it moves up when a tile's maximum exceeds it
    // by more than RISE (then O and the sum shrink by 2^-(the move)), and stays otherwise, so that P reaches at most
    // 2^RISE and O is rescaled on a row's first tiles only.  The result O / sum does not depend on the reference.
    const float m_new = mx > m_run + RISE ? mx : m_run;
    const float m_safe = m_new == -INFINITY ? 0.f : m_new;
    const float alpha = exp2_neg(m_run - m_safe);
    float sum = 0.f;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      s[r] = exp2_neg(fmaf(s[r], sc2, -m_safe));
      sum += s[r];
    }
    l_run = l_run * alpha + (sum + __shfl_xor(sum, 32, WAVE));
    m_run = m_new;
    if (__builtin_amdgcn_ballot_w64(alpha != 1.0f)) {
#pragma unroll
      for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int r = 0; r < 16; ++r) o[dt][r] *= alpha;
    }
    // O^T += V^T P^T, two steps of 16 keys
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      Frag pf;
#pragma unroll
      for (int w = 0; w < 4; ++w) pf.w[w] = bf16_pair(s[8 * j + 2 * w], s[8 * j + 2 * w + 1]);
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) {
        const Frag vf = *reinterpret_cast<const Frag*>(vrd + dt * 32 * VROW + j * 16);
        o[dt] = mfma32(vf, pf, o[dt]);
      }
    }
    __syncthreads();
    store_tile();
    __syncthreads();
  }

  // the two key halves of a row half meet: wave kh = 1 leaves its maximum, sum and O^T in LDS, wave kh = 0 adds
  float* mo = reinterpret_cast<float*>(smem);            // [rh][dt][r][lane]
  float* ml = mo + 2 * DT * 16 * 64;                     // [rh][m, l][32 rows]
  if (kh == 1) {
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
      for (int r = 0; r < 16; ++r) mo[((rh * DT + dt) * 16 + r) * 64 + lane] = o[dt][r];
    if (lh == 0) {
      ml[(rh * 2 + 0) * 32 + li] = m_run;
      ml[(rh * 2 + 1) * 32 + li] = l_run;
    }
  }
  __syncthreads();
  if (kh == 0 && my_row < nrows) {
    const float m2 = ml[(rh * 2 + 0) * 32 + li], l2 = ml[(rh * 2 + 1) * 32 + li];
    const float m = fmaxf(m_run, m2);
    const float m_safe = m == -INFINITY ? 0.f : m;
    const float a1 = exp2_neg(m_run - m_safe), a2 = exp2_neg(m2 - m_safe);
    const float inv = 1.0f / (l_run * a1 + l2 * a2);
    bf16_t* orow = out + (size_t)(row0 + my_row) * ldo + (size_t)h * d;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int e = dt * 32 + g * 8 + lh * 4;
        if (e < d) {
          float y[4];
#pragma unroll
          for (int r = 0; r < 4; ++r)
            y[r] = (o[dt][g * 4 + r] * a1 + mo[((rh * DT + dt) * 16 + g * 4 + r) * 64 + lane] * a2) * inv;
          uint2 pk;
          pk.x = bf16_pair(y[0], y[1]);
          pk.y = bf16_pair(y[2], y[3]);
          *reinterpret_cast<uint2*>(orow + e) = pk;
        }
      }
    }
  }
}

// ------------------------------------------------------------------------------------------ decode
// parts[row][head][part][d + 2]: o[0..d), m, l
template <int DP>
struct KVRegs {
  Frag k[2][DP / 32];  // two tiles of 16 keys
  Frag v[DP / 16];     // 32 positions of 16 value elements per tile
};

// Three ways to the finished heads of a (row, kv head):
//  DEC_PARTS  a block is 4 parts (ranges of KW keys) of the pair; its waves leave their results in `parts` and
//             attn_merge_kernel, a second launch, finishes.  Kept for the sizes the other two do not take.
//  DEC_LAST   the same split over blocks, but a block first adds its 4 waves' results in LDS, leaves ONE partial
//             result, and the block of a pair that finishes last adds the blocks' results in block order and writes
//             the heads: no second launch (4.7-5.6 us a layer at 8B shapes, as much as the attention itself with one
//             row).  Who is last is found with one counter per pair (a block adds 1 when its result is in memory;
//             the one that reads blocks - 1 is last, and sets the counter back to 0 for the next launch).  The
//             partial results go through memory with stores and loads that are coherent across the chip's eight L2
//             caches one by one (sc1), not with a fence: a device-wide fence writes back and invalidates a whole L2
//             and cost ten times what the second launch did.
//  DEC_WHOLE  the block's 4 waves take all ranges of KW keys of the pair in turn (wave w the ranges w, w + 4, ..; with
//             KW == 0 the row's own keys in 4 equal ranges, one a wave, so that a short row beside a long one still
//             has work for every wave: 32 rows of 328 to 4,296 keys 69.1 -> 66.7 us, equal rows as before),
//             meet in LDS and the block writes the finished heads itself: no partial result goes through memory,
//             which pays once the pairs alone fill the chip (8B shapes, 2,048 keys a row: 32 rows 52.9 -> 49.1 us, 64
//             rows 98.2 -> 91.6 us, 128 rows 196 -> 181 us; with 16 rows 30.2 -> 34.7 us.  Blocks of 8 waves were 2 %
//             faster at one block a compute unit and 8-15 % slower at two).
// The order of additions for a row depends on its position, KW and the number of parts only.
constexpr int NW = 4;  // waves of a block of the decode kernel
constexpr int LAST_DIRECT = 8;  // up to so many blocks a pair the last one reads the others' results in one go
enum { DEC_PARTS = 0, DEC_WHOLE = 1, DEC_LAST = 2 };
// Keys a part of a row takes when the launch gives the number of parts and not their length (KW == 0): the row's
// `span` keys in n_parts equal ranges, in whole steps of 32 keys and no fewer than 64.  Rows of different lengths in
// one launch then all use every block of their pair, and a launch's shape (blocks a pair) does not change with the
// rows' lengths, which is what a recorded graph needs.
__device__ __forceinline__ int row_keys_per_part(int KW, int span, int n_parts) {
  if (KW > 0) return KW;
  return max(64, ((span + n_parts - 1) / n_parts + 31) / 32 * 32);
}
// Why the hand-over of DEC_LAST holds without a release/acquire pair.  Every access to a partial result, on either
// side, is a relaxed atomic of agent scope: on this chip such a store goes through to memory past the block's own L2
// (sc1) and such a load is served from memory, so neither a write-back of the writer's L2 nor an invalidation of the
// reader's is needed for these words.  What is left is order: a writer thread's stores are issued before its
// `s_waitcnt vmcnt(0)`, which returns when memory has acknowledged them; the block's barrier behind it puts all its
// threads' acknowledged stores before thread 0's add to the counter; the counter's adds are atomics on one word, so the
// block that reads `nz - 1` adds after every other block's add, hence after their stores were acknowledged; its
// loads are issued behind its own barrier, which stands behind that add.  The language's memory model does not
// promise this for relaxed atomics; the instructions they compile to here do (the kernel is built for gfx950 alone).
// The counters are zero before the first launch and every launch leaves them zero; a launch that dies half-way
// would leave a count behind, so whoever owns them zeroes them when an engine is set up (engine/native.py).
__device__ __forceinline__ void st_coh(float* p, float v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ float ld_coh(const float* p) {
  return __hip_atomic_load(const_cast<float*>(p), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
template <int DP, int MODE>
__global__ __launch_bounds__(NW * 64) void attn_decode_kernel(
    const bf16_t* __restrict__ q, int ldq, int q_off, int H, int Hk, int d, const bf16_t* __restrict__ cache, int P,
    const int* __restrict__ block_table, int max_blocks, const int* __restrict__ positions,
    const int* __restrict__ row_seg, const int* __restrict__ rows, int window, float scale, int KW, int n_parts,
    float* __restrict__ parts, bf16_t* __restrict__ out, int ldo, int* __restrict__ counters) {
  constexpr bool WHOLE = MODE == DEC_WHOLE, LAST = MODE == DEC_LAST;
  __shared__ __attribute__((aligned(16))) bf16_t Ps[NW * 16 * (32 + KPAD)];
  extern __shared__ __attribute__((aligned(16))) float meet[];  // WHOLE, LAST: [NW][heads of the tile][d + 2]
  const int lane = threadIdx.x % WAVE, wave = threadIdx.x / WAVE;
  const int li = lane % 16, lc = lane / 16;
  const int G = H / Hk, gtiles = (G + 15) / 16;
  const int ri = blockIdx.x;
  const int row = rows ? rows[ri] : ri;
  const int kvh = blockIdx.y / gtiles, gt = blockIdx.y % gtiles;
  const int part = blockIdx.z * NW + wave;
  const int pos = positions[row];
  const int first = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
  const int seen0 = (first / 32) * 32;  // the first position that is loaded
  // KW == 0: the row's own keys, from the first one it sees, in n_parts equal ranges (see row_keys_per_part); else
  // ranges of KW keys counted from position 0
  const int base = KW > 0 ? 0 : seen0;
  KW = row_keys_per_part(KW, pos + 1 - seen0, n_parts);
  // nothing to see for this part: the wave leaves (DEC_PARTS), or stays with an empty result (DEC_LAST: the block's
  // waves meet)
  const bool empty =
      !WHOLE && (part >= n_parts || max(base + part * KW, seen0) >= min(base + (part + 1) * KW, pos + 1));
  if (MODE == DEC_PARTS && empty) return;
  const int* bt = block_table + (size_t)row_seg[row] * max_blocks;
  const size_t page_stride = (size_t)2 * Hk * P * d;
  const size_t head_off = (size_t)kvh * P * d, v_off = (size_t)Hk * P * d;
  // the page ids of a range of keys, one per lane, fetched once per range: the loads of keys and values then
  // do not wait for a look-up in the block table (a range of KW keys spans at most 64 pages: checked by the host)
  int page0 = 0, my_page = 0;

  Frag qf[DP / 32];
  {
    const int g = gt * 16 + li;
    const bf16_t* qrow = q + (size_t)row * ldq + q_off + (size_t)(kvh * G + min(g, G - 1)) * d;
#pragma unroll
    for (int ks = 0; ks < DP / 32; ++ks) {
      const int e = ks * 32 + lc * 8;
      qf[ks] = (g < G && e < d) ? load_frag(qrow + e) : zero_frag();
    }
  }
  floatx4 o[DP / 16];
#pragma unroll
  for (int dt = 0; dt < DP / 16; ++dt) o[dt] = floatx4{0.f, 0.f, 0.f, 0.f};
  float m_run = -INFINITY, l_run = 0.f;
  bf16_t* pw = Ps + wave * 16 * (32 + KPAD);

  // Operands of 32 keys straight from the pages, with loads that the caches do not keep (a decoded row reads its keys
  // and values once).  Nothing is loaded conditionally: a key beyond the row's own
  // position is read from that position instead (its score is masked), an element beyond d from element 0 or
  // d - 1 (the query is zero there; such output columns are not stored), so the loads of the next 32 keys can be
  // in flight while these are used.
  auto load_kv = [&](KVRegs<DP>& r, int kb) {
#pragma unroll
    for (int nt = 0; nt < 2; ++nt) {
      const int t = min(kb + nt * 16 + li, pos);
      const int page = __shfl(my_page, t / P - page0, WAVE);
      const bf16_t* krow = cache + (size_t)page * page_stride + head_off + (size_t)(t % P) * d;
#pragma unroll
      for (int ks = 0; ks < DP / 32; ++ks) {
        const int e = ks * 32 + lc * 8;
        r.k[nt][ks] = load_frag_once(krow + (e < d ? e : 0));
      }
    }
    const int tv = min(kb + lc * 8, (pos / 8) * 8);
    const int vpage = __shfl(my_page, tv / P - page0, WAVE);
    const bf16_t* vbase = cache + (size_t)vpage * page_stride + v_off + head_off + (tv % P);
#pragma unroll
    for (int dt = 0; dt < DP / 16; ++dt) r.v[dt] = load_frag_once(vbase + (size_t)min(dt * 16 + li, d - 1) * P);
  };

  // lane holds keys kb + nt*16 + lc*4 + r (scores) and elements dt*16 + lc*4 + r (output) of head li of the group
  const float sc2 = scale * LOG2E;
  auto step = [&](KVRegs<DP>& r, int kb) {
    if (kb + 31 > pos || kb < first) {  // a step with positions the row does not see (see keep_positions)
      const int tv = min(kb + lc * 8, (pos / 8) * 8);  // as load_kv placed this lane's 8 positions
      const int lo = first - tv, hi = pos - tv + 1;
      if (lo > 0 || hi < 8) {
#pragma unroll
        for (int dt = 0; dt < DP / 16; ++dt) keep_positions(r.v[dt], lo, hi);
      }
    }
    floatx4 s[2];
#pragma unroll
    for (int nt = 0; nt < 2; ++nt) {
      s[nt] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ks = 0; ks < DP / 32; ++ks) s[nt] = mfma16(r.k[nt][ks], qf[ks], s[nt]);
    }
    float mx = -INFINITY;
#pragma unroll
    for (int nt = 0; nt < 2; ++nt)
#pragma unroll
      for (int rr = 0; rr < 4; ++rr) {
        const int t = kb + nt * 16 + lc * 4 + rr;
        const float v = (t >= first && t <= pos) ? s[nt][rr] * sc2 : -INFINITY;
        s[nt][rr] = v;
        mx = fmaxf(mx, v);
      }
    mx = row4_max(mx);
    const float m_new = fmaxf(m_run, mx);
    const float m_safe = m_new == -INFINITY ? 0.f : m_new;
    const float alpha = exp2_neg(m_run - m_safe);
    float sum = 0.f;
#pragma unroll
    for (int nt = 0; nt < 2; ++nt) {
#pragma unroll
      for (int rr = 0; rr < 4; ++rr) {
        const float pv = exp2_neg(s[nt][rr] - m_safe);
        s[nt][rr] = pv;
        sum += pv;
      }
      uint2 pk;
      pk.x = bf16_pair(s[nt][0], s[nt][1]);
      pk.y = bf16_pair(s[nt][2], s[nt][3]);
      *reinterpret_cast<uint2*>(&pw[li * (32 + KPAD) + nt * 16 + lc * 4]) = pk;
    }
    l_run = l_run * alpha + row4_sum(sum);
    m_run = m_new;
#pragma unroll
    for (int dt = 0; dt < DP / 16; ++dt)
#pragma unroll
      for (int rr = 0; rr < 4; ++rr) o[dt][rr] *= alpha;
    wave_lds_order();
    const Frag pf = *reinterpret_cast<const Frag*>(&pw[li * (32 + KPAD) + lc * 8]);
#pragma unroll
    for (int dt = 0; dt < DP / 16; ++dt) o[dt] = mfma16(r.v[dt], pf, o[dt]);
    wave_lds_order();
  };

  auto run_range = [&](int k_lo, int k_hi) {
    page0 = k_lo / P;
    my_page = bt[min(page0 + lane, pos / P)];
    const int nsteps = (k_hi - k_lo + 31) / 32;
    KVRegs<DP> ra, rb;
    load_kv(ra, k_lo);
    int done = 0, kb = k_lo;
    while (done + 2 < nsteps) {
      load_kv(rb, kb + 32);
      step(ra, kb);
      load_kv(ra, kb + 64);
      step(rb, kb + 32);
      kb += 64;
      done += 2;
    }
    if (done + 1 < nsteps) {
      load_kv(rb, kb + 32);
      step(ra, kb);
      step(rb, kb + 32);
    } else {
      step(ra, kb);
    }
  };
  // a range in pieces of no more keys than a wave keeps page ids for (one piece, but for rows far longer than the
  // launch's parts were counted for, and for the one range a wave of DEC_WHOLE has of a long row)
  const int piece = max(32, (62 * P) / 32 * 32);
  if constexpr (WHOLE) {
    // ranges wave, wave + NW, ..: with the row's own ranges (the launch gave no length) that is one range a wave
    for (int r = wave; base + r * KW <= pos; r += NW) {
      const int k_lo = max(base + r * KW, seen0), k_hi = min(base + (r + 1) * KW, pos + 1);
      for (int k = k_lo; k < k_hi; k += piece) run_range(k, min(k + piece, k_hi));
    }
  } else if (!empty) {
    const int k_lo = max(base + part * KW, seen0), k_hi = min(base + (part + 1) * KW, pos + 1);
    for (int k = k_lo; k < k_hi; k += piece) run_range(k, min(k + piece, k_hi));
  }

  // this wave's result for the heads of the group (maxima are in base-2 units, as the merge expects)
  const int g = gt * 16 + li;
  const int tile_heads = min(G - gt * 16, 16);
  if (g < G) {
    float* dst = (WHOLE || LAST) ? meet + ((size_t)wave * tile_heads + li) * (d + 2)
                                 : parts + (((size_t)ri * H + (kvh * G + g)) * n_parts + part) * (d + 2);
#pragma unroll
    for (int dt = 0; dt < DP / 16; ++dt) {
      const int e = dt * 16 + lc * 4;
      if (e < d) {
#pragma unroll
        for (int rr = 0; rr < 4; ++rr) dst[e + rr] = o[dt][rr];
      }
    }
    if (lc == 0) { dst[d] = m_run; dst[d + 1] = l_run; }
  }
  if constexpr (WHOLE) {
    // the waves' results of a head, in wave order (a wave that saw no key left a maximum of -inf and zeros)
    __syncthreads();
    const int stride = d + 2;
    for (int idx = threadIdx.x; idx < tile_heads * d; idx += NW * 64) {
      const int hg = idx / d, e = idx % d;
      const float* src = meet + (size_t)hg * stride;
      float m = -INFINITY;
#pragma unroll
      for (int w = 0; w < NW; ++w) m = fmaxf(m, src[(size_t)w * tile_heads * stride + d]);
      float l = 0.f, acc = 0.f;
#pragma unroll
      for (int w = 0; w < NW; ++w) {
        const float* ws = src + (size_t)w * tile_heads * stride;
        const float pm = ws[d];
        const float wgt = pm == -INFINITY ? 0.f : exp2_neg(pm - m);
        l += ws[d + 1] * wgt;
        acc = fmaf(ws[e], wgt, acc);
      }
      out[(size_t)row * ldo + (size_t)(kvh * G + gt * 16 + hg) * d + e] = float_to_bf16(acc / l);
    }
  }
  if constexpr (LAST) {
    // The block's partial result for every head of the tile: the waves' results added in wave order, not divided by
    // the sum; to parts[row][head][block][d + 2] = o, maximum, sum.
    __syncthreads();
    const int stride = d + 2, nz = gridDim.z, z = blockIdx.z;
    for (int idx = threadIdx.x; idx < tile_heads * d; idx += NW * 64) {
      const int hg = idx / d, e = idx % d;
      const float* src = meet + (size_t)hg * stride;
      float m = -INFINITY;
#pragma unroll
      for (int w = 0; w < NW; ++w) m = fmaxf(m, src[(size_t)w * tile_heads * stride + d]);
      float l = 0.f, acc = 0.f;
#pragma unroll
      for (int w = 0; w < NW; ++w) {
        const float* ws = src + (size_t)w * tile_heads * stride;
        const float pm = ws[d];
        const float wgt = pm == -INFINITY ? 0.f : exp2_neg(pm - m);
        l += ws[d + 1] * wgt;
        acc = fmaf(ws[e], wgt, acc);
      }
      float* dst = parts + (((size_t)ri * H + (kvh * G + gt * 16 + hg)) * nz + z) * stride;
      st_coh(dst + e, acc);
      if (e == 0) {
        st_coh(dst + d, m);
        st_coh(dst + d + 1, l);
      }
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // this thread's stores have reached memory
    __syncthreads();
    __shared__ int is_last;
    int* counter = counters + (size_t)ri * gridDim.y + blockIdx.y;
    if (threadIdx.x == 0) {
      const int before = __hip_atomic_fetch_add(counter, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      is_last = before == nz - 1;
      if (is_last) __hip_atomic_store(counter, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);  // for the next launch
    }
    __syncthreads();
    if (!is_last) return;
    // the last block of the pair: the blocks' results of every head, in block order (only blocks with a visible key)
    const int p_lo = (seen0 - base) / KW, p_hi = min((pos - base) / KW, n_parts - 1);
    const int z_lo = p_lo / NW, nzv = p_hi / NW - z_lo + 1;
    if (nzv <= LAST_DIRECT) {
      // few blocks: a thread asks for the maxima, sums and its element of all of them at once (one trip to memory
      // where the general way below makes two with a barrier between); the same additions in the same order
      for (int idx = threadIdx.x; idx < tile_heads * d; idx += NW * 64) {
        const int hg = idx / d, e = idx % d;
        const float* src = parts + (((size_t)ri * H + (kvh * G + gt * 16 + hg)) * nz + z_lo) * stride;
        float pm[LAST_DIRECT], pl[LAST_DIRECT], po[LAST_DIRECT];
#pragma unroll
        for (int zz = 0; zz < LAST_DIRECT; ++zz) {
          const float* sz = src + (size_t)min(zz, nzv - 1) * stride;
          pm[zz] = ld_coh(sz + d);
          pl[zz] = ld_coh(sz + d + 1);
          po[zz] = ld_coh(sz + e);
        }
        float m = -INFINITY;
#pragma unroll
        for (int zz = 0; zz < LAST_DIRECT; ++zz)
          if (zz < nzv) m = fmaxf(m, pm[zz]);
        float l = 0.f, acc = 0.f;
#pragma unroll
        for (int zz = 0; zz < LAST_DIRECT; ++zz)
          if (zz < nzv) {
            const float wgt = pm[zz] == -INFINITY ? 0.f : exp2_neg(pm[zz] - m);
            l += pl[zz] * wgt;
            acc = fmaf(po[zz], wgt, acc);
          }
        out[(size_t)row * ldo + (size_t)(kvh * G + gt * 16 + hg) * d + e] = float_to_bf16(acc / l);
      }
      return;
    }
    float* ml = meet;  // [heads of the tile][nzv][2]: maximum, sum (the waves' results are not needed any more)
    for (int idx = threadIdx.x; idx < tile_heads * nzv; idx += NW * 64) {
      const int hg = idx / nzv, zz = idx % nzv;
      const float* src = parts + (((size_t)ri * H + (kvh * G + gt * 16 + hg)) * nz + z_lo + zz) * stride;
      ml[idx * 2] = ld_coh(src + d);
      ml[idx * 2 + 1] = ld_coh(src + d + 1);
    }
    __syncthreads();
    for (int idx = threadIdx.x; idx < tile_heads * d; idx += NW * 64) {
      const int hg = idx / d, e = idx % d;
      const float* src = parts + (((size_t)ri * H + (kvh * G + gt * 16 + hg)) * nz + z_lo) * stride + e;
      const float* mlh = ml + (size_t)hg * nzv * 2;
      float m = -INFINITY;
      for (int zz = 0; zz < nzv; ++zz) m = fmaxf(m, mlh[zz * 2]);
      float l = 0.f, acc = 0.f;
      for (int zz = 0; zz < nzv; ++zz) {
        const float pm = mlh[zz * 2];
        const float wgt = pm == -INFINITY ? 0.f : exp2_neg(pm - m);
        l += mlh[zz * 2 + 1] * wgt;
        acc = fmaf(ld_coh(src + (size_t)zz * stride), wgt, acc);
      }
      out[(size_t)row * ldo + (size_t)(kvh * G + gt * 16 + hg) * d + e] = float_to_bf16(acc / l);
    }
  }
}

// Merge of the parts of one (row, head).  Lane p of every wave reads part p's maximum and sum (64 parts a pass), a
// thread owns elements of the head and asks for its elements of the first MERGE_CHUNK parts at the same time: with up
// to that many parts the kernel makes one trip to memory, and nothing goes through LDS.  The parts' weights
// 2^(maximum - overall maximum) are computed once per lane and handed round the wave; sums over parts are taken in a
// fixed order (over the lanes of a wave as `wave_sum` adds them, over a thread's elements in part order).
constexpr int MERGE_NT = 128;
constexpr int MERGE_CHUNK = 16;
__global__ __launch_bounds__(MERGE_NT) void attn_merge_kernel(const float* __restrict__ parts, int n_parts, int KW,
                                                              int H, int d, const int* __restrict__ positions,
                                                              const int* __restrict__ rows, int window,
                                                              bf16_t* __restrict__ out, int ldo) {
  const int ri = blockIdx.x, h = blockIdx.y, tid = threadIdx.x, lane = tid % WAVE;
  const int row = rows ? rows[ri] : ri;
  const int pos = positions[row];
  const int first = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
  const int seen0 = (first / 32) * 32, part_base = KW > 0 ? 0 : seen0;  // as attn_decode_kernel counts the parts
  KW = row_keys_per_part(KW, pos + 1 - seen0, n_parts);
  const int p_lo = (seen0 - part_base) / KW, p_hi = min((pos - part_base) / KW, n_parts - 1);  // parts with a visible key
  const int np = p_hi - p_lo + 1;
  const size_t stride = (size_t)d + 2;
  const float* base = parts + (((size_t)ri * H + h) * n_parts + p_lo) * stride;
  bf16_t* orow = out + (size_t)row * ldo + (size_t)h * d;
  const int e0 = tid, e1 = tid + MERGE_NT;  // d <= 256: at most two elements a thread
  const bool on0 = e0 < d, on1 = e1 < d;
  float o0[MERGE_CHUNK], o1[MERGE_CHUNK];
  auto load_outputs = [&](int q0) {  // this thread's elements of parts q0 .. q0 + MERGE_CHUNK - 1 (the last part again beyond)
#pragma unroll
    for (int p = 0; p < MERGE_CHUNK; ++p) {
      const float* src = base + (size_t)min(q0 + p, np - 1) * stride;
      o0[p] = src[on0 ? e0 : 0];
      o1[p] = on1 ? src[e1] : 0.f;
    }
  };
  auto load_max = [&](int c0) { return c0 + lane < np ? base[(size_t)(c0 + lane) * stride + d] : -INFINITY; };
  auto load_sum = [&](int c0) { return c0 + lane < np ? base[(size_t)(c0 + lane) * stride + d + 1] : 0.f; };
  const float pm_first = load_max(0), pl_first = load_sum(0);
  load_outputs(0);
  float m = wave_max(pm_first);
  for (int c0 = WAVE; c0 < np; c0 += WAVE) m = fmaxf(m, wave_max(load_max(c0)));
  float l = 0.f, a0 = 0.f, a1 = 0.f;
  for (int c0 = 0; c0 < np; c0 += WAVE) {
    const float pm = c0 == 0 ? pm_first : load_max(c0), pl = c0 == 0 ? pl_first : load_sum(c0);
    const float w = pm == -INFINITY ? 0.f : exp2_neg(pm - m);
    l += wave_sum(pl * w);
    for (int q0 = c0; q0 < min(np, c0 + WAVE); q0 += MERGE_CHUNK) {
      if (q0 > 0) load_outputs(q0);
#pragma unroll
      for (int p = 0; p < MERGE_CHUNK; ++p) {
        if (q0 + p < np) {
          const float wp = __shfl(w, q0 + p - c0, WAVE);
          a0 = fmaf(o0[p], wp, a0);
          a1 = fmaf(o1[p], wp, a1);
        }
      }
    }
  }
  const float inv = 1.0f / l;
  if (on0) orow[e0] = float_to_bf16(a0 * inv);
  if (on1) orow[e1] = float_to_bf16(a1 * inv);
}

// ------------------------------------------------------------------------------------------ entry points
static bool aligned16(const void* p) { return ((uintptr_t)p & 15u) == 0; }

static int check_common(const void* q, int ldq, int q_off, const void* cache, int H, int Hk, int d, int P) {
  if (H <= 0 || Hk <= 0 || H % Hk || d <= 0 || P <= 0) return APC_ERR_BAD_ARG;
  if (d % 16 || d > 256 || P % 8 || ldq % 8 || q_off % 8 || !aligned16(q) || !aligned16(cache)) return APC_ERR_UNSUPPORTED;
  return 0;
}

APC_EXPORT int apc_attention_prefill_bf16(const void* q, int ldq, int q_off, void* out, int ldo, int H, int Hk, int d,
                                          const void* cache, int page_tokens, const int* block_table, int max_blocks,
                                          const int* positions, const int* row_seg, const int* tile_row0,
                                          const int* tile_rows, int n_tiles, int n_rows, int window, float scale,
                                          int n_splits, int part_rows, float* parts, hipStream_t stream) {
  if (n_tiles <= 0) return 0;
  int e = check_common(q, ldq, q_off, cache, H, Hk, d, page_tokens);
  if (e) return e;
  if (ldo % 4 || ((uintptr_t)out & 7u)) return APC_ERR_UNSUPPORTED;  // outputs are stored 8 bytes at a time
  if (max_blocks <= 0 || window < 0 || (long)n_tiles * H > 0x7fffffffL) return APC_ERR_BAD_ARG;
  if (!(scale > 0.f)) return APC_ERR_UNSUPPORTED;  // the kernel takes the maximum before it scales
  // n_rows: the rows of all tiles together.  Tiles of 64 rows and more on average go to the kernel that takes 128 rows a
  // block; with many short ones (many small requests) half of its waves would have no rows (measured at 8B shapes: 17-32
  // rows a tile 2-4 % slower than the 64-row kernel, 16 rows over 128 keys 36 %; 33-128 rows a tile 1.2-1.35 times as fast).
  if (attn_wide_takes(d, page_tokens) && (long)n_rows * 2 >= (long)n_tiles * TILE_ROWS)
    return launch_attn_prefill_wide((const bf16_t*)q, ldq, q_off, (bf16_t*)out, ldo, H, Hk, (const bf16_t*)cache,
                                    page_tokens, block_table, max_blocks, positions, row_seg, tile_row0, tile_rows,
                                    n_tiles, window, scale, n_splits < 1 ? 1 : n_splits, part_rows, parts, d, stream);
  n_tiles *= 2;  // halves
  if ((long)n_tiles * H > 0x7fffffffL) return APC_ERR_BAD_ARG;
  dim3 grid(n_tiles * H), block(256);
#define PF_LAUNCH(DP_)                                                                                             \
  hipLaunchKernelGGL((attn_prefill_kernel<DP_>), grid, block, 0, stream, (const bf16_t*)q, ldq, q_off, (bf16_t*)out, \
                     ldo, H, Hk, d, (const bf16_t*)cache, page_tokens, block_table, max_blocks, positions, row_seg,  \
                     tile_row0, tile_rows, n_tiles, window, scale)
#define PF32_LAUNCH(DP_)                                                                                             \
  hipLaunchKernelGGL((attn_prefill32_kernel<DP_>), grid, block, 0, stream, (const bf16_t*)q, ldq, q_off, (bf16_t*)out, \
                     ldo, H, Hk, d, (const bf16_t*)cache, page_tokens, block_table, max_blocks, positions, row_seg,    \
                     tile_row0, tile_rows, n_tiles, window, scale)
  if (d <= 32) PF32_LAUNCH(32);
  else if (d <= 64) PF32_LAUNCH(64);
  else if (d <= 96) PF32_LAUNCH(96);
  else if (d <= 128) PF32_LAUNCH(128);
  else if (d <= 192) PF_LAUNCH(192);
  else PF_LAUNCH(256);
#undef PF_LAUNCH
#undef PF32_LAUNCH
  APC_LAUNCH_CHECK();
  return 0;
}

// Whether a block can take a (row, kv head) whole: the meeting place of its waves in LDS (waves x heads of the tile x
// (d + 2) floats) must fit 64 KiB.
static bool whole_fits(int G, int d) {
  return (long)NW * (G < 16 ? G : 16) * (d + 2) * sizeof(float) <= 65536;
}

// Whether the blocks of a (row, kv head) can leave one partial result each and the last one finish (DEC_LAST): the
// meeting place must fit, and the maxima and sums of the blocks' results must fit into it afterwards.
static bool last_fits(int G, int d, int n_parts) {
  return whole_fits(G, d) && (n_parts + NW - 1) / NW <= 2 * (d + 2);
}

// Three ways (see attn_decode_kernel), chosen by the operands:
//   workspace null                every (row, kv head) is one block that finishes its heads itself
//                                 (`apc_attention_decode_whole_fits` says whether it can; n_parts is not used);
//   workspace and counters        workspace: n_rows * H * ceil(n_parts / 4) * (d + 2) floats; counters: one int per
//                                 (row, kv head tile) = n_rows * Hk * ceil(H / Hk / 16), zero before the first call
//                                 (every call leaves them zero); `apc_attention_decode_last_fits` says whether it can;
//   workspace, counters null      workspace: n_rows * H * n_parts * (d + 2) floats; a second kernel merges.
// keys_per_part: the keys of a part (a multiple of 32; the parts are counted from position 0, and n_parts of them
// must reach the longest row's position), or 0: every row's own keys in n_parts equal ranges (rows of any length;
// without a workspace in 4, one a wave of the pair's block).
// Calls that share counters or a workspace must not overlap (one stream).
APC_EXPORT int apc_attention_decode_bf16(const void* q, int ldq, int q_off, void* out, int ldo, int n_rows, int H,
                                         int Hk, int d, const void* cache, int page_tokens, const int* block_table,
                                         int max_blocks, const int* positions, const int* row_seg, const int* rows,
                                         int window, float scale, int keys_per_part, int n_parts, float* workspace,
                                         int* counters, hipStream_t stream) {
  if (n_rows <= 0) return 0;
  int e = check_common(q, ldq, q_off, cache, H, Hk, d, page_tokens);
  if (e) return e;
  if (keys_per_part < 0 || keys_per_part % 32 || max_blocks <= 0 || window < 0 || !out) return APC_ERR_BAD_ARG;
  if (keys_per_part / page_tokens + 2 > 64) return APC_ERR_BAD_ARG;  // a wave keeps one page id per lane
  const int G = H / Hk, gtiles = (G + 15) / 16;
  if (Hk * gtiles > 65535 || H > 65535) return APC_ERR_BAD_ARG;
  const size_t lds = (size_t)NW * (G < 16 ? G : 16) * (d + 2) * sizeof(float);
#define DEC_LAUNCH(DP_, MODE_, GRID_, LDS_, PARTS_, WS_, CTR_)                                                         \
  hipLaunchKernelGGL((attn_decode_kernel<DP_, MODE_>), GRID_, dim3(NW * 64), LDS_, stream, (const bf16_t*)q, ldq, q_off, \
                     H, Hk, d, (const bf16_t*)cache, page_tokens, block_table, max_blocks, positions, row_seg, rows,   \
                     window, scale, keys_per_part, PARTS_, WS_, (bf16_t*)out, ldo, CTR_)
#define DEC_BY_HEAD(MODE_, GRID_, LDS_, PARTS_, WS_, CTR_)            \
  if (d <= 32) DEC_LAUNCH(32, MODE_, GRID_, LDS_, PARTS_, WS_, CTR_);  \
  else if (d <= 64) DEC_LAUNCH(64, MODE_, GRID_, LDS_, PARTS_, WS_, CTR_);  \
  else if (d <= 96) DEC_LAUNCH(96, MODE_, GRID_, LDS_, PARTS_, WS_, CTR_);  \
  else if (d <= 128) DEC_LAUNCH(128, MODE_, GRID_, LDS_, PARTS_, WS_, CTR_); \
  else if (d <= 192) DEC_LAUNCH(192, MODE_, GRID_, LDS_, PARTS_, WS_, CTR_); \
  else DEC_LAUNCH(256, MODE_, GRID_, LDS_, PARTS_, WS_, CTR_)
  if (!workspace) {
    if (!whole_fits(G, d)) return APC_ERR_UNSUPPORTED;
    dim3 grid(n_rows, Hk * gtiles, 1);
    // without a length of the ranges every row's own keys go in NW equal ranges, one a wave
    DEC_BY_HEAD(DEC_WHOLE, grid, lds, NW, (float*)nullptr, (int*)nullptr);
    APC_LAUNCH_CHECK();
    return 0;
  }
  if (n_parts <= 0 || (n_parts + 3) / 4 > 65535) return APC_ERR_BAD_ARG;
  dim3 grid(n_rows, Hk * gtiles, (n_parts + NW - 1) / NW);
  if (counters) {
    if (!last_fits(G, d, n_parts)) return APC_ERR_UNSUPPORTED;
    DEC_BY_HEAD(DEC_LAST, grid, lds, n_parts, workspace, counters);
    APC_LAUNCH_CHECK();
    return 0;
  }
  DEC_BY_HEAD(DEC_PARTS, grid, 0, n_parts, workspace, (int*)nullptr);
#undef DEC_BY_HEAD
#undef DEC_LAUNCH
  APC_LAUNCH_CHECK();
  hipLaunchKernelGGL(attn_merge_kernel, dim3(n_rows, H), dim3(MERGE_NT), 0, stream,
                     workspace, n_parts, keys_per_part, H, d, positions, rows, window, (bf16_t*)out, ldo);
  APC_LAUNCH_CHECK();
  return 0;
}

// 1 if the blocks of a (row, kv head) can leave one partial result each and the last one finish, at these sizes.
APC_EXPORT int apc_attention_decode_last_fits(int H, int Hk, int d, int n_parts) {
  if (H <= 0 || Hk <= 0 || H % Hk || d <= 0 || n_parts <= 0) return 0;
  return last_fits(H / Hk, d, n_parts) ? 1 : 0;
}

// 1 if apc_attention_prefill_bf16 sends a step of `n_tiles` tiles with `n_rows` rows in all to the kernel of 128-row
// blocks (the only one that cuts a tile's keys into ranges and reads `parts`), else 0.
APC_EXPORT int apc_attention_prefill_wide_takes(int d, int page_tokens, int n_tiles, int n_rows) {
  return (n_tiles > 0 && attn_wide_takes(d, page_tokens) && (long)n_rows * 2 >= (long)n_tiles * TILE_ROWS) ? 1 : 0;
}

// Rows of a tile of the prefill kernels: the caller cuts every segment of several rows into tiles of at most this many
// consecutive rows (tile_row0, tile_rows).
APC_EXPORT int apc_attention_prefill_tile_rows() { return TILE_ROWS; }

// 1 if a block can take a (row, kv head) whole at these sizes (workspace = null above), else 0.
APC_EXPORT int apc_attention_decode_whole_fits(int H, int Hk, int d) {
  if (H <= 0 || Hk <= 0 || H % Hk || d <= 0) return 0;
  return whole_fits(H / Hk, d) ? 1 : 0;
}
