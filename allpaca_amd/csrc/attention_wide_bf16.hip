// Attention of prompt portions over the paged cache for head sizes of 128 and 64: tiles of 128 rows, keys and values
// straight from global memory into LDS, softmax and matrix products of one wave woven together by hand.  (The text
// below gives the figures of a head size of 128; what a head size of 64 changes stands at its end.)
//
// A block of 4 waves takes up to 128 consecutive rows of one request and one head: wave (rh, kh) owns the rows
// rh * 64 .. + 63 (two MFMA tiles of 32 rows, "row tiles") and the keys kh * 32 .. + 31 of every tile of 64 keys, with a
// reference and a sum per row of its own; the two waves of a row half meet once at the end through LDS.  As in
// attention_bf16.hip the products are S^T = K Q^T and O^T = V^T P^T on v_mfma_f32_32x32x16_bf16, so a lane holds
// scores of one row and P goes from the first product's result registers into the second product's operand.
// What differs from the 64-row kernel there, and why (that kernel ran at 28 % of the matrix cores' rate on long
// prompts, with LDS, vector instructions and matrix cores each busy half of the time and waiting for one another):
// * An operand read from LDS feeds two MFMAs (the two row tiles of the wave) instead of one: one read per MFMA is
//   all that LDS can deliver when the matrix cores run at their full rate.
// * Keys and values go from global memory into LDS by direct loads (no registers, no LDS store instructions, no
//   address arithmetic: a wave's 16 keys lie in one page, whose descriptors sit in scalar registers), three passes
//   ahead of their use in four stages.  K rows are not padded; a piece of 16 bytes lies at (piece index XOR row
//   index) instead, which the direct load does by fetching the piece that belongs at its lane's place, and reads of
//   16 lanes still fall into different banks.  The rows of a K tile are stored in the order in which the first
//   product's result registers want them (bits 2 and 3 of the key index swapped), so that a lane's 8 results of a
//   16-key step are 8 consecutive keys and the matching values are one 16-byte piece of V^T as a page holds it.
//   V^T lies in LDS by groups of 16 keys, [half of the keys][element of d]: a wave's read of 32 elements x 16 keys is
//   1 KiB in lane order.
// * One wave a SIMD (O of 64 rows x 128 alone takes 128 accumulation registers, the query rows 64 more), so
//   nothing overlaps by itself: a pass of the loop is two slots of 16 MFMAs each, and the vector work of one row
//   tile's softmax stands in the issue slots between the MFMAs of the other's products:
//     slot A: S0(i + 1) = K(i + 1) Q0 and O0 += V(i) P0(i), beside the softmax of S1(i)
//     slot B: S1(i + 1) = K(i + 1) Q1 and O1 += V(i) P1(i), beside the softmax of S0(i + 1)
//   (0, 1: the row tiles; i: the tile of keys).  The fragments of K(i + 1) and V(i) stay in registers through both
//   slots; slot B asks LDS for the next pass's fragments as soon as a fragment's registers are free (the MFMA behind
//   the one that read them has gone out), half a pass before they are used, and issues the direct loads, one a step.
//   The block's one barrier a pass stands between the slots.  Each result is written in one slot and read in the
//   next, so nothing needs a second set of registers and the loop body has no branch.
// * A row's reference for the exponents is the largest score among its first keys (the first tile of its wave that
//   it sees a key of) and stays: O lives in accumulation registers that only MFMAs touch in the loop, so it cannot
//   shrink there.  P = 2^(score - reference) may then exceed 1; sums stay far inside float32 as long as no P goes
//   beyond 2^64 (passes that look at the maximum) or the sum beyond 2^90 (checked at the end).  A block in which that
//   happens throws its work away and computes its rows again in a plain loop (one thing after the other, references
//   that move, as attn_prefill32_kernel does).
// * Passes in which every row sees every key of both tiles in work, and has its reference, take a softmax without
//   masks and without a maximum (16 x (fma, exp), 8 x (pack, add to the sum) a row tile); a block's first passes
//   (until every row has its reference) take the general one, and the last few, under the causal mask, one with
//   masks but no maximum.  The three kinds of passes are three loops one after the other.
// The MFMAs are written as instructions: the compiler does not know them, so it neither waits for their results
// nor keeps reads behind them; the order of the slots keeps every read of a result at least one MFMA behind the
// one that wrote it, and a wait stands at the end of a block's last pass, behind which the compiler may read the
// accumulators to write the rows (between the loops it leaves them where they are: no loop and no place between two
// loops has a move of an accumulator, which is worth checking in the compiler's output after a change).
// Positions outside a block's view that lie in stale slots are cleared in LDS before the value product sees them
// (only tiles at the edge of a request's keys have any).
// A step of few tiles (a chunk of 512 prompt tokens is 4 tiles x 32 heads = 128 blocks for 256 compute units) may have
// the keys of every tile cut into ranges of whole key tiles, a block each: a block then leaves its rows as float32
// with their reference and sum, and attn_wide_merge_kernel adds the ranges (512 rows over 32,768 keys: 449 -> 288 us;
// 128 rows: 424 -> 109 us; at 2,048 keys nothing is gained, the caller cuts from 4,096 keys on).
// Tried and not kept: O in fixed registers so that instructions written out could shrink it (the compiler then moved O
// to the vector registers and back in every pass); one loop that chooses the kind of pass each time (two copies of O,
// one moved into the other every pass); the direct loads of K in slot A (the general passes ran out of registers,
// and the compiler's moves of accumulators read MFMA results too early); K and V fragments read for this pass only,
// two steps ahead (same speed: the wave waits for LDS either way, see the counters in profiles/).
// Heads of 64 (the kernel's parameter HD): half the fragments, MFMAs and direct loads a slot for the same softmax, whose
// 16 steps a slot stand four to a pair of MFMAs instead of two; a row of K is 128 bytes, so a direct load brings 8 rows
// and a piece lies at (piece index XOR (row / 2) % 8).  Its 64 KiB of stages and 256 registers a lane (the kernel is
// compiled for two waves a SIMD at this head size) let two blocks share a compute unit, one's softmax beside the
// other's MFMAs.  Measured at 32 heads, 2,048 rows over 32,768 keys: 643 us (828 TFLOP/s; one block a compute unit:
// 742 us; the 64-row kernels: 543 TFLOP/s), 2,048 rows over 2,048 keys 49 us; the softmax's vector instructions bound
// it (118 of them beside 16 MFMAs in the short pass).
// (Two blocks a compute unit once gave rows that differed from run to run; the cause was two LDS reads without a
// taker, see lds_frag below, not the waits on the direct loads: with those reads gone the same waits give equal
// bits with two blocks a compute unit.)
// Formula: crates/allpaca-cpu/src/kernels.rs:293-356.  Reference kernel (contiguous K/V, no matrix cores):
// attention_qtile_kernel hip/src/kernels.cpp:2203.
#include "attention_wide.h"
#include "mfma.h"
#include <math.h>
#include <mutex>
#include <type_traits>
#include <utility>

namespace {

constexpr int KT = 64;                     // keys a tile
constexpr int STG = 4;                     // stages of K and of V in LDS
// bytes of the stages for a head size of hd (the block asks for 16 more): K [64 rows][2 hd], V^T [4 groups of 16
// keys][hd elements][32]
constexpr int lds_bytes(int hd) { return STG * (KT * hd * 2 + hd * KT * 2); }
// What a launch asks for: the stages and a flag behind them.  Heads of 64 leave room for two blocks a compute unit
// (64 KiB each, and the kernel is compiled for 256 registers a lane there).
constexpr int lds_request(int hd) { return lds_bytes(hd) + 16; }
constexpr float LOG2E = 1.4426950408889634f;
constexpr float RISE = 64.f;               // by how much (in powers of 2) a score may exceed its row's reference

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) void* lds_ptr;

// The fragments of K and V come out of LDS through ds_read_b128 written as an instruction, and the MFMA that takes one
// waits for it by count (LDS returns in order; LGKM = how many younger LDS reads may still be out).  Left to the
// compiler, every LDS read behind a direct load waits until all direct loads have landed: it cannot tell that the
// loads in flight fill other stages than the one being read.
// The compiler takes the result of such a read for finished when the instruction has gone out.  So every read's
// registers must be taken by a statement that waits for it (an MFMA with its count, or reads_done below) while the
// compiler still holds them for the fragment: registers of a fragment that nothing takes any more are handed to the
// next value at once, and the fragment then arrives on top of that value, sooner or later with the load on LDS.
// (That happened here twice: the prologue read the last V fragment, which the first pass reads again, and the
// softmax temporaries of the first tile got its registers, 128 cycles of s_nop behind the read; and the fragments
// that the last pass asks for the pass that never comes were still out when the rows' sums moved into their
// registers.  With one block a compute unit LDS answered in time; with a second block's reads and direct loads on the
// same LDS it did not always, and rows differed from run to run.  tests/test_kernel_waits.py checks the compiler's
// output for both patterns.)
template <int OFFSET>
__device__ __forceinline__ Frag lds_frag(int addr) {
  u32x4 v;
  asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "n"(OFFSET));
  return __builtin_bit_cast(Frag, v);
}
// waits for every LDS read of this wave and holds the fragments' registers until then
template <int N>
__device__ __forceinline__ void reads_done(const Frag (&a)[N], const Frag (&b)[N]) {
  static_assert(N == 4 || N == 8, "one operand a fragment");
  u32x4 x[2 * N];
#pragma unroll
  for (int g = 0; g < N; ++g) {
    x[g] = __builtin_bit_cast(u32x4, a[g]);
    x[N + g] = __builtin_bit_cast(u32x4, b[g]);
  }
  if constexpr (N == 4)
    asm volatile("s_waitcnt lgkmcnt(0)" ::"v"(x[0]), "v"(x[1]), "v"(x[2]), "v"(x[3]), "v"(x[4]), "v"(x[5]), "v"(x[6]), "v"(x[7]));
  else
    asm volatile("s_waitcnt lgkmcnt(0)" ::"v"(x[0]), "v"(x[1]), "v"(x[2]), "v"(x[3]), "v"(x[4]), "v"(x[5]), "v"(x[6]), "v"(x[7]),
                 "v"(x[8]), "v"(x[9]), "v"(x[10]), "v"(x[11]), "v"(x[12]), "v"(x[13]), "v"(x[14]), "v"(x[15]));
}
constexpr int NO_WAIT = -1;  // an operand that has been in registers for long
// c = a . q and c += a . q with the result in vector registers and q, the wave's query rows, which only MFMAs read, in
// accumulation registers (an MFMA takes its operands from either file); c += a . b with c in accumulation registers.
template <int LGKM>
__device__ __forceinline__ void mfma_set(floatx16& c, const Frag& a, const Frag& q) {
  const u32x4 av = __builtin_bit_cast(u32x4, a), qv = __builtin_bit_cast(u32x4, q);
  if constexpr (LGKM < 0) asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, 0" : "=&v"(c) : "v"(av), "a"(qv));
  else asm volatile("s_waitcnt lgkmcnt(%3)\n\tv_mfma_f32_32x32x16_bf16 %0, %1, %2, 0" : "=&v"(c) : "v"(av), "a"(qv), "n"(LGKM));
}
template <int LGKM>
__device__ __forceinline__ void mfma_add(floatx16& c, const Frag& a, const Frag& q) {
  const u32x4 av = __builtin_bit_cast(u32x4, a), qv = __builtin_bit_cast(u32x4, q);
  if constexpr (LGKM < 0) asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(c) : "v"(av), "a"(qv));
  else asm volatile("s_waitcnt lgkmcnt(%3)\n\tv_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(c) : "v"(av), "a"(qv), "n"(LGKM));
}
template <int LGKM>
__device__ __forceinline__ void mfma_acc(floatx16& c, const Frag& a, const Frag& b) {
  const u32x4 av = __builtin_bit_cast(u32x4, a), bv = __builtin_bit_cast(u32x4, b);
  if constexpr (LGKM < 0) asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+a"(c) : "v"(av), "v"(bv));
  else asm volatile("s_waitcnt lgkmcnt(%3)\n\tv_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+a"(c) : "v"(av), "v"(bv), "n"(LGKM));
}

template <int N>
__device__ __forceinline__ void wait_loads_but() {  // until at most N vector memory loads of this wave are in flight
  __builtin_amdgcn_s_waitcnt(((N & 15) | ((N >> 4) << 14)) | 0x0f70);
}

// The two halves of a wave exchange a value: every lane gets f(lower half's value, upper half's value).
__device__ __forceinline__ float halves_max(float v) {
  const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float halves_sum(float v) {
  const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}
__device__ __forceinline__ float exp2_neg(float x) { return __builtin_amdgcn_exp2f(x); }
// The largest of 8 scores and m, as instructions: fmaxf on values the compiler has not seen computed first makes each
// of them canonical (one more instruction each), and one statement keeps the compiler's guard against what an unknown
// instruction may need (a wait state in front of every reader) to one place.
__device__ __forceinline__ float max_of_8(float m, const floatx16& s, int r0) {
  float r;
  if (r0 == 0)
    asm("v_max3_f32 %0, %1, %2, %3\n\tv_max3_f32 %0, %0, %4, %5\n\tv_max3_f32 %0, %0, %6, %7\n\tv_max3_f32 %0, %0, %8, %9"
        : "=&v"(r) : "v"(m), "v"(s[0]), "v"(s[1]), "v"(s[2]), "v"(s[3]), "v"(s[4]), "v"(s[5]), "v"(s[6]), "v"(s[7]));
  else
    asm("v_max3_f32 %0, %1, %2, %3\n\tv_max3_f32 %0, %0, %4, %5\n\tv_max3_f32 %0, %0, %6, %7\n\tv_max3_f32 %0, %0, %8, %9"
        : "=&v"(r) : "v"(m), "v"(s[8]), "v"(s[9]), "v"(s[10]), "v"(s[11]), "v"(s[12]), "v"(s[13]), "v"(s[14]), "v"(s[15]));
  return r;
}
// sum + the two bfloat16 values of `pair` (v_dot2c_f32_bf16 with a pair of ones): the row's sum is taken over P as the
// value product sees it, two values an instruction
__device__ __forceinline__ float add_pair(float sum, uint32_t pair) {
  typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
  const bf16x2_t ones = {(__bf16)1.0f, (__bf16)1.0f};
  return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, pair), ones, sum, false);
}

// all but the positions lo <= p < hi of the 8 that a value piece holds are cleared
__device__ __forceinline__ void keep_positions(Frag& v, int lo, int hi) {
#pragma unroll
  for (int w = 0; w < 4; ++w) {
    const uint32_t a = (2 * w >= lo && 2 * w < hi) ? 0x0000ffffu : 0u;
    const uint32_t b = (2 * w + 1 >= lo && 2 * w + 1 < hi) ? 0xffff0000u : 0u;
    v.w[w] &= a | b;
  }
}

// Softmax state of one row tile of a wave (a lane: one row, half of the wave's 32 keys of a tile)
struct Soft {
  float m, l;      // the row's reference (-inf before its first key) and sum
  float mx, sum;   // of the tile in work
  int beyond;      // a score went beyond the reference by more than RISE: the woven loop's result is not to be used
  int pos, lo;     // the row sees keys lo .. pos
};

// Step h (0..15) of the softmax of 16 scores: the work is cut up so that it can stand between MFMAs.  s: raw
// scores, then P; pf: P as the second product's operand; tk: the first of the wave's 32 keys of this tile.
// Register r of a lane holds key tk + 16 (r / 8) + 8 lh + r % 8.
__device__ __forceinline__ constexpr int score_step(int r) { return 3 + r * 12 / 16; }
template <bool MASKED>
__device__ __forceinline__ void soft_step(int h, floatx16& s, Frag (&pf)[2], Soft& st, int tk, int lh, float sc2) {
  if (h == 0 || h == 1) {
    const int r0 = h * 8;
    if (MASKED) {
      // key tk + 8 lh + c with c = 16 (r / 8) + r % 8: seen if lo <= key <= pos, that is first <= c <= last
      const int base = tk + 8 * lh, first = st.lo - base, last = st.pos - base;
#pragma unroll
      for (int r = r0; r < r0 + 8; ++r) {
        const int c = 16 * (r / 8) + r % 8;
        s[r] = (c >= first && c <= last) ? s[r] : -INFINITY;
      }
    }
    const float mx = max_of_8(h == 0 ? -INFINITY : st.mx, s, r0);
    st.mx = h == 0 ? mx : halves_max(mx) * sc2;
  }
  if (h == 2) {
    const bool fresh = st.m == -INFINITY;
    st.beyond |= (!fresh && st.mx > st.m + RISE) ? 1 : 0;
    st.m = fresh ? st.mx : st.m;
    st.sum = 0.f;
  }
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    // a row that has seen no key yet: m = -inf and every score is -inf; -inf - -inf would be NaN
    if (score_step(r) == h) s[r] = exp2_neg(fmaf(s[r], sc2, st.m == -INFINITY ? 0.f : -st.m));
    if ((r & 1) && score_step(r) + 1 == h) {
      const uint32_t pair = pack_bf16x2(s[r - 1], s[r]);
      pf[r / 8].w[(r % 8) / 2] = pair;
      st.sum = add_pair(st.sum, pair);
    }
  }
  if (h == 15) st.l += halves_sum(st.sum);
}

// The same for a tile all of whose keys every row sees, when every row has its reference: no masks and no maximum
// (a P beyond float32 shows in the sum, which is checked when all is done).  One score a step; the sum runs on
// over the tiles per lane, and the two halves of the wave add theirs when the loop of such passes ends.
__device__ __forceinline__ void soft_step_seen(int h, floatx16& s, Frag (&pf)[2], Soft& st, float sc2) {
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    if (r == h) s[r] = exp2_neg(fmaf(s[r], sc2, -st.m));
    // a pair is packed two steps behind its second value: an exponential's result wants a wait state before its reader
    if ((r & 1) && (r + 2 == h || (r == 15 && h == 15))) {
      const uint32_t pair = pack_bf16x2(s[r - 1], s[r]);
      pf[r / 8].w[(r % 8) / 2] = pair;
      st.sum = add_pair(st.sum, pair);
    }
  }
}
// The same with masks, for rows that have their reference: what a block's last passes need (a row's first keys lie
// in its first passes).  A key that the row does not see gets the exponent -inf.
__device__ __forceinline__ void soft_step_late(int h, floatx16& s, Frag (&pf)[2], Soft& st, int tk, int lh, float sc2) {
  const int base = tk + 8 * lh, first = st.lo - base, last = st.pos - base;
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    const int c = 16 * (r / 8) + r % 8;
    if (r == h) s[r] = exp2_neg((c >= first && c <= last) ? fmaf(s[r], sc2, -st.m) : -INFINITY);
    if ((r & 1) && (r + 2 == h || (r == 15 && h == 15))) {
      const uint32_t pair = pack_bf16x2(s[r - 1], s[r]);
      pf[r / 8].w[(r % 8) / 2] = pair;
      st.sum = add_pair(st.sum, pair);
    }
  }
}
enum { SOFT_MASKED = 0, SOFT_SEEN = 1, SOFT_LATE = 2 };
template <int MODE>
__device__ __forceinline__ void soft_any(int h, floatx16& s, Frag (&pf)[2], Soft& st, int tk, int lh, float sc2) {
  if constexpr (MODE == SOFT_SEEN) soft_step_seen(h, s, pf, st, sc2);
  else if constexpr (MODE == SOFT_LATE) soft_step_late(h, s, pf, st, tk, lh, sc2);
  else soft_step<true>(h, s, pf, st, tk, lh, sc2);
}

// WIN: the rows see a window of keys (without one, a row's first key is key 0, which costs no register)
// HD: the head size, 128 or 64 (half the MFMAs a pass for the same softmax)
template <int HD, bool WIN>
__global__ __launch_bounds__(256, HD == 64 ? 2 : 1) void attn_prefill_wide_kernel(
    const bf16_t* __restrict__ q, int ldq, int q_off, bf16_t* __restrict__ out, int ldo, int H, int Hk,
    const bf16_t* __restrict__ cache, int lgP, const int* __restrict__ block_table, int max_blocks,
    const int* __restrict__ positions, const int* __restrict__ row_seg, const int* __restrict__ tile_row0,
    const int* __restrict__ tile_rows, int n_tiles, int window_arg, float scale, int n_splits, int part_rows,
    float* __restrict__ parts) {
  extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];
  const int window = WIN ? window_arg : 0;
  constexpr int d = HD;
  constexpr int DT = d / 32;                 // tiles of 32 elements of a head; also a wave's direct loads per K or V tile
  constexpr int NG = d / 16;                 // fragments of K, and of V, that a wave takes of a tile
  constexpr int K_STAGE = KT * HD * 2, V_STAGE = HD * KT * 2, V_BASE = STG * K_STAGE, LDS_BYTES = lds_bytes(HD);
  constexpr int LOADS_PER_TILE = 2 * DT;     // a wave's direct loads per pass of the loop
  constexpr int ROW_BYTES = d * 2;           // of a row of K in LDS
  constexpr int PPR = d / 8;                 // 16-byte pieces of such a row
  const int P = 1 << lgP;
  const int tid = threadIdx.x, lane = tid % WAVE, wave = __builtin_amdgcn_readfirstlane(tid / WAVE);
  const int li = lane % 32, lh = lane / 32;
  const int rh = wave / 2, kh = wave % 2;  // half of the rows, half of each tile's keys
  int tile, h, split;
  {
    // heads of one kv head go to one XCD (their keys and values then lie in one L2), long tiles first
    const int id = blockIdx.x, G = H / Hk;
    if (Hk % 8 == 0) {
      const int xcd = id % 8;
      int slot = id / 8;
      split = slot % n_splits;
      slot /= n_splits;
      const int lhd = slot / n_tiles;
      tile = n_tiles - 1 - slot % n_tiles;
      h = (xcd + 8 * (lhd / G)) * G + lhd % G;
    } else {
      split = id % n_splits;
      tile = n_tiles - 1 - (id / n_splits) % n_tiles;
      h = id / n_splits / n_tiles;
    }
  }
  const int row0 = tile_row0[tile], nrows = tile_rows[tile];
  const int kvh = h / (H / Hk);
  const int pos0 = positions[row0];
  const int* bt = block_table + (size_t)row_seg[row0] * max_blocks;
  const int first = (window > 0 && pos0 - window + 1 > 0) ? pos0 - window + 1 : 0;
  const size_t page_stride = (size_t)2 * Hk * P * d;
  // The keys of the block: those its rows see, or with the tile's keys cut into n_splits ranges of whole key tiles,
  // one of them: `last` is then the range's last key, the rows see nothing beyond it, and what the block leaves is a
  // partial result that attn_wide_merge_kernel adds to the other ranges'.
  int t_begin = (first / KT) * KT;
  int last = pos0 + nrows - 1;
  if (n_splits > 1) {
    const int per = ceil_div((last - t_begin) / KT + 1, n_splits);
    t_begin += split * per * KT;
    last = min(last, t_begin + per * KT - 1);
  }
  // Where a block with a range of keys leaves its rows: [range][row][head][d] floats, then [range][row][head][m, l].
  // Worked out where it is needed, from the kernel's arguments, so that nothing of it lives through the loop.
  auto part_index = [&]() {
    const int id = blockIdx.x;
    const int sp = (Hk % 8 == 0 ? id / 8 : id) % n_splits;
    return (size_t)sp * part_rows * H + h;  // + row * H
  };
  if (t_begin > last) {  // more ranges than key tiles: nothing here
    if (parts && tid < nrows) {
      float* ml = parts + (size_t)n_splits * part_rows * H * d + (part_index() + (size_t)(row0 + tid) * H) * 2;
      ml[0] = -INFINITY;
      ml[1] = 0.f;
    }
    return;
  }
  const int n_kt = (last - t_begin) / KT + 1;
  const int last16 = (last / 16) * 16;
  const bf16_t* k_head = cache + (size_t)kvh * P * d;
  const bf16_t* v_head = cache + (size_t)(Hk + kvh) * P * d;
  const float sc2 = scale * LOG2E;

  // the wave's 2 x 32 query rows as second operands: row = lane % 32, 8 elements of d per lane and step of 16
  Frag qf[2][d / 16];
  Soft st[2];
  u32x4 qv[2][d / 16];  // on their way from memory while the first keys and values are asked for
  {
#pragma unroll
    for (int rt = 0; rt < 2; ++rt) {
      const int my_row = rh * 64 + rt * 32 + li;
      const bf16_t* qrow = q + (size_t)(row0 + min(my_row, nrows - 1)) * ldq + q_off + (size_t)h * d;
#pragma unroll
      for (int ks = 0; ks < d / 16; ++ks) qv[rt][ks] = __builtin_bit_cast(u32x4, load_frag(qrow + ks * 16 + lh * 8));
      st[rt].m = -INFINITY;
      st[rt].l = 0.f;
      st[rt].mx = st[rt].sum = 0.f;
      st[rt].beyond = 0;
      st[rt].pos = min(pos0 + my_row, last);
      st[rt].lo = (window > 0 && pos0 + my_row - window + 1 > 0) ? pos0 + my_row - window + 1 : 0;
    }
  }
  // whether every row of row tile rt sees all of the wave's 32 keys of the tile that starts at t0
  auto sees_all = [&](int rt, int t0) {
    const int tk = t0 + kh * 32, low = min(pos0 + rh * 64 + rt * 32, last), top = pos0 + rh * 64 + rt * 32 + 31;
    const int win_lo = (window > 0 && top - window + 1 > 0) ? top - window + 1 : 0;
    return tk + 31 <= low && tk >= win_lo;
  };

  // ---- direct loads.  Wave w brings the keys 16 w .. + 15 of a tile and their values: they lie in one page (pages
  // hold a multiple of 16 positions), whose descriptors sit in scalar registers, so a load costs no address arithmetic.
  // K: load i brings LDS rows 16 w + 4 i .. + 3 = keys 16 w + 4 sw(i) .. + 3, lane -> (row lane / 16, place lane % 16,
  // which holds piece place ^ row).  V^T: load i brings elements 32 i .. + 31 of the wave's 16 keys, lane -> (element
  // lane / 2, half lane % 2), into [group w][element][16 keys].
  // The 4 loads of a tile's K (and of its V) differ by 1 KiB in LDS, which the instruction's offset field gives; that
  // field counts for the address in memory too, so the lanes' offsets take it back (and 3 KiB more, which the base
  // gives back, so that none is negative).
  // (The lanes' offsets of the 4 loads of V differ by the same step, which goes into the loads' scalar offset: one
  // register instead of four.)
  // (Heads of 64: a row of K is 128 bytes, a load brings 8 of them, and a piece lies at piece ^ (row / 2) % 8, so that
  // the rows r and r + 8, which share a place, differ in the half of the 256 bytes of banks they fall into.)
  auto k_swizzle = [](int row) { return HD == 128 ? row % 16 : (row >> 1) & 7; };
  int koff[DT];
#pragma unroll
  for (int i = 0; i < DT; ++i) {
    if constexpr (HD == 128) {
      const int sw = 2 * (i & 1) + (i >> 1);
      koff[i] = (4 * sw + lane / 16) * (d * 2) + (((lane % 16) ^ (lane / 16) ^ (4 * i)) * 16) + 3072 - i * 1024;
    } else {
      const int row = 8 * i + lane / PPR;                       // LDS row among the wave's 16
      const int g = row / 4, key = 4 * (2 * (g & 1) + (g >> 1)) + row % 4;
      koff[i] = key * ROW_BYTES + (((lane % PPR) ^ k_swizzle(row)) * 16) + (DT - 1) * 1024 - i * 1024;
    }
  }
  // (as scalars for the loads below: with the array itself named in them, the host's pass of the compiler left the
  // kernel's launch stub out without a word)
  const int koff0 = koff[0], koff1 = koff[1], koff2 = koff[DT > 2 ? 2 : 0], koff3 = koff[DT > 2 ? 3 : 0];
  const int voff = (lane % 32) * (P * 2) + (lane / 32) * 16 + (DT - 1) * 1024;
  const int vstep = 32 * P * 2 - 1024;  // load i: elements 32 i .. of a page row of 2 P bytes, 1 KiB further in LDS
  auto group_of = [&](int j) { return min(t_begin + j * KT + 16 * wave, last16); };  // first key of the wave's 16
  auto page_of = [&](int j) { return __builtin_amdgcn_readfirstlane(bt[group_of(j) >> lgP]); };
  const bf16_t* k_head_low = k_head - (DT - 1) * 512;  // 3 KiB lower (1 KiB with two loads a tile)
  const bf16_t* v_head_low = v_head - (DT - 1) * 512;
  // one of the 4 loads of a tile's K or V (to stand between other work)
  auto k_load_piece = [&](int j, int page, int i) {
    const BufferRsrc kr = make_rsrc(k_head_low + (size_t)__builtin_amdgcn_readfirstlane(page) * page_stride);
    const int soff = (group_of(j) & (P - 1)) * (d * 2);
    const lds_ptr dst = (lds_ptr)(smem + (j % STG) * K_STAGE + (16 * wave) * ROW_BYTES);
    if (i == 0) __builtin_amdgcn_raw_ptr_buffer_load_lds(kr, dst, 16, koff0, soff, 0, 0);
    if (i == 1) __builtin_amdgcn_raw_ptr_buffer_load_lds(kr, dst, 16, koff1, soff, 1024, 0);
    if constexpr (DT > 2) {
      if (i == 2) __builtin_amdgcn_raw_ptr_buffer_load_lds(kr, dst, 16, koff2, soff, 2048, 0);
      if (i == 3) __builtin_amdgcn_raw_ptr_buffer_load_lds(kr, dst, 16, koff3, soff, 3072, 0);
    }
  };
  auto v_load_piece = [&](int j, int page, int i) {
    const BufferRsrc vr = make_rsrc(v_head_low + (size_t)__builtin_amdgcn_readfirstlane(page) * page_stride);
    const int soff = (group_of(j) & (P - 1)) * 2;
    const lds_ptr dst = (lds_ptr)(smem + V_BASE + (j % STG) * V_STAGE + wave * (DT * 1024));
    if (i == 0) __builtin_amdgcn_raw_ptr_buffer_load_lds(vr, dst, 16, voff, soff, 0, 0);
    if (i == 1) __builtin_amdgcn_raw_ptr_buffer_load_lds(vr, dst, 16, voff, soff + vstep, 1024, 0);
    if constexpr (DT > 2) {
      if (i == 2) __builtin_amdgcn_raw_ptr_buffer_load_lds(vr, dst, 16, voff, soff + 2 * vstep, 2048, 0);
      if (i == 3) __builtin_amdgcn_raw_ptr_buffer_load_lds(vr, dst, 16, voff, soff + 3 * vstep, 3072, 0);
    }
  };
  auto k_load = [&](int j, int page) {
    const BufferRsrc kr = make_rsrc(k_head_low + (size_t)__builtin_amdgcn_readfirstlane(page) * page_stride);
    const int soff = (group_of(j) & (P - 1)) * (d * 2);
    const lds_ptr dst = (lds_ptr)(smem + (j % STG) * K_STAGE + (16 * wave) * ROW_BYTES);
    __builtin_amdgcn_raw_ptr_buffer_load_lds(kr, dst, 16, koff0, soff, 0, 0);
    __builtin_amdgcn_raw_ptr_buffer_load_lds(kr, dst, 16, koff1, soff, 1024, 0);
    if constexpr (DT > 2) {
      __builtin_amdgcn_raw_ptr_buffer_load_lds(kr, dst, 16, koff2, soff, 2048, 0);
      __builtin_amdgcn_raw_ptr_buffer_load_lds(kr, dst, 16, koff3, soff, 3072, 0);
    }
  };
  auto v_load = [&](int j, int page) {
    const BufferRsrc vr = make_rsrc(v_head_low + (size_t)__builtin_amdgcn_readfirstlane(page) * page_stride);
    const int soff = (group_of(j) & (P - 1)) * 2;
    const lds_ptr dst = (lds_ptr)(smem + V_BASE + (j % STG) * V_STAGE + wave * (DT * 1024));
    __builtin_amdgcn_raw_ptr_buffer_load_lds(vr, dst, 16, voff, soff, 0, 0);
    __builtin_amdgcn_raw_ptr_buffer_load_lds(vr, dst, 16, voff, soff + vstep, 1024, 0);
    if constexpr (DT > 2) {
      __builtin_amdgcn_raw_ptr_buffer_load_lds(vr, dst, 16, voff, soff + 2 * vstep, 2048, 0);
      __builtin_amdgcn_raw_ptr_buffer_load_lds(vr, dst, 16, voff, soff + 3 * vstep, 3072, 0);
    }
  };
  // The same with the lanes' offsets worked out on the spot, for the passes that have no register to spare for them
  // (the compiler would otherwise keep them through the loop and spill something else)
  auto kv_load_tight = [&](int jk, int pagek, int jv, int pagev) {
    int ln = lane;
    asm volatile("" : "+v"(ln));
    const BufferRsrc kr = make_rsrc(k_head_low + (size_t)__builtin_amdgcn_readfirstlane(pagek) * page_stride);
    const int ksoff = (group_of(jk) & (P - 1)) * (d * 2);
    const lds_ptr kdst = (lds_ptr)(smem + (jk % STG) * K_STAGE + (16 * wave) * ROW_BYTES);
    if constexpr (HD == 128) {
      const int x = (ln / 16) * (d * 2) + (((ln % 16) ^ (ln / 16)) * 16);  // (row, place) of load 0; load i: place ^ 4 i
      __builtin_amdgcn_raw_ptr_buffer_load_lds(kr, kdst, 16, x + 3072, ksoff, 0, 0);
      __builtin_amdgcn_raw_ptr_buffer_load_lds(kr, kdst, 16, (x ^ 64) + 8 * (d * 2) + 2048, ksoff, 1024, 0);
      __builtin_amdgcn_raw_ptr_buffer_load_lds(kr, kdst, 16, (x ^ 128) + 4 * (d * 2) + 1024, ksoff, 2048, 0);
      __builtin_amdgcn_raw_ptr_buffer_load_lds(kr, kdst, 16, (x ^ 192) + 12 * (d * 2), ksoff, 3072, 0);
    } else {
#pragma unroll
      for (int i = 0; i < DT; ++i) {
        const int row = 8 * i + ln / PPR;
        const int g = row / 4, key = 4 * (2 * (g & 1) + (g >> 1)) + row % 4;
        const int off = key * ROW_BYTES + (((ln % PPR) ^ k_swizzle(row)) * 16) + (DT - 1) * 1024 - i * 1024;
        if (i == 0) __builtin_amdgcn_raw_ptr_buffer_load_lds(kr, kdst, 16, off, ksoff, 0, 0);
        else __builtin_amdgcn_raw_ptr_buffer_load_lds(kr, kdst, 16, off, ksoff, 1024, 0);
      }
    }
    const BufferRsrc vr = make_rsrc(v_head_low + (size_t)__builtin_amdgcn_readfirstlane(pagev) * page_stride);
    const int vsoff = (group_of(jv) & (P - 1)) * 2;
    const lds_ptr vdst = (lds_ptr)(smem + V_BASE + (jv % STG) * V_STAGE + wave * (DT * 1024));
    const int vo = (ln % 32) * (P * 2) + (ln / 32) * 16 + (DT - 1) * 1024;
    __builtin_amdgcn_raw_ptr_buffer_load_lds(vr, vdst, 16, vo, vsoff, 0, 0);
    __builtin_amdgcn_raw_ptr_buffer_load_lds(vr, vdst, 16, vo, vsoff + vstep, 1024, 0);
    if constexpr (DT > 2) {
      __builtin_amdgcn_raw_ptr_buffer_load_lds(vr, vdst, 16, vo, vsoff + 2 * vstep, 2048, 0);
      __builtin_amdgcn_raw_ptr_buffer_load_lds(vr, vdst, 16, vo, vsoff + 3 * vstep, 3072, 0);
    }
  };
  // Stale positions of the V^T stage of tile j are cleared: what lies beyond the last key or in front of the first
  // one that a row of the block sees may be anything, and 0 x NaN is NaN.  (A group of 16 keys beyond the last one
  // holds a copy of the last group.)
  auto clear_unseen = [&](int j) {
    const int t0 = t_begin + j * KT;
    unsigned char* stage = smem + V_BASE + (j % STG) * V_STAGE;
    for (int idx = tid; idx < HD * 8; idx += 256) {  // piece idx: group idx / (2 HD), half (idx % 64) / 32 of an element
      const int t16 = t0 + 16 * (idx / (HD * 2)), tg = t16 + 8 * ((idx % 64) / 32);
      Frag* piece = reinterpret_cast<Frag*>(stage + idx * 16);
      if (t16 > last16) {
        *piece = zero_frag();
      } else if (first - tg > 0 || last - tg + 1 < 8) {
        Frag f = *piece;
        keep_positions(f, first - tg, last - tg + 1);
        *piece = f;
      }
    }
  };
  auto at_edge = [&](int j) {
    const int t0 = t_begin + j * KT;
    return t0 < first || t0 + KT - 1 > last;
  };

  // ---- operand reads.  K: lane (li, lh) reads piece 2 ks + lh of LDS row kh * 32 + li; V^T: the 16 keys' group
  // 2 kh + j, element dt * 32 + li, half lh.
  // (byte offsets in `smem`; the read instruction wants addresses in LDS, which begin at lds0)
  const int lds0 = (int)(uintptr_t)(__attribute__((address_space(3))) unsigned char*)smem;
  int kaddr[d / 16];
#pragma unroll
  for (int ks = 0; ks < d / 16; ++ks) kaddr[ks] = (kh * 32 + li) * ROW_BYTES + ((((2 * ks) | lh) ^ k_swizzle(li)) * 16);
  const int vaddr = V_BASE + 2 * kh * (DT * 1024) + lane * 16;
  auto k_frag = [&](int stage_bytes, int ks) { return lds_frag<0>(lds0 + kaddr[ks] + stage_bytes); };
  // fragment g: the group of 16 keys g / DT, the elements 32 (g % DT) ..  All but the last one: slot A of every pass
  // reads that one itself, and a read whose result nobody takes must not be asked for (see lds_frag).
  auto read_v_frags_but_last = [&](Frag (&vf)[NG], int va) {
    vf[0] = lds_frag<0>(va);
    vf[1] = lds_frag<1024>(va);
    vf[2] = lds_frag<2048>(va);
    if constexpr (NG > 4) {
      vf[3] = lds_frag<3072>(va);
      vf[4] = lds_frag<4096>(va);
      vf[5] = lds_frag<5120>(va);
      vf[6] = lds_frag<6144>(va);
    }
  };
  // the same through the compiler's own loads (the plain loop)
  auto k_frag_plain = [&](int stage_bytes, int ks) { return *reinterpret_cast<const Frag*>(smem + kaddr[ks] + stage_bytes); };
  auto v_frag_plain = [&](int stage_bytes, int g) {
    return *reinterpret_cast<const Frag*>(smem + vaddr + stage_bytes + g * 1024);
  };

  // The two key halves of a row half meet: wave kh = 1 leaves its reference, sum and O^T of row tile rt in LDS, wave
  // kh = 0 adds its own and writes the rows.  LDS must be free of other use.
  float* meet_o = reinterpret_cast<float*>(smem);            // [rh][rt][dt][r][lane]
  float* meet_ml = meet_o + 2 * 2 * DT * 16 * 64;            // [rh][rt][m, l][32 rows]
  auto leave = [&](int rt, const floatx16 (&o)[DT], float m, float l) {
    if (kh != 1) return;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
      for (int r = 0; r < 16; ++r) meet_o[(((rh * 2 + rt) * DT + dt) * 16 + r) * 64 + lane] = o[dt][r];
    if (lh == 0) {
      meet_ml[((rh * 2 + rt) * 2 + 0) * 32 + li] = m;
      meet_ml[((rh * 2 + rt) * 2 + 1) * 32 + li] = l;
    }
  };
  auto add_and_write = [&](int rt, const floatx16 (&o)[DT], float m1, float l1) {
    const int my_row = rh * 64 + rt * 32 + li;
    if (kh != 0 || my_row >= nrows) return;
    const float m2 = meet_ml[((rh * 2 + rt) * 2 + 0) * 32 + li], l2 = meet_ml[((rh * 2 + rt) * 2 + 1) * 32 + li];
    const float m = fmaxf(m1, m2);
    const float m_safe = m == -INFINITY ? 0.f : m;
    const float a1 = exp2_neg(m1 - m_safe), a2 = exp2_neg(m2 - m_safe);
    const float l = l1 * a1 + l2 * a2;
    if (parts) {  // the row over this range of keys, as a float32 row with its reference and sum
      const size_t at = part_index() + (size_t)(row0 + my_row) * H;
      if (lh == 0) {
        float* ml = parts + (size_t)n_splits * part_rows * H * d + at * 2;
        ml[0] = l > 0.f ? m : -INFINITY;
        ml[1] = l;
      }
      if (!(l > 0.f)) return;  // the row sees no key of the range
      const float inv = 1.0f / l;
      float* prow = parts + at * d;
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) {
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          floatx4 y;
#pragma unroll
          for (int r = 0; r < 4; ++r)
            y[r] = (o[dt][g * 4 + r] * a1 + meet_o[(((rh * 2 + rt) * DT + dt) * 16 + g * 4 + r) * 64 + lane] * a2) * inv;
          *reinterpret_cast<floatx4*>(prow + dt * 32 + g * 8 + lh * 4) = y;
        }
      }
      return;
    }
    const float inv = 1.0f / l;
    bf16_t* orow = out + (size_t)(row0 + my_row) * ldo + (size_t)h * d;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int e = dt * 32 + g * 8 + lh * 4;
        float y[4];
#pragma unroll
        for (int r = 0; r < 4; ++r)
          y[r] = (o[dt][g * 4 + r] * a1 + meet_o[(((rh * 2 + rt) * DT + dt) * 16 + g * 4 + r) * 64 + lane] * a2) * inv;
        uint2 pk;
        pk.x = pack_bf16x2(y[0], y[1]);
        pk.y = pack_bf16x2(y[2], y[3]);
        *reinterpret_cast<uint2*>(orow + e) = pk;
      }
    }
  };

  int& block_beyond = *reinterpret_cast<int*>(smem + LDS_BYTES);  // behind the stages
  if (tid == 0) block_beyond = 0;
  {
    floatx16 o[2][DT];  // O^T of the two row tiles: element dt*32 + (r/4)*8 + lh*4 + r%4 of row li
#pragma unroll
    for (int rt = 0; rt < 2; ++rt)
#pragma unroll
      for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int r = 0; r < 16; ++r) o[rt][dt][r] = 0.f;
    floatx16 s0, s1;     // raw scores of the two row tiles, then P
    Frag p0[2], p1[2];   // P as the second product's operands

    // ---- prologue.  Tile j's K fragments are read from LDS in slot B of pass j - 2 and its V fragments in slot B of
    // pass j - 1 (see below); the direct loads of K(j) and V(j - 1) go out in the middle of pass j - 5.
    int kpg, vpg;  // pages of the wave's keys of the tiles whose K and V the next pass loads
    {
      const int pg0 = page_of(0), pg1 = page_of(1), pg2 = page_of(2), pg3 = page_of(3);
      k_load(0, pg0);
      k_load(1, pg1);
      v_load(0, pg0);
      k_load(2, pg2);
      v_load(1, pg1);
      k_load(3, pg3);
      v_load(2, pg2);
      vpg = pg3;
      kpg = page_of(4);
    }
    __builtin_amdgcn_sched_barrier(0);
    // from here on the query rows live in accumulation registers (left to the compiler, they are copied there in every
    // pass)
#pragma unroll
    for (int rt = 0; rt < 2; ++rt)
#pragma unroll
      for (int ks = 0; ks < d / 16; ++ks) {
        asm volatile("" : "+a"(qv[rt][ks]));
        qf[rt][ks] = __builtin_bit_cast(Frag, qv[rt][ks]);
      }
    __builtin_amdgcn_sched_barrier(0);
    wait_loads_but<2 * LOADS_PER_TILE>();  // K(0), K(1), V(0)
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
    if (at_edge(0)) {
      clear_unseen(0);
      __syncthreads();
    }
    Frag kfr[NG], vfr[NG];  // the fragments of K(i + 1) and V(i) of this wave, in registers through a pass
    {  // S(0) of both row tiles and the softmax of row tile 0, one thing after the other
      Frag kf[d / 16];
#pragma unroll
      for (int ks = 0; ks < d / 16; ++ks) kf[ks] = k_frag(0, ks);
#pragma unroll
      for (int ks = 0; ks < d / 16; ++ks) {
        if (ks == 0) {
          mfma_set<0>(s0, kf[ks], qf[0][ks]);
          mfma_set<NO_WAIT>(s1, kf[ks], qf[1][ks]);
        } else {
          mfma_add<NO_WAIT>(s0, kf[ks], qf[0][ks]);
          mfma_add<NO_WAIT>(s1, kf[ks], qf[1][ks]);
        }
      }
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int g = 0; g < NG; ++g) kfr[g] = k_frag(K_STAGE, g);
      read_v_frags_but_last(vfr, lds0 + vaddr);
      asm volatile("s_nop 15\n\ts_nop 15");  // the MFMAs have left the matrix cores: their results may be read
      __builtin_amdgcn_sched_barrier(0);
      const int tk = t_begin + kh * 32;
#pragma unroll
      for (int hh = 0; hh < 16; ++hh) soft_step<true>(hh, s0, p0, st[0], tk, lh, sc2);
      {  // Row tile 1 takes its references from tile 0 now (its softmax of tile 0 comes in pass 0): with every row's
         // reference there, the passes of the short kind can begin with pass 0.
        const int base = tk + 8 * lh, first_c = st[1].lo - base, last_c = st[1].pos - base;
        float mx = -INFINITY;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int c = 16 * (r / 8) + r % 8;
          mx = fmaxf(mx, (c >= first_c && c <= last_c) ? s1[r] : -INFINITY);
        }
        st[1].m = halves_max(mx) * sc2;
      }
      __builtin_amdgcn_sched_barrier(0);
      __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0): this wave has read K(0)
      __builtin_amdgcn_s_barrier();        // every wave has: its stage may be filled again
      __builtin_amdgcn_sched_barrier(0);
      k_load(4, kpg);
      v_load(3, vpg);
      vpg = kpg;
      kpg = page_of(5);
    }

    // ---- a pass of the loop.  Before pass i: S1(i) raw in s1, P0(i) in p0, the fragments of K(i + 1) and V(i) in kfr
    // and vfr (on their way from LDS).  MASKED: some row may not see some key of tile i (row tile 1) or tile i + 1 (row
    // tile 0), or tile i + 1 has stale positions.
    auto pass = [&](auto MODE_, int i) {
      constexpr int MODE = decltype(MODE_)::value;
      constexpr bool MASKED = MODE != SOFT_SEEN;  // tiles at an edge, and the loads in one place
      constexpr int SPG = 16 / NG;                // softmax steps (of 16 a slot) beside the two MFMAs of a step
      const int t0 = t_begin + i * KT;
      __builtin_amdgcn_sched_barrier(0);
      {  // slot A: the fragments have been asked for half a pass ago
        const int tk = t0 + kh * 32;
        const int va = lds0 + vaddr + (i % STG) * V_STAGE;
#pragma unroll
        for (int g = 0; g < NG; ++g) {
#define SOFT_STEPS(G, HALF, S_, P_, ST_) /* half of the SPG softmax steps that stand beside the two MFMAs of step G */ \
  _Pragma("unroll") for (int q_ = 0; q_ < SPG / 2; ++q_)                                          \
    soft_any<MODE>(SPG * G + HALF * (SPG / 2) + q_, S_, P_, ST_, tk, lh, sc2);
#define SLOT_A_STEP(G)  /* slot B asked for K0 V0 K1 V1 .. K7 in this order (NG = 8), and V7 follows here behind the \
                           first MFMA (whose going out tells that the last MFMA of slot B has read V7's           \
                           registers): behind read n, 2 NG - 1 - n may still be out */                             \
  if constexpr (G < NG) if (g == G) {                                                             \
    if (G == 0) {                                                                                 \
      mfma_set<2 * NG - 2>(s0, kfr[G], qf[0][G]);                                                 \
      vfr[NG - 1] = lds_frag<(NG - 1) * 1024>(va);                                                \
    } else {                                                                                      \
      mfma_add<2 * NG - 1 - 2 * G>(s0, kfr[G], qf[0][G]);                                         \
    }                                                                                             \
    SOFT_STEPS(G, 0, s1, p1, st[1])                                                               \
    __builtin_amdgcn_sched_barrier(0);                                                            \
    mfma_acc<2 * NG - 2 - 2 * G>(o[0][G % DT], vfr[G], p0[G / DT]);                               \
    SOFT_STEPS(G, 1, s1, p1, st[1])                                                               \
    __builtin_amdgcn_sched_barrier(0);                                                            \
  }
          SLOT_A_STEP(0) SLOT_A_STEP(1) SLOT_A_STEP(2) SLOT_A_STEP(3)
          SLOT_A_STEP(4) SLOT_A_STEP(5) SLOT_A_STEP(6) SLOT_A_STEP(7)
#undef SLOT_A_STEP
        }
      }
      // The middle of the pass: K(i + 2) and V(i + 1), whose fragments slot B reads, are in LDS for every wave; every
      // wave has read K(i + 1) and V(i) (in slot B of the pass before), so the direct loads of K(i + 5) and V(i + 4) may
      // fill their stages.
      wait_loads_but<2 * LOADS_PER_TILE>();
      __builtin_amdgcn_s_barrier();
      __builtin_amdgcn_sched_barrier(0);
      if constexpr (MASKED) {
        if (at_edge(i + 1)) {
          clear_unseen(i + 1);
          __syncthreads();
        }
      }
      if constexpr (MASKED) {  // this kind of pass has no registers to spare for keeping the loads' operands through slot B
        kv_load_tight(i + 5, kpg, i + 4, vpg);
        vpg = kpg;
        kpg = page_of(i + 6);
        __builtin_amdgcn_sched_barrier(0);
      }
      {  // slot B; a fragment's registers take the next pass's fragment as soon as its MFMA has gone out
        const int tk = t0 + KT + kh * 32;
        const int stage_k = ((i + 2) % STG) * K_STAGE;
        const int va = lds0 + vaddr + ((i + 1) % STG) * V_STAGE;
#define SLOT_B_STEP(G)  /* a fragment's registers are free once the MFMA behind the one that read them has gone out; \
                           the direct loads of K(i + 5) and V(i + 4) go out one a step */                          \
  if constexpr (G < NG) {                                                                           \
    if (G == 0) mfma_set<NO_WAIT>(s1, kfr[G], qf[1][G]);                                            \
    else mfma_add<NO_WAIT>(s1, kfr[G], qf[1][G]);                                                   \
    if constexpr (G > 0) vfr[G - 1] = lds_frag<(G > 0 ? G - 1 : 0) * 1024>(va);                     \
    if (!MASKED && G < DT) k_load_piece(i + 5, kpg, G);                                             \
    if (!MASKED && G >= DT) v_load_piece(i + 4, vpg, G - DT);                                       \
    SOFT_STEPS(G, 0, s0, p0, st[0])                                                                 \
    __builtin_amdgcn_sched_barrier(0);                                                              \
    mfma_acc<NO_WAIT>(o[1][G % DT], vfr[G], p1[G / DT]);                                            \
    kfr[G] = k_frag(stage_k, G);                                                                    \
    if (!MASKED && G == NG - 1) {                                                                   \
      vpg = kpg;                                                                                    \
      kpg = page_of(i + 6);                                                                         \
    }                                                                                               \
    SOFT_STEPS(G, 1, s0, p0, st[0])                                                                 \
    __builtin_amdgcn_sched_barrier(0);                                                              \
  }
        SLOT_B_STEP(0) SLOT_B_STEP(1) SLOT_B_STEP(2) SLOT_B_STEP(3)
        SLOT_B_STEP(4) SLOT_B_STEP(5) SLOT_B_STEP(6) SLOT_B_STEP(7)
#undef SLOT_B_STEP
#undef SOFT_STEPS
      }
      // The last MFMAs must have left the matrix cores before O is read.  The compiler does not know these
      // instructions: it reads the accumulators right behind the loop, in front of any wait that stands there.
      if (i + 1 >= n_kt) asm volatile("s_nop 15\n\ts_nop 15");
      __builtin_amdgcn_sched_barrier(0);
    };
    // Passes in which every row sees every key of both tiles in work, and has seen a key before, run the short
    // softmax; with a window the first passes are of the other kind, under the causal mask the last ones.
    auto all_seen = [&](int i) {
      return sees_all(1, t_begin + i * KT) && sees_all(0, t_begin + (i + 1) * KT) && !at_edge(i + 1);
    };
    // Three loops one after the other, not one loop that chooses a kind of pass each time: the compiler then moved O
    // between two sets of registers in every pass.
    int i = 0;
    while (i < n_kt && !(all_seen(i) && __builtin_amdgcn_ballot_w64(st[0].m == -INFINITY || st[1].m == -INFINITY) == 0)) {
      pass(std::integral_constant<int, SOFT_MASKED>{}, i);
      ++i;
    }
    // (what the passes above saw, as one scalar: the loops below have no register to spare for the lanes' flags)
    const bool beyond_early = __builtin_amdgcn_ballot_w64((st[0].beyond | st[1].beyond) != 0) != 0;
    if (i < n_kt) {
      int i_end = i + 1;
      while (i_end < n_kt && all_seen(i_end)) ++i_end;
      st[0].sum = st[1].sum = 0.f;
      for (; i < i_end; ++i) pass(std::integral_constant<int, SOFT_SEEN>{}, i);
      st[0].l += halves_sum(st[0].sum);
      st[1].l += halves_sum(st[1].sum);
    }
    if (i < n_kt) {  // the rest: masks, but every row has its reference (the loop above began when all had)
      st[0].sum = st[1].sum = 0.f;
      for (; i < n_kt; ++i) pass(std::integral_constant<int, SOFT_LATE>{}, i);
      st[0].l += halves_sum(st[0].sum);
      st[1].l += halves_sum(st[1].sum);
    }
    // the fragments that the last pass asked for (for a pass that does not come) have arrived: their registers are free
    reads_done(kfr, vfr);
    __builtin_amdgcn_sched_barrier(0);
    // a sum this large (or no number at all) means that some P was: such a block computes its rows again below
    const bool beyond_late = __builtin_amdgcn_ballot_w64(!(st[0].l < 0x1p90f) || !(st[1].l < 0x1p90f)) != 0;

    __builtin_amdgcn_sched_barrier(0);
    wait_loads_but<0>();                    // no direct load is on its way into LDS
    __builtin_amdgcn_sched_barrier(0);
    if ((beyond_early || beyond_late) && lane == 0) block_beyond = 1;
    __syncthreads();
    if (!block_beyond) {
      leave(0, o[0], st[0].m, st[0].l);
      leave(1, o[1], st[1].m, st[1].l);
      __syncthreads();
      add_and_write(0, o[0], st[0].m, st[0].l);
      add_and_write(1, o[1], st[1].m, st[1].l);
      return;
    }
  }

  // ---- the plain loop: a score outran its row's reference somewhere in the block.  One row tile after the other,
  // one thing after the other, references that move and O shrunk by vector instructions when they do.
  // (the row tile as a constant: indexed by a variable, the query rows and the rows' state would live in memory, and
  // the loops above would keep that memory up to date)
  auto plain_rows = [&](auto RT_) {
    constexpr int rt = decltype(RT_)::value;
    floatx16 o[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
      for (int r = 0; r < 16; ++r) o[dt][r] = 0.f;
    float m_run = -INFINITY, l_run = 0.f;
    const int my_pos = st[rt].pos, my_lo = st[rt].lo;
    for (int j = 0; j < n_kt; ++j) {
      __syncthreads();  // every wave has left the stage
      const int pg = page_of(j);
      k_load(j, pg);
      v_load(j, pg);
      wait_loads_but<0>();
      __syncthreads();
      if (at_edge(j)) {
        clear_unseen(j);
        __syncthreads();
      }
      const int stage_k = (j % STG) * K_STAGE, stage_v = (j % STG) * V_STAGE;
      floatx16 s;
#pragma unroll
      for (int r = 0; r < 16; ++r) s[r] = 0.f;
#pragma unroll
      for (int ks = 0; ks < d / 16; ++ks) s = mfma32(k_frag_plain(stage_k, ks), qf[rt][ks], s);
      const int tk = t_begin + j * KT + kh * 32;
      float mx = -INFINITY;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int t = tk + 16 * (r / 8) + 8 * lh + r % 8;
        s[r] = (t >= my_lo && t <= my_pos) ? s[r] : -INFINITY;
        mx = fmaxf(mx, s[r]);
      }
      mx = halves_max(mx) * sc2;
      const float m_new = fmaxf(m_run, mx);
      const float m_safe = m_new == -INFINITY ? 0.f : m_new;
      const float alpha = exp2_neg(m_run - m_safe);
      float sum = 0.f;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        s[r] = exp2_neg(fmaf(s[r], sc2, -m_safe));
        sum += s[r];
      }
      l_run = l_run * alpha + halves_sum(sum);
      m_run = m_new;
#pragma unroll
      for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int r = 0; r < 16; ++r) o[dt][r] *= alpha;
#pragma unroll
      for (int jj = 0; jj < 2; ++jj) {
        Frag pf;
#pragma unroll
        for (int w = 0; w < 4; ++w) pf.w[w] = pack_bf16x2(s[8 * jj + 2 * w], s[8 * jj + 2 * w + 1]);
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) o[dt] = mfma32(v_frag_plain(stage_v, jj * DT + dt), pf, o[dt]);
      }
    }
    __syncthreads();
    leave(rt, o, m_run, l_run);
    __syncthreads();
    add_and_write(rt, o, m_run, l_run);
  };
  plain_rows(std::integral_constant<int, 0>{});
  plain_rows(std::integral_constant<int, 1>{});
}

// The ranges of keys of a row added up: out = sum_s w_s O_s / sum_s w_s with w_s = l_s 2^(m_s - max m).  A thread
// takes four elements of a head of a row; blockIdx.y counts the blocks of 256 threads a row needs.
__global__ __launch_bounds__(256) void attn_wide_merge_kernel(const float* __restrict__ parts, int n_splits, int part_rows,
                                                              int H, const int* __restrict__ tile_row0,
                                                              const int* __restrict__ tile_rows, bf16_t* __restrict__ out,
                                                              int ldo, int d) {
  const int tile = blockIdx.x / ATTN_WIDE_ROWS, r = blockIdx.x % ATTN_WIDE_ROWS;
  const int hq = blockIdx.y * 256 + threadIdx.x;
  if (r >= tile_rows[tile] || hq >= H * (d / 4)) return;
  const int row = tile_row0[tile] + r;
  const float* part_ml = parts + (size_t)n_splits * part_rows * H * d;
  const size_t plane = (size_t)part_rows * H;
  const int h = hq / (d / 4), e = (hq % (d / 4)) * 4;
  const size_t at = (size_t)row * H + h;
  constexpr int MOST = 8;  // ranges (the launch code refuses more)
  float ms[MOST], ls[MOST];
  floatx4 os[MOST];
  float m = -INFINITY;
#pragma unroll
  for (int s = 0; s < MOST; ++s) {
    if (s < n_splits) {
      ms[s] = part_ml[(s * plane + at) * 2];
      ls[s] = part_ml[(s * plane + at) * 2 + 1];
      os[s] = *reinterpret_cast<const floatx4*>(parts + (s * plane + at) * d + e);
      m = fmaxf(m, ms[s]);
    }
  }
  floatx4 acc = {0.f, 0.f, 0.f, 0.f};
  float sum = 0.f;
#pragma unroll
  for (int s = 0; s < MOST; ++s) {
    if (s < n_splits && ms[s] != -INFINITY) {  // (a range that the row sees no key of has left no row)
      const float w = ls[s] * exp2_neg(ms[s] - m);
      acc += w * os[s];
      sum += w;
    }
  }
  const float inv = sum > 0.f ? 1.0f / sum : 0.f;
  uint2 pk;
  pk.x = pack_bf16x2(acc[0] * inv, acc[1] * inv);
  pk.y = pack_bf16x2(acc[2] * inv, acc[3] * inv);
  *reinterpret_cast<uint2*>(out + (size_t)row * ldo + (size_t)h * d + e) = pk;
}

}  // namespace

bool attn_wide_takes(int d, int page_tokens) {
  return (d == 128 || d == 64) && page_tokens >= 16 && (page_tokens & (page_tokens - 1)) == 0;
}

int launch_attn_prefill_wide(const bf16_t* q, int ldq, int q_off, bf16_t* out, int ldo, int H, int Hk,
                             const bf16_t* cache, int page_tokens, const int* block_table, int max_blocks,
                             const int* positions, const int* row_seg, const int* tile_row0, const int* tile_rows,
                             int n_tiles, int window, float scale, int n_splits, int part_rows, float* parts,
                             int d, hipStream_t stream) {
  if (!attn_wide_takes(d, page_tokens)) return APC_ERR_UNSUPPORTED;
  if (n_splits < 1 || n_splits > 8 || (n_splits > 1 && (!parts || part_rows <= 0)) ||
      (long)n_tiles * H * n_splits > 0x7fffffffL)
    return APC_ERR_BAD_ARG;
  if (n_splits == 1) parts = nullptr;
  int lgP = 0;
  while ((1 << lgP) < page_tokens) ++lgP;
  static bool configured[64] = {};
  static std::mutex configured_lock;
  const auto kernel = d == 128 ? (window > 0 ? attn_prefill_wide_kernel<128, true> : attn_prefill_wide_kernel<128, false>)
                               : (window > 0 ? attn_prefill_wide_kernel<64, true> : attn_prefill_wide_kernel<64, false>);
  const int lds = lds_request(d);
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return (int)e;
  if (dev < 0 || dev >= 64) return APC_ERR_UNSUPPORTED;
  {  // more LDS than a kernel gets without asking: once per device
    std::lock_guard<std::mutex> hold(configured_lock);
    if (!configured[dev]) {
      const std::pair<const void*, int> instances[] = {
          {(const void*)attn_prefill_wide_kernel<128, true>, 128}, {(const void*)attn_prefill_wide_kernel<128, false>, 128},
          {(const void*)attn_prefill_wide_kernel<64, true>, 64}, {(const void*)attn_prefill_wide_kernel<64, false>, 64}};
      for (const auto& [f, hd] : instances) {
        e = hipFuncSetAttribute(f, hipFuncAttributeMaxDynamicSharedMemorySize, lds_request(hd));
        if (e != hipSuccess) return (int)e;
      }
      configured[dev] = true;
    }
  }
  hipLaunchKernelGGL(kernel, dim3(n_tiles * H * n_splits), dim3(256), lds, stream, q, ldq,
                     q_off, out, ldo, H, Hk, cache, lgP, block_table, max_blocks, positions, row_seg, tile_row0, tile_rows,
                     n_tiles, window, scale, n_splits, part_rows, parts);
  APC_LAUNCH_CHECK();
  if (n_splits > 1) {
    hipLaunchKernelGGL(attn_wide_merge_kernel, dim3(n_tiles * ATTN_WIDE_ROWS, ceil_div(H * (d / 4), 256)),
                       dim3(256), 0, stream, parts, n_splits,
                       part_rows, H, tile_row0, tile_rows, out, ldo, d);
    APC_LAUNCH_CHECK();
  }
  return 0;
}
