// Rotation of q and k and the write of k and v into the paged cache, bfloat16 rows and cache, 16 bytes a lane.
//
// The same operation as rope_kv_write_kernel in plain_ops.hip (pairs (i, i + rot/2) of a head turn by the
// row's position, angles from cos_sin[pos][2][rot/2] in float32; k goes to cache[page][0][kv_head][slot][:], v to
// cache[page][1][kv_head][:][slot]), for the sizes of the MFMA path: head size a multiple of 8, rotated width a
// multiple of 16 (so a lane's 8 elements and their 8 partners are whole 16-byte pieces), 16-byte aligned rows.
// A block of 256 threads takes one row (token): 8 elements of one head a lane, so 8 lanes turn one head of 128;
// values are read 16 bytes a lane and scattered, one element per slot column of the transposed page.
// Formula: crates/allpaca-cpu/src/kernels.rs:676-682; cache position page = pos / P, slot = pos % P:
// crates/allpaca-core/src/model.rs:10439-10443.
#include "mfma.h"

__global__ __launch_bounds__(256) void rope_kv_write_bf16_kernel(
    bf16_t* __restrict__ qkv, int ld, int q_off, int k_off, int v_off, int H, int Hk, int d, int rot,
    const float* __restrict__ cos_sin, const int* __restrict__ positions, const int* __restrict__ row_seg,
    const int* __restrict__ block_table, int max_blocks, bf16_t* __restrict__ cache, int P) {
  const int t = blockIdx.x;
  const int pos = positions[t];
  const int half = rot / 2, pieces = d / 8;          // 16-byte pieces of a head
  const int turn = half / 8;                          // pieces of a head that have a partner above them
  bf16_t* row = qkv + (size_t)t * ld;
  const float* cs = cos_sin + (size_t)pos * rot;      // [2][half]
  bf16_t* page = nullptr;
  int slot = 0;
  if (cache) {
    page = cache + (size_t)block_table[(size_t)row_seg[t] * max_blocks + pos / P] * ((size_t)2 * Hk * P * d);
    slot = pos % P;
  }
  // q and k heads: a work item is (head, piece of the first half of the rotated width) or (head, piece beyond it)
  const int per_head = turn + (pieces - 2 * turn);    // items of one head
  const int n_items = (H + Hk) * per_head;
  for (int item = threadIdx.x; item < n_items; item += 256) {
    const int head = item / per_head, j = item % per_head;
    const bool is_k = head >= H;
    bf16_t* x = row + (is_k ? k_off + (size_t)(head - H) * d : q_off + (size_t)head * d);
    bf16_t* dst = is_k ? (page ? page + ((size_t)(head - H) * P + slot) * d : x) : x;
    if (j < turn) {
      const int e = j * 8;
      const Frag a = load_frag(x + e), b = load_frag(x + e + half);
      const floatx4 c0 = *reinterpret_cast<const floatx4*>(cs + e), c1 = *reinterpret_cast<const floatx4*>(cs + e + 4);
      const floatx4 s0 = *reinterpret_cast<const floatx4*>(cs + half + e);
      const floatx4 s1 = *reinterpret_cast<const floatx4*>(cs + half + e + 4);
      Frag lo, hi;
#pragma unroll
      for (int w = 0; w < 4; ++w) {
        float ya[2], yb[2];
#pragma unroll
        for (int h = 0; h < 2; ++h) {
          const float av = bf16_to_float((bf16_t)(a.w[w] >> (16 * h))), bv = bf16_to_float((bf16_t)(b.w[w] >> (16 * h)));
          const int i = 2 * w + h;
          const float c = i < 4 ? c0[i % 4] : c1[i % 4], sn = i < 4 ? s0[i % 4] : s1[i % 4];
          ya[h] = av * c - bv * sn;
          yb[h] = av * sn + bv * c;
        }
        lo.w[w] = pack_bf16x2(ya[0], ya[1]);
        hi.w[w] = pack_bf16x2(yb[0], yb[1]);
      }
      *reinterpret_cast<Frag*>(dst + e) = lo;
      *reinterpret_cast<Frag*>(dst + e + half) = hi;
    } else if (is_k && page) {  // beyond the rotated width: k is copied into the cache, q stays where it is
      const int e = rot + (j - turn) * 8;
      *reinterpret_cast<Frag*>(dst + e) = load_frag(x + e);
    }
  }
  // v: 8 elements a lane, each into its own column of the transposed page
  if (page) {
    const int n_v = Hk * pieces;
    bf16_t* vpage = page + (size_t)Hk * P * d;
    for (int item = threadIdx.x; item < n_v; item += 256) {
      const int head = item / pieces, e = (item % pieces) * 8;
      const Frag v = load_frag(row + v_off + (size_t)head * d + e);
      bf16_t* col = vpage + ((size_t)head * d + e) * P + slot;
#pragma unroll
      for (int w = 0; w < 4; ++w) {
        col[(size_t)(2 * w) * P] = (bf16_t)(v.w[w] & 0xffffu);
        col[(size_t)(2 * w + 1) * P] = (bf16_t)(v.w[w] >> 16);
      }
    }
  }
}

APC_EXPORT int apc_rope_kv_write_bf16(void* qkv, int ld, int q_off, int k_off, int v_off, int n_tok, int H, int Hk,
                                      int d, int rot, const float* cos_sin, const int* positions, const int* row_seg,
                                      const int* block_table, int max_blocks, void* cache, int page_tokens,
                                      hipStream_t stream) {
  if (n_tok <= 0) return 0;
  if (H < 0 || Hk < 0 || H + Hk == 0 || d <= 0 || rot < 0 || rot > d || (rot > 0 && !cos_sin) || !positions)
    return APC_ERR_BAD_ARG;
  if (cache && (page_tokens <= 0 || !block_table || !row_seg || max_blocks <= 0)) return APC_ERR_BAD_ARG;
  if (d % 8 || rot % 16 || ld % 8 || q_off % 8 || k_off % 8 || v_off % 8 || ((uintptr_t)qkv & 15u) ||
      ((uintptr_t)cache & 15u) || ((uintptr_t)cos_sin & 15u))
    return APC_ERR_UNSUPPORTED;
  hipLaunchKernelGGL(rope_kv_write_bf16_kernel, dim3(n_tok), dim3(256), 0, stream, (bf16_t*)qkv, ld, q_off, k_off, v_off,
                     H, Hk, d, rot, cos_sin, positions, row_seg, block_table, max_blocks, (bf16_t*)cache, page_tokens);
  APC_LAUNCH_CHECK();
  return 0;
}
