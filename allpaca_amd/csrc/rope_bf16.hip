// Rotation of q and k and the write of k and v into the paged cache, bfloat16 rows and cache, 16 bytes a lane.
//
// The same operation as rope_kv_write_kernel in plain_ops.hip (pairs (i, i + rot/2) of a head turn by the
// row's position, angles from cos_sin[pos][2][rot/2] in float32; k goes to cache[page][0][kv_head][slot][:], v to
// cache[page][1][kv_head][:][slot]), for the sizes of the MFMA path: head size a multiple of 8, rotated width a
// multiple of 16 (so a lane's 8 elements and their 8 partners are whole 16-byte pieces), 16-byte aligned rows.
// A block of 256 threads takes one row (token): 8 elements of one head a lane, so 8 lanes turn one head of 128.
// The values go into a transposed page, where a token owns one 2-byte slot of every column, so blocks of a second
// kind, in front of the others in the grid, take 16 consecutive rows x 512 columns each: the rows' values meet in LDS, and 8 rows that are 8 consecutive
// slots of one page from a slot that is a multiple of 8 on (the rows of a prompt portion) leave as one 16-byte store a
// column; rows that are not (decoded rows of different requests, a portion that starts elsewhere) leave slot by slot.
// 2,048 tokens of 8 kv heads of 128, pages of 16: 11 us, of which the rotation is 8.5 (22 us with every value stored
// by itself).
// Formula: crates/allpaca-cpu/src/kernels.rs:676-682; cache position page = pos / P, slot = pos % P:
// crates/allpaca-core/src/model.rs:10439-10443.
#include "mfma.h"

constexpr int V_ROWS = 16;     // rows a block of the second kind takes
constexpr int V_COLS = 512;    // columns (kv head, element) it has in LDS at a time (16.5 KiB: the blocks of the first kind keep their 8 a unit)
constexpr int V_PAD = 8;       // elements between the rows in LDS: a row starts on 16 bytes, rows 8 apart on other banks

// v of rows r0 .. r0 + 15, columns c0 .. c0 + V_COLS - 1 (kv head * d + element), into the transposed pages
__device__ __forceinline__ void write_values(const bf16_t* __restrict__ qkv, int ld, int v_off, int Hk, int d,
                                             const int* __restrict__ positions, const int* __restrict__ row_seg,
                                             const int* __restrict__ block_table, int max_blocks,
                                             bf16_t* __restrict__ cache, int P, int n_tok, int r0, int c0) {
  __shared__ __attribute__((aligned(16))) bf16_t vt[V_ROWS][V_COLS + V_PAD];
  __shared__ long long v_base[V_ROWS];  // element offset of the row's page's values; -1: no such row
  __shared__ int v_slot[V_ROWS];
  const int tid = threadIdx.x;
  if (tid < V_ROWS) {
    const int t = r0 + tid;
    long long base = -1;
    int slot = 0;
    if (t < n_tok) {
      const int pos = positions[t];
      const long long page = block_table[(size_t)row_seg[t] * max_blocks + pos / P];
      base = page * ((long long)2 * Hk * P * d) + (long long)Hk * P * d;
      slot = pos % P;
    }
    v_base[tid] = base;
    v_slot[tid] = slot;
  }
  __syncthreads();
  // the half (8 rows) this thread stores: one piece of 16 bytes a column, or slot by slot
  const int h = tid % 2;
  bool run = P % 8 == 0 && v_slot[8 * h] % 8 == 0;
#pragma unroll
  for (int r = 0; r < 8; ++r)
    run = run && v_base[8 * h + r] >= 0 && v_base[8 * h + r] == v_base[8 * h] && v_slot[8 * h + r] == v_slot[8 * h] + r;
  const int cw = min(V_COLS, Hk * d - c0), pieces = cw / 8;
  for (int item = tid; item < V_ROWS * pieces; item += 256) {
    const int r = item / pieces, p = item % pieces;
    if (r0 + r < n_tok)
      *reinterpret_cast<Frag*>(&vt[r][p * 8]) = load_frag(qkv + (size_t)(r0 + r) * ld + v_off + c0 + p * 8);
  }
  __syncthreads();
  for (int item = tid; item < 2 * cw; item += 256) {  // item % 2 == h: 256 is even
    const int col = item / 2;
    const size_t at = (size_t)(c0 + col) * P;
    if (run) {
      Frag f;
#pragma unroll
      for (int w = 0; w < 4; ++w)
        f.w[w] = (uint32_t)vt[8 * h + 2 * w][col] | ((uint32_t)vt[8 * h + 2 * w + 1][col] << 16);
      *reinterpret_cast<Frag*>(cache + v_base[8 * h] + at + v_slot[8 * h]) = f;
    } else {
#pragma unroll
      for (int r = 0; r < 8; ++r)
        if (v_base[8 * h + r] >= 0) cache[v_base[8 * h + r] + at + v_slot[8 * h + r]] = vt[8 * h + r][col];
    }
  }
}

__global__ __launch_bounds__(256) void rope_kv_write_bf16_kernel(
    bf16_t* __restrict__ qkv, int ld, int q_off, int k_off, int v_off, int H, int Hk, int d, int rot,
    const float* __restrict__ cos_sin, const int* __restrict__ positions, const int* __restrict__ row_seg,
    const int* __restrict__ block_table, int max_blocks, bf16_t* __restrict__ cache, int P, int n_tok,
    int v_blocks) {
  if ((int)blockIdx.x < v_blocks) {  // the blocks for the values go first: they are fewer and each has more to do
    const int chunks = ceil_div(Hk * d, V_COLS);
    write_values(qkv, ld, v_off, Hk, d, positions, row_seg, block_table, max_blocks, cache, P, n_tok,
                 ((int)blockIdx.x / chunks) * V_ROWS, ((int)blockIdx.x % chunks) * V_COLS);
    return;
  }
  const int t = (int)blockIdx.x - v_blocks;
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
  const int v_blocks = cache ? ceil_div(n_tok, V_ROWS) * ceil_div(Hk * d, V_COLS) : 0;
  hipLaunchKernelGGL(rope_kv_write_bf16_kernel, dim3(n_tok + v_blocks), dim3(256), 0, stream, (bf16_t*)qkv, ld, q_off, k_off,
                     v_off, H, Hk, d, rot, cos_sin, positions, row_seg, block_table, max_blocks, (bf16_t*)cache, page_tokens,
                     n_tok, v_blocks);
  APC_LAUNCH_CHECK();
  return 0;
}
