// Attention over the paged cache in bfloat16 on MFMA, float32 softmax.
//
//   prefill kernel   a tile of up to 64 consecutive rows of one request x one head; keys in tiles of 64
//                    through LDS; S = Q K^T and O += P V on v_mfma_f32_16x16x32_bf16; online softmax.
//   decode kernel    one row x one kv head (the H/Hk query heads of the group are the 16 rows of the MFMA
//                    tile, so keys and values are read once per group); each wave is a "part" that covers
//                    KW consecutive keys straight from global memory; parts are merged by a second kernel
//                    in key order.
// Cache pages: keys [kv_head][slot][d] (d contiguous), values [kv_head][d][slot] (slots contiguous): both
// MFMA operands want the summed axis contiguous per lane, d for the scores and positions for the values.
// Masking: a row at position p sees keys max(0, p - window + 1) .. p.  Scores are scaled on the finished
// dot product; softmax maxima, sums and exponentials are float32; P is rounded to bfloat16 for the
// value product (as every activation between two matrix products is in this path).
// Formula: crates/allpaca-cpu/src/kernels.rs:293-356.  Reference kernels (contiguous K/V, no matrix
// cores): attention_qtile_kernel hip/src/kernels.cpp:2203, attention_split_gqa_kernel 2276, merges 2479-2516.
#include "mfma.h"
#include <math.h>

constexpr int KT = 64;            // keys per tile in the prefill kernel
constexpr int QT = 64;            // rows per tile in the prefill kernel
constexpr int KPAD = 8;

__device__ __forceinline__ float group16_max(float v) {  // over the 16 lanes that share lane/16
#pragma unroll
  for (int o = 8; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, WAVE));
  return v;
}
__device__ __forceinline__ float group16_sum(float v) {
#pragma unroll
  for (int o = 8; o > 0; o >>= 1) v += __shfl_xor(v, o, WAVE);
  return v;
}

// ------------------------------------------------------------------------------------------ prefill
template <int DP>  // head_dim rounded up to a multiple of 32
__global__ __launch_bounds__(256) void attn_prefill_kernel(
    const bf16_t* __restrict__ q, int ldq, int q_off, bf16_t* __restrict__ out, int ldo, int H, int Hk, int d,
    const bf16_t* __restrict__ cache, int P, const int* __restrict__ block_table, int max_blocks,
    const int* __restrict__ positions, const int* __restrict__ row_seg, const int* __restrict__ tile_row0,
    const int* __restrict__ tile_rows, int window, float scale) {
  __shared__ __attribute__((aligned(16))) bf16_t Ks[KT * (DP + KPAD)];
  __shared__ __attribute__((aligned(16))) bf16_t Vs[DP * (KT + KPAD)];
  __shared__ __attribute__((aligned(16))) bf16_t Ps[4 * 16 * (KT + KPAD)];
  const int tid = threadIdx.x, lane = tid % WAVE, wave = tid / WAVE;
  const int li = lane % 16, lc = lane / 16;
  const int tile = blockIdx.x, h = blockIdx.y;
  const int row0 = tile_row0[tile], nrows = tile_rows[tile];
  const int kvh = h / (H / Hk);
  const int pos0 = positions[row0];
  const int* bt = block_table + (size_t)row_seg[row0] * max_blocks;
  const int last = pos0 + nrows - 1;
  const int first = (window > 0 && pos0 - window + 1 > 0) ? pos0 - window + 1 : 0;
  const size_t page_stride = (size_t)2 * Hk * P * d;
  const size_t head_off = (size_t)kvh * P * d, v_off = (size_t)Hk * P * d;
  const int dchunks = d / 8;

  // the padding columns of K stay zero for the whole kernel (a padded q column is zero as well, but 0 * NaN is NaN)
  for (int idx = tid; idx < KT * (DP + KPAD); idx += 256) Ks[idx] = 0;

  // this wave's 16 query rows as A operands
  Frag qf[DP / 32];
  {
    const int r = wave * 16 + li;
    const bf16_t* qrow = q + (size_t)(row0 + min(r, nrows - 1)) * ldq + q_off + (size_t)h * d;
#pragma unroll
    for (int ks = 0; ks < DP / 32; ++ks) {
      const int e = ks * 32 + lc * 8;
      qf[ks] = (r < nrows && e < d) ? load_frag(qrow + e) : zero_frag();
    }
  }
  floatx4 o[DP / 16];
#pragma unroll
  for (int dt = 0; dt < DP / 16; ++dt) o[dt] = floatx4{0.f, 0.f, 0.f, 0.f};
  float mrow[4], lrow[4];
#pragma unroll
  for (int r = 0; r < 4; ++r) { mrow[r] = -INFINITY; lrow[r] = 0.f; }
  bf16_t* pw = Ps + wave * 16 * (KT + KPAD);

  for (int t0 = (first / KT) * KT; t0 <= last; t0 += KT) {
    __syncthreads();  // the previous tile's K, V and P are no longer read
    // K tile: 64 keys x d, 16-byte chunks along d
    for (int idx = tid; idx < KT * dchunks; idx += 256) {
      const int key = idx / dchunks, ch = idx % dchunks;
      const int t = t0 + key;
      Frag f = zero_frag();
      if (t <= last) {
        const int page = bt[t / P];
        f = load_frag(cache + (size_t)page * page_stride + head_off + (size_t)(t % P) * d + ch * 8);
      }
      *reinterpret_cast<Frag*>(&Ks[key * (DP + KPAD) + ch * 8]) = f;
    }
    // V tile, stored [d][key]: chunks of 8 consecutive positions of one element
    for (int idx = tid; idx < d * (KT / 8); idx += 256) {
      const int dv = idx / (KT / 8), kc = idx % (KT / 8);
      const int t = t0 + kc * 8;
      Frag f = zero_frag();
      if (t <= last) {
        const int page = bt[t / P];
        f = load_frag(cache + (size_t)page * page_stride + v_off + head_off + (size_t)dv * P + (t % P));
      }
      *reinterpret_cast<Frag*>(&Vs[dv * (KT + KPAD) + kc * 8]) = f;
    }
    __syncthreads();

    // scores of this wave's 16 rows against the 64 keys
    floatx4 s[KT / 16];
#pragma unroll
    for (int nt = 0; nt < KT / 16; ++nt) {
      s[nt] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ks = 0; ks < DP / 32; ++ks) {
        const Frag kf = *reinterpret_cast<const Frag*>(&Ks[(nt * 16 + li) * (DP + KPAD) + ks * 32 + lc * 8]);
        s[nt] = mfma16(qf[ks], kf, s[nt]);
      }
    }
    // lane holds rows lc*4 + r and key nt*16 + li
    float alpha[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int pos = pos0 + wave * 16 + lc * 4 + r;
      const int lo = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
      float mx = -INFINITY;
#pragma unroll
      for (int nt = 0; nt < KT / 16; ++nt) {
        const int t = t0 + nt * 16 + li;
        const float v = (t >= lo && t <= pos) ? s[nt][r] * scale : -INFINITY;
        s[nt][r] = v;
        mx = fmaxf(mx, v);
      }
      mx = group16_max(mx);
      const float m_new = fmaxf(mrow[r], mx);
      const float m_safe = m_new == -INFINITY ? 0.f : m_new;
      alpha[r] = __expf(mrow[r] - m_safe);
      float sum = 0.f;
#pragma unroll
      for (int nt = 0; nt < KT / 16; ++nt) {
        const float p = __expf(s[nt][r] - m_safe);
        s[nt][r] = p;
        sum += p;
      }
      lrow[r] = lrow[r] * alpha[r] + group16_sum(sum);
      mrow[r] = m_new;
    }
#pragma unroll
    for (int dt = 0; dt < DP / 16; ++dt)
#pragma unroll
      for (int r = 0; r < 4; ++r) o[dt][r] *= alpha[r];
    // P through LDS into the A operand layout
#pragma unroll
    for (int nt = 0; nt < KT / 16; ++nt)
#pragma unroll
      for (int r = 0; r < 4; ++r) pw[(lc * 4 + r) * (KT + KPAD) + nt * 16 + li] = float_to_bf16(s[nt][r]);
    __syncthreads();
#pragma unroll
    for (int kstep = 0; kstep < KT / 32; ++kstep) {
      const Frag pf = *reinterpret_cast<const Frag*>(&pw[li * (KT + KPAD) + kstep * 32 + lc * 8]);
#pragma unroll
      for (int dt = 0; dt < DP / 16; ++dt) {
        const Frag vf = *reinterpret_cast<const Frag*>(&Vs[(dt * 16 + li) * (KT + KPAD) + kstep * 32 + lc * 8]);
        o[dt] = mfma16(pf, vf, o[dt]);
      }
    }
  }
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const int row = wave * 16 + lc * 4 + r;
    if (row >= nrows) continue;
    const float inv = 1.0f / lrow[r];
    bf16_t* orow = out + (size_t)(row0 + row) * ldo + (size_t)h * d;
#pragma unroll
    for (int dt = 0; dt < DP / 16; ++dt) {
      const int e = dt * 16 + li;
      if (e < d) orow[e] = float_to_bf16(o[dt][r] * inv);
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

template <int DP>
__global__ __launch_bounds__(256) void attn_decode_kernel(
    const bf16_t* __restrict__ q, int ldq, int q_off, int H, int Hk, int d, const bf16_t* __restrict__ cache, int P,
    const int* __restrict__ block_table, int max_blocks, const int* __restrict__ positions,
    const int* __restrict__ row_seg, const int* __restrict__ rows, int window, float scale, int KW, int n_parts,
    float* __restrict__ parts) {
  __shared__ __attribute__((aligned(16))) bf16_t Ps[4 * 16 * (32 + KPAD)];
  const int lane = threadIdx.x % WAVE, wave = threadIdx.x / WAVE;
  const int li = lane % 16, lc = lane / 16;
  const int G = H / Hk, gtiles = (G + 15) / 16;
  const int ri = blockIdx.x;
  const int row = rows ? rows[ri] : ri;
  const int kvh = blockIdx.y / gtiles, gt = blockIdx.y % gtiles;
  const int part = blockIdx.z * 4 + wave;
  const int pos = positions[row];
  const int first = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
  const int k_lo = max(part * KW, (first / 32) * 32), k_hi = min((part + 1) * KW, pos + 1);
  if (part >= n_parts || k_lo >= k_hi) return;  // nothing to see for this part (whole wave leaves together)
  const int* bt = block_table + (size_t)row_seg[row] * max_blocks;
  const size_t page_stride = (size_t)2 * Hk * P * d;
  const size_t head_off = (size_t)kvh * P * d, v_off = (size_t)Hk * P * d;
  // the page ids of this wave's range of keys, one per lane, fetched once: the loads of keys and values then
  // do not wait for a look-up in the block table (a range of KW keys spans at most 64 pages: checked by the host)
  const int page0 = k_lo / P;
  const int my_page = bt[min(page0 + lane, pos / P)];

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
  float mrow[4], lrow[4];
#pragma unroll
  for (int r = 0; r < 4; ++r) { mrow[r] = -INFINITY; lrow[r] = 0.f; }
  bf16_t* pw = Ps + wave * 16 * (32 + KPAD);

  // Operands of 32 keys straight from the pages.  Nothing is loaded conditionally: a key beyond the row's own
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
        r.k[nt][ks] = load_frag(krow + (e < d ? e : 0));
      }
    }
    const int tv = min(kb + lc * 8, (pos / 8) * 8);
    const int vpage = __shfl(my_page, tv / P - page0, WAVE);
    const bf16_t* vbase = cache + (size_t)vpage * page_stride + v_off + head_off + (tv % P);
#pragma unroll
    for (int dt = 0; dt < DP / 16; ++dt) r.v[dt] = load_frag(vbase + (size_t)min(dt * 16 + li, d - 1) * P);
  };

  auto step = [&](const KVRegs<DP>& r, int kb) {
    floatx4 s[2];
#pragma unroll
    for (int nt = 0; nt < 2; ++nt) {
      s[nt] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ks = 0; ks < DP / 32; ++ks) s[nt] = mfma16(qf[ks], r.k[nt][ks], s[nt]);
    }
    float alpha[4];
#pragma unroll
    for (int rr = 0; rr < 4; ++rr) {
      float mx = -INFINITY;
#pragma unroll
      for (int nt = 0; nt < 2; ++nt) {
        const int t = kb + nt * 16 + li;
        const float v = (t >= first && t <= pos) ? s[nt][rr] * scale : -INFINITY;
        s[nt][rr] = v;
        mx = fmaxf(mx, v);
      }
      mx = group16_max(mx);
      const float m_new = fmaxf(mrow[rr], mx);
      const float m_safe = m_new == -INFINITY ? 0.f : m_new;
      alpha[rr] = __expf(mrow[rr] - m_safe);
      const float p0 = __expf(s[0][rr] - m_safe), p1 = __expf(s[1][rr] - m_safe);
      s[0][rr] = p0;
      s[1][rr] = p1;
      lrow[rr] = lrow[rr] * alpha[rr] + group16_sum(p0 + p1);
      mrow[rr] = m_new;
    }
#pragma unroll
    for (int dt = 0; dt < DP / 16; ++dt)
#pragma unroll
      for (int rr = 0; rr < 4; ++rr) o[dt][rr] *= alpha[rr];
    // P through this wave's LDS rows into the A operand layout
#pragma unroll
    for (int nt = 0; nt < 2; ++nt)
#pragma unroll
      for (int rr = 0; rr < 4; ++rr) pw[(lc * 4 + rr) * (32 + KPAD) + nt * 16 + li] = float_to_bf16(s[nt][rr]);
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    const Frag pf = *reinterpret_cast<const Frag*>(&pw[li * (32 + KPAD) + lc * 8]);
#pragma unroll
    for (int dt = 0; dt < DP / 16; ++dt) o[dt] = mfma16(pf, r.v[dt], o[dt]);
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
  };

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

  // this part's result for the heads of the group
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const int g = gt * 16 + lc * 4 + r;
    if (g >= G) continue;
    float* dst = parts + (((size_t)ri * H + (kvh * G + g)) * n_parts + part) * (d + 2);
#pragma unroll
    for (int dt = 0; dt < DP / 16; ++dt) {
      const int e = dt * 16 + li;
      if (e < d) dst[e] = o[dt][r];
    }
    if (li == 0) { dst[d] = mrow[r]; dst[d + 1] = lrow[r]; }
  }
}

// merge of the parts of one (row, head), in key order: first the weights of all parts (their maxima against
// the overall maximum), then the weighted sum of their outputs with independent loads
constexpr int MERGE_NT = 128;
__global__ __launch_bounds__(MERGE_NT) void attn_merge_kernel(const float* __restrict__ parts, int n_parts, int KW,
                                                              int H, int d, const int* __restrict__ positions,
                                                              const int* __restrict__ rows, int window,
                                                              bf16_t* __restrict__ out, int ldo) {
  extern __shared__ float wgt[];  // [n_parts] weights, then 1 float: 1 / l
  const int ri = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
  const int row = rows ? rows[ri] : ri;
  const int pos = positions[row];
  const int first = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
  const int p_lo = ((first / 32) * 32) / KW, p_hi = min(pos / KW, n_parts - 1);  // parts with a visible key
  const int np = p_hi - p_lo + 1;
  const float* base = parts + (((size_t)ri * H + h) * n_parts + p_lo) * (d + 2);
  for (int p = tid; p < np; p += MERGE_NT) wgt[p] = base[(size_t)p * (d + 2) + d];  // the parts' maxima
  __syncthreads();
  float m = -INFINITY;
  for (int p = 0; p < np; ++p) m = fmaxf(m, wgt[p]);
  __syncthreads();
  for (int p = tid; p < np; p += MERGE_NT) {
    const float pm = wgt[p];
    wgt[p] = pm == -INFINITY ? 0.f : __expf(pm - m);
  }
  __syncthreads();
  if (tid == 0) {
    float l = 0.f;
    for (int p = 0; p < np; ++p) l += base[(size_t)p * (d + 2) + d + 1] * wgt[p];
    wgt[np] = 1.0f / l;
  }
  __syncthreads();
  const float inv = wgt[np];
  for (int e = tid; e < d; e += MERGE_NT) {
    float acc = 0.f;
#pragma unroll 8
    for (int p = 0; p < np; ++p) acc = fmaf(base[(size_t)p * (d + 2) + e], wgt[p], acc);
    out[(size_t)row * ldo + (size_t)h * d + e] = float_to_bf16(acc * inv);
  }
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
                                          const int* tile_rows, int n_tiles, int window, float scale,
                                          hipStream_t stream) {
  if (n_tiles <= 0) return 0;
  int e = check_common(q, ldq, q_off, cache, H, Hk, d, page_tokens);
  if (e) return e;
  if (H > 65535 || max_blocks <= 0 || window < 0) return APC_ERR_BAD_ARG;
  dim3 grid(n_tiles, H), block(256);
#define PF_LAUNCH(DP_)                                                                                             \
  hipLaunchKernelGGL((attn_prefill_kernel<DP_>), grid, block, 0, stream, (const bf16_t*)q, ldq, q_off, (bf16_t*)out, \
                     ldo, H, Hk, d, (const bf16_t*)cache, page_tokens, block_table, max_blocks, positions, row_seg,  \
                     tile_row0, tile_rows, window, scale)
  if (d <= 32) PF_LAUNCH(32);
  else if (d <= 64) PF_LAUNCH(64);
  else if (d <= 96) PF_LAUNCH(96);
  else if (d <= 128) PF_LAUNCH(128);
  else if (d <= 192) PF_LAUNCH(192);
  else PF_LAUNCH(256);
#undef PF_LAUNCH
  APC_LAUNCH_CHECK();
  return 0;
}

// workspace: n_rows * H * n_parts * (d + 2) floats
APC_EXPORT int apc_attention_decode_bf16(const void* q, int ldq, int q_off, void* out, int ldo, int n_rows, int H,
                                         int Hk, int d, const void* cache, int page_tokens, const int* block_table,
                                         int max_blocks, const int* positions, const int* row_seg, const int* rows,
                                         int window, float scale, int keys_per_part, int n_parts, float* workspace,
                                         hipStream_t stream) {
  if (n_rows <= 0) return 0;
  int e = check_common(q, ldq, q_off, cache, H, Hk, d, page_tokens);
  if (e) return e;
  if (keys_per_part <= 0 || keys_per_part % 32 || n_parts <= 0 || !workspace || max_blocks <= 0 || window < 0)
    return APC_ERR_BAD_ARG;
  if (keys_per_part / page_tokens + 2 > 64) return APC_ERR_BAD_ARG;  // a wave keeps one page id per lane
  const int G = H / Hk, gtiles = (G + 15) / 16;
  if (Hk * gtiles > 65535 || (n_parts + 3) / 4 > 65535 || H > 65535) return APC_ERR_BAD_ARG;
  dim3 grid(n_rows, Hk * gtiles, (n_parts + 3) / 4), block(256);
#define DC_LAUNCH(DP_)                                                                                            \
  hipLaunchKernelGGL((attn_decode_kernel<DP_>), grid, block, 0, stream, (const bf16_t*)q, ldq, q_off, H, Hk, d,   \
                     (const bf16_t*)cache, page_tokens, block_table, max_blocks, positions, row_seg, rows, window, \
                     scale, keys_per_part, n_parts, workspace)
  if (d <= 32) DC_LAUNCH(32);
  else if (d <= 64) DC_LAUNCH(64);
  else if (d <= 96) DC_LAUNCH(96);
  else if (d <= 128) DC_LAUNCH(128);
  else if (d <= 192) DC_LAUNCH(192);
  else DC_LAUNCH(256);
#undef DC_LAUNCH
  APC_LAUNCH_CHECK();
  hipLaunchKernelGGL(attn_merge_kernel, dim3(n_rows, H), dim3(MERGE_NT), (n_parts + 1) * sizeof(float), stream,
                     workspace, n_parts, keys_per_part, H, d, positions, rows, window, (bf16_t*)out, ldo);
  APC_LAUNCH_CHECK();
  return 0;
}
