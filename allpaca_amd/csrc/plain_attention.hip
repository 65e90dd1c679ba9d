// Plain attention over the paged cache: one wave per (query row, head), keys in
// order in chunks of 64 anchored at key 0, online softmax in float32.
//
// For the row at position `pos` of its request:  keys t in [first, pos],
// first = 0 or pos - window + 1;  s_t = (q . K[t]) * scale;  m = max s;
// p_t = exp(s_t - m);  out = sum p_t V[t] / sum p_t;  query head h reads kv head
// h / (H/Hk).  Reference: crates/allpaca-cpu/src/kernels.rs:293-356 (the causal
// rule `t <= qi + (n_kv - n_q)` is `t <= pos` once rows carry their position);
// the chunked online form follows hip/src/kernels.cpp:1917-1934 in spirit: the
// order of additions for a row is fixed by its position alone, never by what
// else is in the batch or how the prompt was cut.
//
// keys cache[page][0][kv_head][slot][i], values cache[page][1][kv_head][i][slot];
// page = block_table[seg][t / P], slot = t % P.
#include "common.h"
#include <math.h>

constexpr int MAX_D_PER_LANE = 4;  // head_dim <= 256

__global__ __launch_bounds__(64) void paged_attention_plain_kernel(
    const void* __restrict__ q, int q_dtype, int ldq, int q_off, void* __restrict__ out, int out_dtype, int ldo, int H,
    int Hk, int d, const void* __restrict__ cache, int cache_dtype, int P, const int* __restrict__ block_table,
    int max_blocks, const int* __restrict__ positions, const int* __restrict__ row_seg, int window, float scale) {
  __shared__ float qs[MAX_D_PER_LANE * WAVE];
  __shared__ float ps[WAVE];
  const int r = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const int kvh = h / (H / Hk);
  const int pos = positions[r];
  const int* bt = block_table + (size_t)row_seg[r] * max_blocks;
  const int first = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;

  for (int i = lane; i < d; i += WAVE) qs[i] = load_f(q, q_dtype, (size_t)r * ldq + q_off + (size_t)h * d + i);
  __syncthreads();

  float o[MAX_D_PER_LANE];
#pragma unroll
  for (int i = 0; i < MAX_D_PER_LANE; ++i) o[i] = 0.f;
  float m = -INFINITY, l = 0.f;

  for (int c = first / WAVE; c <= pos / WAVE; ++c) {
    const int t = c * WAVE + lane;
    const bool valid = t >= first && t <= pos;
    float s = -INFINITY;
    if (valid) {
      const int page = bt[t / P];
      const size_t kb = ((((size_t)page * 2 + 0) * Hk + kvh) * P + (t % P)) * d;
      float dot = 0.f;
      for (int i = 0; i < d; ++i) dot = fmaf(qs[i], load_f(cache, cache_dtype, kb + i), dot);
      s = dot * scale;
    }
    const float m_new = fmaxf(m, wave_max(s));  // finite: every chunk in the range holds a valid key
    const float alpha = expf(m - m_new);        // exp(-inf) = 0 on the first chunk
    const float p = valid ? expf(s - m_new) : 0.f;
    l = l * alpha + wave_sum(p);
    m = m_new;
#pragma unroll
    for (int i = 0; i < MAX_D_PER_LANE; ++i) o[i] *= alpha;
    __syncthreads();
    ps[lane] = p;
    __syncthreads();
    const int j_end = min(WAVE, pos - c * WAVE + 1);
    const int j_begin = max(0, first - c * WAVE);
    for (int j = j_begin; j < j_end; ++j) {
      const float pj = ps[j];
      const int tj = c * WAVE + j;
      const int page = bt[tj / P];
      const size_t vb = (((size_t)page * 2 + 1) * Hk + kvh) * (size_t)P * d + (tj % P);
#pragma unroll
      for (int i = 0; i < MAX_D_PER_LANE; ++i) {
        const int e = lane + i * WAVE;
        if (e < d) o[i] = fmaf(pj, load_f(cache, cache_dtype, vb + (size_t)e * P), o[i]);
      }
    }
  }
  const float inv = 1.0f / l;
#pragma unroll
  for (int i = 0; i < MAX_D_PER_LANE; ++i) {
    const int e = lane + i * WAVE;
    if (e < d) store_f(out, out_dtype, (size_t)r * ldo + (size_t)h * d + e, o[i] * inv);
  }
}

APC_EXPORT int apc_paged_attention_plain(const void* q, int q_dtype, int ldq, int q_off, void* out, int out_dtype,
                                         int ldo, int n_rows, int H, int Hk, int d, const void* cache,
                                         int cache_dtype, int page_tokens, const int* block_table, int max_blocks,
                                         const int* positions, const int* row_seg, int window, float scale,
                                         hipStream_t stream) {
  if (n_rows <= 0) return 0;
  if (H <= 0 || Hk <= 0 || H % Hk || d <= 0 || page_tokens <= 0 || max_blocks <= 0 || window < 0)
    return APC_ERR_BAD_ARG;
  if (d > MAX_D_PER_LANE * WAVE || H > 65535) return APC_ERR_UNSUPPORTED;
  hipLaunchKernelGGL(paged_attention_plain_kernel, dim3(n_rows, H), dim3(64), 0, stream, q, q_dtype, ldq, q_off, out,
                     out_dtype, ldo, H, Hk, d, cache, cache_dtype, page_tokens, block_table, max_blocks, positions,
                     row_seg, window, scale);
  APC_LAUNCH_CHECK();
  return 0;
}
