// Plain kernels: one obvious loop nest each, all arithmetic in 32-bit float with
// a fixed order of additions per output element, any element type in and out.
// They are the whole float32 path and the small memory-bound steps of the
// bfloat16 path (embedding, norm, rotation + cache write, gathers).
#include "common.h"

// ---------------------------------------------------------------------------
// embedding: out[t, :] = table[tokens[t], :]
// Reference: embed_gather_rows_kernel, hip/src/kernels.cpp:11337-11356.
// ---------------------------------------------------------------------------
__global__ void embed_rows_kernel(const void* __restrict__ table, int table_dtype, const int* __restrict__ tokens,
                                  void* __restrict__ out, int out_dtype, int dim, int ldo) {
  const int t = blockIdx.x;
  const size_t src = (size_t)tokens[t] * dim;
  for (int i = threadIdx.x; i < dim; i += blockDim.x)
    store_f(out, out_dtype, (size_t)t * ldo + i, load_f(table, table_dtype, src + i));
}

APC_EXPORT int apc_embed_rows(const void* table, int table_dtype, const int* tokens, void* out, int out_dtype,
                              int n_tok, int dim, int ldo, hipStream_t stream) {
  if (n_tok <= 0) return 0;
  if (dim <= 0 || ldo < dim) return APC_ERR_BAD_ARG;
  hipLaunchKernelGGL(embed_rows_kernel, dim3(n_tok), dim3(256), 0, stream, table, table_dtype, tokens, out, out_dtype,
                     dim, ldo);
  APC_LAUNCH_CHECK();
  return 0;
}

// The same from a bfloat16 table kept in the tiled layout of the MFMA kernels (tiles of 16 rows x 32 columns,
// lane = (k % 32) / 8 * 16 + n % 16 holding the 8 elements k % 8; `chunks` tiles per 16-row band): a tied
// output head and the embedding then share one buffer.
__global__ void embed_rows_tiled_kernel(const bf16_t* __restrict__ table, int chunks, const int* __restrict__ tokens,
                                        void* __restrict__ out, int out_dtype, int dim, int ldo) {
  const int t = blockIdx.x;
  const int n = tokens[t];
  const bf16_t* band = table + (size_t)(n / 16) * chunks * 512 + (n % 16) * 8;
  for (int k = threadIdx.x; k < dim; k += blockDim.x) {
    const bf16_t v = band[(size_t)(k / 32) * 512 + ((k % 32) / 8) * 128 + (k % 8)];
    store_f(out, out_dtype, (size_t)t * ldo + k, bf16_to_float(v));
  }
}

APC_EXPORT int apc_embed_rows_tiled(const void* table, int chunks, const int* tokens, void* out, int out_dtype,
                                    int n_tok, int dim, int ldo, hipStream_t stream) {
  if (n_tok <= 0) return 0;
  if (dim <= 0 || ldo < dim || chunks * 32 < dim) return APC_ERR_BAD_ARG;
  hipLaunchKernelGGL(embed_rows_tiled_kernel, dim3(n_tok), dim3(256), 0, stream, (const bf16_t*)table, chunks, tokens,
                     out, out_dtype, dim, ldo);
  APC_LAUNCH_CHECK();
  return 0;
}

// ---------------------------------------------------------------------------
// gather rows: out[r, :] = x[rows[r], :]   (same element type)
// ---------------------------------------------------------------------------
__global__ void gather_rows_kernel(const void* __restrict__ x, int dtype, int ldx, const int* __restrict__ rows,
                                   void* __restrict__ out, int ldo, int dim) {
  const int r = blockIdx.x;
  const size_t src = (size_t)rows[r] * ldx;
  for (int i = threadIdx.x; i < dim; i += blockDim.x)
    store_f(out, dtype, (size_t)r * ldo + i, load_f(x, dtype, src + i));
}

APC_EXPORT int apc_gather_rows(const void* x, int dtype, int ldx, const int* rows, void* out, int ldo, int n_rows,
                               int dim, hipStream_t stream) {
  if (n_rows <= 0) return 0;
  if (dim <= 0 || ldx < dim || ldo < dim) return APC_ERR_BAD_ARG;
  hipLaunchKernelGGL(gather_rows_kernel, dim3(n_rows), dim3(256), 0, stream, x, dtype, ldx, rows, out, ldo, dim);
  APC_LAUNCH_CHECK();
  return 0;
}

// ---------------------------------------------------------------------------
// RMS norm over rows: ss = sum x^2, inv = 1/sqrt(ss/D + eps), out = x*inv*w.
// eps inside the root, added to the mean; the weight multiplies after.
// Reference: crates/allpaca-cpu/src/kernels.rs:492-507, hip/src/kernels.cpp:9639-9654.
// `rows` (optional) selects input rows: out[r] = norm(x[rows[r]]).
// ---------------------------------------------------------------------------
template <int NT>
__global__ void rmsnorm_rows_kernel(const void* __restrict__ x, int x_dtype, int ldx, const int* __restrict__ rows,
                                    const float* __restrict__ w, float eps, void* __restrict__ out, int out_dtype,
                                    int ldo, int dim) {
  __shared__ float red[NT / WAVE];
  const int r = blockIdx.x;
  const size_t src = (size_t)(rows ? rows[r] : r) * ldx;
  float ss = 0.f;
  for (int i = threadIdx.x; i < dim; i += NT) {
    const float v = load_f(x, x_dtype, src + i);
    ss = fmaf(v, v, ss);
  }
  ss = block_sum<NT>(ss, red);
  const float inv = 1.0f / sqrtf(ss / (float)dim + eps);
  for (int i = threadIdx.x; i < dim; i += NT) {
    const float v = load_f(x, x_dtype, src + i);
    store_f(out, out_dtype, (size_t)r * ldo + i, (v * inv) * w[i]);
  }
}

// The same for float32 rows whose width is a multiple of 4 and at most NT*4*VPT: every thread keeps its
// elements in registers between the sum and the scaling, and all its loads are in flight together.
// Which of the two kernels runs, and so the order of the additions, is fixed by the width and the
// alignment of the rows alone, never by the batch.
template <int NT, int VPT>
__global__ __launch_bounds__(NT) void rmsnorm_rows_f32_kernel(const float* __restrict__ x, int ldx,
                                                              const int* __restrict__ rows,
                                                              const float* __restrict__ w, float eps,
                                                              void* __restrict__ out, int out_dtype, int ldo,
                                                              int dim) {
  __shared__ float red[NT / WAVE];
  const int r = blockIdx.x;
  const float4* src = reinterpret_cast<const float4*>(x + (size_t)(rows ? rows[r] : r) * ldx);
  const int n4 = dim / 4;
  float4 v[VPT];
#pragma unroll
  for (int j = 0; j < VPT; ++j) {
    const int i = threadIdx.x + j * NT;
    v[j] = i < n4 ? src[i] : float4{0.f, 0.f, 0.f, 0.f};
  }
  float ss = 0.f;
#pragma unroll
  for (int j = 0; j < VPT; ++j) {
    ss = fmaf(v[j].x, v[j].x, ss);
    ss = fmaf(v[j].y, v[j].y, ss);
    ss = fmaf(v[j].z, v[j].z, ss);
    ss = fmaf(v[j].w, v[j].w, ss);
  }
  ss = block_sum<NT>(ss, red);
  const float inv = 1.0f / sqrtf(ss / (float)dim + eps);
  const float4* w4 = reinterpret_cast<const float4*>(w);
#pragma unroll
  for (int j = 0; j < VPT; ++j) {
    const int i = threadIdx.x + j * NT;
    if (i >= n4) continue;
    const float4 g = w4[i];
    const float o0 = (v[j].x * inv) * g.x, o1 = (v[j].y * inv) * g.y, o2 = (v[j].z * inv) * g.z,
                o3 = (v[j].w * inv) * g.w;
    const size_t at = (size_t)r * ldo + (size_t)i * 4;
    if (out_dtype == APC_F32) {
      *reinterpret_cast<float4*>((float*)out + at) = float4{o0, o1, o2, o3};
    } else {
      uint2 pk;
      pk.x = (uint32_t)float_to_bf16(o0) | ((uint32_t)float_to_bf16(o1) << 16);
      pk.y = (uint32_t)float_to_bf16(o2) | ((uint32_t)float_to_bf16(o3) << 16);
      *reinterpret_cast<uint2*>((bf16_t*)out + at) = pk;
    }
  }
}

APC_EXPORT int apc_rmsnorm_rows(const void* x, int x_dtype, int ldx, const int* rows, const float* w, float eps,
                                void* out, int out_dtype, int ldo, int n_rows, int dim, hipStream_t stream) {
  if (n_rows <= 0) return 0;
  if (dim <= 0 || ldx < dim || ldo < dim) return APC_ERR_BAD_ARG;
  const bool vec = x_dtype == APC_F32 && dim % 4 == 0 && ldx % 4 == 0 && ldo % 4 == 0 && dim <= 256 * 4 * 8 &&
                   ((uintptr_t)x % 16) == 0 && ((uintptr_t)w % 16) == 0 && ((uintptr_t)out % 16) == 0;
  if (vec) {
    const int n4 = dim / 4;
#define RN_LAUNCH(VPT_)                                                                                             \
  hipLaunchKernelGGL((rmsnorm_rows_f32_kernel<256, VPT_>), dim3(n_rows), dim3(256), 0, stream, (const float*)x, ldx, \
                     rows, w, eps, out, out_dtype, ldo, dim)
    if (n4 <= 256) RN_LAUNCH(1);
    else if (n4 <= 512) RN_LAUNCH(2);
    else if (n4 <= 1024) RN_LAUNCH(4);
    else RN_LAUNCH(8);
#undef RN_LAUNCH
  } else {
    hipLaunchKernelGGL(rmsnorm_rows_kernel<256>, dim3(n_rows), dim3(256), 0, stream, x, x_dtype, ldx, rows, w, eps,
                       out, out_dtype, ldo, dim);
  }
  APC_LAUNCH_CHECK();
  return 0;
}

// ---------------------------------------------------------------------------
// residual: acc[t, :] += y[t, :]  (acc float32; the sum is made in 32-bit)
// Reference: residual_add, hip/src/kernels.cpp:11357-11365.
// ---------------------------------------------------------------------------
__global__ void add_into_kernel(float* __restrict__ acc, int lda, const void* __restrict__ y, int y_dtype, int ldy,
                                int dim) {
  const int t = blockIdx.x;
  for (int i = threadIdx.x; i < dim; i += blockDim.x)
    acc[(size_t)t * lda + i] += load_f(y, y_dtype, (size_t)t * ldy + i);
}

APC_EXPORT int apc_add_into(float* acc, int lda, const void* y, int y_dtype, int ldy, int n_rows, int dim,
                            hipStream_t stream) {
  if (n_rows <= 0) return 0;
  if (dim <= 0 || lda < dim || ldy < dim) return APC_ERR_BAD_ARG;
  hipLaunchKernelGGL(add_into_kernel, dim3(n_rows), dim3(256), 0, stream, acc, lda, y, y_dtype, ldy, dim);
  APC_LAUNCH_CHECK();
  return 0;
}

// ---------------------------------------------------------------------------
// SwiGLU activation: out[t, f] = silu(gu[t, f]) * gu[t, F + f], silu(z) = z/(1+exp(-z)).
// Reference: silu_mul_kernel, hip/src/kernels.cpp:10003-10010; kernels.rs:869-871.
// ---------------------------------------------------------------------------
__global__ void silu_mul_kernel(const void* __restrict__ gu, int in_dtype, int ldg, void* __restrict__ out,
                                int out_dtype, int ldo, int F) {
  const int t = blockIdx.y;
  const int f = blockIdx.x * blockDim.x + threadIdx.x;
  if (f >= F) return;
  const float g = load_f(gu, in_dtype, (size_t)t * ldg + f);
  const float u = load_f(gu, in_dtype, (size_t)t * ldg + F + f);
  store_f(out, out_dtype, (size_t)t * ldo + f, (g / (1.0f + expf(-g))) * u);
}

APC_EXPORT int apc_silu_mul(const void* gu, int in_dtype, int ldg, void* out, int out_dtype, int ldo, int n_rows,
                            int F, hipStream_t stream) {
  if (n_rows <= 0) return 0;
  if (F <= 0 || ldg < 2 * F || ldo < F || n_rows > 65535) return APC_ERR_BAD_ARG;
  hipLaunchKernelGGL(silu_mul_kernel, dim3(ceil_div(F, 256), n_rows), dim3(256), 0, stream, gu, in_dtype, ldg, out,
                     out_dtype, ldo, F);
  APC_LAUNCH_CHECK();
  return 0;
}

// ---------------------------------------------------------------------------
// Rotation of q and k by position, and the write of k, v into the paged cache.
//
// qkv: [T, ld] rows holding q heads at column q_off, k heads at k_off, v heads at v_off.
// Rotation pairs (i, i + rot/2) inside the first `rot` elements of each head:
//   x_i' = a cos - b sin,  x_{i+rot/2}' = a sin + b cos
// (crates/allpaca-cpu/src/kernels.rs:676-682).  cos/sin come from a table
// [max_pos, 2, rot/2] made on the host in 64-bit and rounded once to float32.
// q is rotated in place.  k (rotated) and v go to the page
//   page = block_table[seg][pos / P], slot = pos % P
// (reference: page = pos / P, slot = pos % P, crates/allpaca-core/src/model.rs:10439-10443):
//   keys    cache[page][0][kv_head][slot][i]      (a key's elements lie together)
//   values  cache[page][1][kv_head][i][slot]      (an element's slots lie together: the
//           value product sums over positions, and matrix cores want that axis contiguous)
// With cache == nullptr only the rotation is done (k in place as well).
// ---------------------------------------------------------------------------
__global__ void rope_kv_write_kernel(void* __restrict__ qkv, int dtype, int ld, int q_off, int k_off, int v_off,
                                     int H, int Hk, int d, int rot, const float* __restrict__ cos_sin,
                                     const int* __restrict__ positions, const int* __restrict__ row_seg,
                                     const int* __restrict__ block_table, int max_blocks, void* __restrict__ cache,
                                     int cache_dtype, int P) {
  const int t = blockIdx.x;
  const int slot_head = blockIdx.y;  // [0,H): q   [H,H+Hk): k   [H+Hk,H+2Hk): v
  const int pos = positions[t];
  const int half = rot / 2;
  size_t src;
  int kind, head;
  if (slot_head < H) { kind = 0; head = slot_head; src = (size_t)t * ld + q_off + (size_t)head * d; }
  else if (slot_head < H + Hk) { kind = 1; head = slot_head - H; src = (size_t)t * ld + k_off + (size_t)head * d; }
  else { kind = 2; head = slot_head - H - Hk; src = (size_t)t * ld + v_off + (size_t)head * d; }

  size_t dst = 0;
  if (kind != 0 && cache) {
    const int page = block_table[(size_t)row_seg[t] * max_blocks + pos / P];
    const size_t head_base = (((size_t)page * 2 + (kind - 1)) * Hk + head) * (size_t)P * d;
    dst = kind == 1 ? head_base + (size_t)(pos % P) * d : head_base + (pos % P);
  }
  if (kind == 2) {
    if (!cache) return;
    for (int i = threadIdx.x; i < d; i += blockDim.x)
      store_f(cache, cache_dtype, dst + (size_t)i * P, load_f(qkv, dtype, src + i));
    return;
  }
  const float* cs = cos_sin + (size_t)pos * rot;  // [2][half]
  for (int i = threadIdx.x; i < half; i += blockDim.x) {
    const float a = load_f(qkv, dtype, src + i), b = load_f(qkv, dtype, src + i + half);
    const float c = cs[i], s = cs[half + i];
    const float ra = a * c - b * s, rb = a * s + b * c;
    if (kind == 0 || !cache) {
      store_f(qkv, dtype, src + i, ra);
      store_f(qkv, dtype, src + i + half, rb);
    } else {
      store_f(cache, cache_dtype, dst + i, ra);
      store_f(cache, cache_dtype, dst + i + half, rb);
    }
  }
  if (kind == 1 && cache)  // the part of a head beyond the rotated width is copied
    for (int i = rot + threadIdx.x; i < d; i += blockDim.x)
      store_f(cache, cache_dtype, dst + i, load_f(qkv, dtype, src + i));
}

APC_EXPORT int apc_rope_kv_write(void* qkv, int dtype, int ld, int q_off, int k_off, int v_off, int n_tok, int H,
                                 int Hk, int d, int rot, const float* cos_sin, const int* positions,
                                 const int* row_seg, const int* block_table, int max_blocks, void* cache,
                                 int cache_dtype, int page_tokens, hipStream_t stream) {
  if (n_tok <= 0) return 0;
  if (H < 0 || Hk < 0 || d <= 0 || rot < 0 || rot > d || (rot & 1) || (rot > 0 && !cos_sin)) return APC_ERR_BAD_ARG;
  if (cache && (page_tokens <= 0 || !block_table || !row_seg || max_blocks <= 0)) return APC_ERR_BAD_ARG;
  if (H + 2 * Hk > 65535 || H + 2 * Hk == 0) return APC_ERR_BAD_ARG;
  hipLaunchKernelGGL(rope_kv_write_kernel, dim3(n_tok, H + 2 * Hk), dim3(64), 0, stream, qkv, dtype, ld, q_off, k_off,
                     v_off, H, Hk, d, rot, cos_sin, positions, row_seg, block_table, max_blocks, cache, cache_dtype,
                     page_tokens);
  APC_LAUNCH_CHECK();
  return 0;
}

// ---------------------------------------------------------------------------
// element type conversion (contiguous)
// ---------------------------------------------------------------------------
__global__ void cast_kernel(const void* __restrict__ in, int in_dtype, void* __restrict__ out, int out_dtype, size_t n) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) store_f(out, out_dtype, i, load_f(in, in_dtype, i));
}

APC_EXPORT int apc_cast(const void* in, int in_dtype, void* out, int out_dtype, size_t n, hipStream_t stream) {
  if (n == 0) return 0;
  const size_t blocks = (n + 255) / 256;
  if (blocks > 0x7fffffffu) return APC_ERR_BAD_ARG;
  hipLaunchKernelGGL(cast_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, in, in_dtype, out, out_dtype, n);
  APC_LAUNCH_CHECK();
  return 0;
}
