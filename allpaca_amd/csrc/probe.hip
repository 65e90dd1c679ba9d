// What this card delivers, measured: a streaming read of a large buffer (the yardstick for the decode step, which
// is bound by reading every weight once) and a loop of independent bfloat16 MFMAs (the yardstick for the prefill
// products).  Fractions of the published peaks (8 TB/s, 2.5 PFLOP/s) say how far a kernel is from the data sheet;
// fractions of these say how far it is from what any kernel can reach here.
// The reference reports against published peaks only (tools/bench/src/roofline.rs:35-70).
#include "mfma.h"

// Every thread reads 16 bytes at a time, UNROLL loads in flight, the block walks through its own contiguous share of
// the buffer; the sums keep the loads alive and go to out[block].  ONCE: with loads that the caches do not keep, which is
// how the decode kernels read weights, keys and values (8 GiB: 7.3 TB/s against 6.2 TB/s with ordinary loads).
typedef uint32_t probe_u32x4 __attribute__((ext_vector_type(4)));
template <bool ONCE>
__device__ __forceinline__ uint4 probe_load(const uint4* p) {
  if constexpr (ONCE) {
    const probe_u32x4 v = __builtin_nontemporal_load(reinterpret_cast<const probe_u32x4*>(p));
    return uint4{v[0], v[1], v[2], v[3]};
  } else {
    return *p;
  }
}
template <int UNROLL, bool ONCE>
__global__ __launch_bounds__(256) void probe_read_kernel(const uint4* __restrict__ p, size_t n16, float* __restrict__ out) {
  const size_t per_block = (n16 + gridDim.x - 1) / gridDim.x;
  const size_t lo = (size_t)blockIdx.x * per_block, hi = lo + per_block < n16 ? lo + per_block : n16;
  uint32_t acc = 0;
  size_t i = lo + threadIdx.x;
  for (; i + (size_t)(UNROLL - 1) * 256 < hi; i += (size_t)UNROLL * 256) {
    uint4 v[UNROLL];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) v[u] = probe_load<ONCE>(p + i + (size_t)u * 256);
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) acc += v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
  }
  for (; i < hi; i += 256) {
    const uint4 v = probe_load<ONCE>(p + i);
    acc += v.x ^ v.y ^ v.z ^ v.w;
  }
  __shared__ float part[4];
  float f = wave_sum((float)(acc & 0xffffu));
  if (threadIdx.x % WAVE == 0) part[threadIdx.x / WAVE] = f;
  __syncthreads();
  if (threadIdx.x == 0) out[blockIdx.x] = part[0] + part[1] + part[2] + part[3];
}

// Reads `bytes` (a multiple of 16) from p with `blocks` blocks of 256 threads; out: float [blocks].  once: 1 for loads
// that the caches do not keep.
APC_EXPORT int apc_probe_read(const void* p, size_t bytes, float* out, int blocks, int unroll, int once,
                              hipStream_t stream) {
  if (!p || !out || blocks <= 0 || bytes % 16 || ((uintptr_t)p & 15u)) return APC_ERR_BAD_ARG;
  const size_t n16 = bytes / 16;
#define PROBE_READ(U_, O_) \
  hipLaunchKernelGGL((probe_read_kernel<U_, O_>), dim3(blocks), dim3(256), 0, stream, (const uint4*)p, n16, out)
  if (unroll == 8 && once) PROBE_READ(8, true);
  else if (unroll == 8) PROBE_READ(8, false);
  else if (unroll == 4 && once) PROBE_READ(4, true);
  else if (unroll == 4) PROBE_READ(4, false);
  else if (unroll == 2 && once) PROBE_READ(2, true);
  else if (unroll == 2) PROBE_READ(2, false);
  else return APC_ERR_BAD_ARG;
#undef PROBE_READ
  APC_LAUNCH_CHECK();
  return 0;
}

// Every wave issues `iters` rounds of 8 independent v_mfma_f32_32x32x16_bf16 on registers (no memory traffic):
// 8 * 2 * 32 * 32 * 16 flops a round and wave.  out: float [blocks * 256] (keeps the work alive).
__global__ __launch_bounds__(256) void probe_mfma_kernel(int iters, float* __restrict__ out) {
  Frag a, b;
#pragma unroll
  for (int w = 0; w < 4; ++w) {
    a.w[w] = 0x3f803f80u + threadIdx.x;  // finite bfloat16 pairs
    b.w[w] = 0x3f003f00u + blockIdx.x;
  }
  floatx16 c[8];
#pragma unroll
  for (int j = 0; j < 8; ++j)
#pragma unroll
    for (int r = 0; r < 16; ++r) c[j][r] = 0.f;
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int j = 0; j < 8; ++j) c[j] = mfma32(a, b, c[j]);
  }
  float s = 0.f;
#pragma unroll
  for (int j = 0; j < 8; ++j)
#pragma unroll
    for (int r = 0; r < 16; ++r) s += c[j][r];
  out[(size_t)blockIdx.x * 256 + threadIdx.x] = s;
}

APC_EXPORT int apc_probe_mfma(int iters, float* out, int blocks, hipStream_t stream) {
  if (!out || blocks <= 0 || iters <= 0) return APC_ERR_BAD_ARG;
  hipLaunchKernelGGL(probe_mfma_kernel, dim3(blocks), dim3(256), 0, stream, iters, out);
  APC_LAUNCH_CHECK();
  return 0;
}
