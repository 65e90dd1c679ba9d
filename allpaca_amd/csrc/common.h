// Shared helpers of the gfx950 kernel libraries: element types, conversions,
// wave and block reductions, error reporting.  Device code for MI355X only.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#define APC_EXPORT extern "C" __attribute__((visibility("default")))

// Element type codes shared with the Python side.
enum ApcDType : int { APC_F32 = 0, APC_BF16 = 1, APC_I32 = 2 };

// Error codes returned by every entry point (0 = ok, >0 = hipError_t, <0 = ours).
#define APC_ERR_BAD_ARG (-1)
#define APC_ERR_UNSUPPORTED (-2)

#define APC_LAUNCH_CHECK()                      \
  do {                                          \
    hipError_t e_ = hipGetLastError();          \
    if (e_ != hipSuccess) return (int)e_;       \
  } while (0)

typedef uint16_t bf16_t;  // storage type: the upper half of an IEEE float32

__device__ __forceinline__ float bf16_to_float(bf16_t v) { return __uint_as_float(((uint32_t)v) << 16); }

// round to nearest even; NaN stays NaN.  gfx950 converts two values with one instruction (v_cvt_pk_bf16_f32).
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
  typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
  typedef float floatx2_t __attribute__((ext_vector_type(2)));
  const floatx2_t v = {lo, hi};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t));
}
__device__ __forceinline__ bf16_t float_to_bf16(float f) { return (bf16_t)(pack_bf16x2(f, 0.f) & 0xffffu); }

__device__ __forceinline__ float load_f(const void* p, int dtype, size_t i) {
  return dtype == APC_F32 ? ((const float*)p)[i] : bf16_to_float(((const bf16_t*)p)[i]);
}
__device__ __forceinline__ void store_f(void* p, int dtype, size_t i, float v) {
  if (dtype == APC_F32) ((float*)p)[i] = v; else ((bf16_t*)p)[i] = float_to_bf16(v);
}

__host__ __device__ __forceinline__ size_t dtype_size(int dtype) { return dtype == APC_BF16 ? 2 : 4; }

constexpr int WAVE = 64;

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = WAVE / 2; o > 0; o >>= 1) v += __shfl_xor(v, o, WAVE);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = WAVE / 2; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, WAVE));
  return v;
}

// Sum over a block of NT threads (NT a multiple of 64, at most 1024); every thread gets the result.
// The order of additions is fixed by NT alone.
template <int NT>
__device__ __forceinline__ float block_sum(float v, float* smem /* >= NT/64 floats */) {
  v = wave_sum(v);
  const int w = threadIdx.x / WAVE, l = threadIdx.x % WAVE;
  __syncthreads();
  if (l == 0) smem[w] = v;
  __syncthreads();
  float t = 0.f;
#pragma unroll
  for (int i = 0; i < NT / WAVE; ++i) t += smem[i];
  return t;
}
template <int NT>
__device__ __forceinline__ float block_max(float v, float* smem) {
  v = wave_max(v);
  const int w = threadIdx.x / WAVE, l = threadIdx.x % WAVE;
  __syncthreads();
  if (l == 0) smem[w] = v;
  __syncthreads();
  float t = smem[0];
#pragma unroll
  for (int i = 1; i < NT / WAVE; ++i) t = fmaxf(t, smem[i]);
  return t;
}

__host__ __device__ static inline int ceil_div(int a, int b) { return (a + b - 1) / b; }
