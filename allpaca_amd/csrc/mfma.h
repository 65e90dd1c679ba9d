// MFMA helpers for gfx950 (CDNA4), 64-wide wavefronts.
//
// v_mfma_f32_16x16x32_bf16:  D[16x16] += A[16x32] * B[32x16]
//   lane l gives A[i = l%16][k = (l/16)*8 .. +7] and B[k = (l/16)*8 .. +7][j = l%16] (8 bfloat16 = 16 bytes each)
//   lane l holds D[i = (l/16)*4 + r][j = l%16] in register r = 0..3
// v_mfma_f32_32x32x16_bf16:  D[32x32] += A[32x16] * B[16x32]
//   lane l gives A[i = l%32][k = (l/32)*8 .. +7] and B[k = (l/32)*8 .. +7][j = l%32]
//   lane l holds D[i = (r/4)*8 + (l/32)*4 + r%4][j = l%32] in register r = 0..15
// Both operands want the summed axis contiguous per lane, which is how row-major
// activations [rows, K] and weights [out, K] already lie.
#pragma once
#include "common.h"

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef float floatx16 __attribute__((ext_vector_type(16)));

struct alignas(16) Frag {  // 8 bfloat16 as raw bits
  uint32_t w[4];
};

__device__ __forceinline__ bf16x8_t as_bf16x8(const Frag& f) { return __builtin_bit_cast(bf16x8_t, f); }

__device__ __forceinline__ Frag load_frag(const bf16_t* p) { return *reinterpret_cast<const Frag*>(p); }
// The same for bytes that are read once (weights of a step with few rows, keys and values of a decoded row): a
// non-temporal load, which the caches do not keep.  A read of 8 GiB streams at 7.3 TB/s this way and at 6.2 TB/s with
// ordinary loads (measured with blocks that walk their own share, 16 bytes a lane, 8 loads in flight a lane).
__device__ __forceinline__ Frag load_frag_once(const bf16_t* p) {
  typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
  return __builtin_bit_cast(Frag, __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p)));
}
__device__ __forceinline__ Frag zero_frag() { Frag f; f.w[0] = f.w[1] = f.w[2] = f.w[3] = 0u; return f; }

// A buffer descriptor over global memory from `base` on (raw, no stride, no bound that matters): a load then takes the
// descriptor and a scalar byte offset from scalar registers and one 32-bit byte offset per lane.
typedef __amdgpu_buffer_rsrc_t BufferRsrc;
__device__ __forceinline__ BufferRsrc make_rsrc(const void* base) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, 0x7fffffff, 0x00020000);
}
__device__ __forceinline__ Frag load_frag_buffer(BufferRsrc rsrc, int lane_bytes, int scalar_bytes) {
  typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
  return __builtin_bit_cast(Frag, (u32x4)__builtin_amdgcn_raw_buffer_load_b128(rsrc, lane_bytes, scalar_bytes, 0));
}

// One wave writes LDS and then reads what its other lanes wrote.  The LDS serves a wave's accesses in the order
// it issues them, so all that is needed is that the compiler keeps that order: a wave barrier (no wait on
// outstanding global loads, unlike a fence, so loads issued ahead stay in flight).
__device__ __forceinline__ void wave_lds_order() { __builtin_amdgcn_wave_barrier(); }

__device__ __forceinline__ floatx4 mfma16(const Frag& a, const Frag& b, floatx4 c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(a), as_bf16x8(b), c, 0, 0, 0);
}
__device__ __forceinline__ floatx16 mfma32(const Frag& a, const Frag& b, floatx16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(as_bf16x8(a), as_bf16x8(b), c, 0, 0, 0);
}

__device__ __forceinline__ float silu_f(float g) { return g / (1.0f + __expf(-g)); }
