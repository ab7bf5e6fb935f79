// Shared device helpers for the gfx950 kernels: vector types, bfloat16 conversion,
// fixed-order wave reductions.  All sources are compiled with -ffp-contract=off, so a
// multiply-add is fused only where the code says fmaf.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

typedef uint16_t bf16_t;  // raw bfloat16 bits
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2;

#define BW_WAVE 64

__device__ __forceinline__ float bf16_to_f32(bf16_t v) { return __uint_as_float(((uint32_t)v) << 16); }

// Round to nearest even; NaN stays NaN.
__device__ __forceinline__ bf16_t f32_to_bf16(float f) {
  uint32_t b = __float_as_uint(f);
  if ((b & 0x7fffffffu) > 0x7f800000u) return (bf16_t)((b >> 16) | 0x40);
  b += 0x7fffu + ((b >> 16) & 1u);
  return (bf16_t)(b >> 16);
}

__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
  return (uint32_t)f32_to_bf16(lo) | ((uint32_t)f32_to_bf16(hi) << 16);
}

__device__ __forceinline__ bf16x8 as_bf16x8(u32x4 v) {
  union { u32x4 u; bf16x8 b; } c;
  c.u = v;
  return c.b;
}

// exp(x) through the hardware exp2; one fixed instruction sequence wherever it is used.
__device__ __forceinline__ float fast_exp(float x) { return __builtin_amdgcn_exp2f(x * 1.44269504088896340736f); }

// Sum over the 64 lanes by xor butterflies.  Addition commutes, so every lane ends with
// the same bits, and the order of additions is the same for every row of every launch.
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) v += __shfl_xor(v, off, BW_WAVE);
  return v;
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, BW_WAVE));
  return v;
}

// The launch wrappers return hipGetLastError() as int; 0 is success.
#define BW_LAUNCH_CHECK() ((int)hipGetLastError())
