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

// Round to nearest even with the hardware conversion (v_cvt_pk_bf16_f32); NaN stays NaN.
typedef __attribute__((ext_vector_type(2))) float f32x2_t;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2_t;

__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
  const f32x2_t v = {lo, hi};
  const bf16x2_t r = __builtin_convertvector(v, bf16x2_t);
  return __builtin_bit_cast(uint32_t, r);
}

__device__ __forceinline__ bf16_t f32_to_bf16(float f) { return (bf16_t)(pack_bf16x2(f, 0.0f) & 0xffffu); }

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

// Sum of squares of one row given as 16-byte vectors: lane l owns vectors l, l+64, ... and runs
// one fused multiply-add chain over their elements in ascending order; the lanes are joined by
// the xor butterflies of wave_sum.  Every kernel that needs a row's sum of squares in bfloat16
// mode calls this, so the bits agree.
__device__ __forceinline__ float row_sumsq_vec(const f32x4* __restrict__ xv, int nvec, int lane) {
  float acc = 0.0f;
  constexpr int UN = 8;
  for (int c0 = 0; c0 < nvec; c0 += 64 * UN) {
    f32x4 v[UN];
#pragma unroll
    for (int j = 0; j < UN; ++j) {
      const int c = c0 + 64 * j + lane;
      v[j] = c < nvec ? xv[c] : (f32x4){0.f, 0.f, 0.f, 0.f};
    }
#pragma unroll
    for (int j = 0; j < UN; ++j)
#pragma unroll
      for (int e = 0; e < 4; ++e) acc = fmaf(v[j][e], v[j][e], acc);
  }
  return wave_sum(acc);
}

// Load 4 norm weights (bfloat16 or 32-bit) starting at element 4c as floats.
__device__ __forceinline__ f32x4 load_norm_w4(const void* __restrict__ w, int is_bf16, int c) {
  if (is_bf16) {
    const u32x2 p = reinterpret_cast<const u32x2*>(w)[c];
    return (f32x4){__uint_as_float(p[0] << 16), __uint_as_float(p[0] & 0xffff0000u), __uint_as_float(p[1] << 16),
                   __uint_as_float(p[1] & 0xffff0000u)};
  }
  return reinterpret_cast<const f32x4*>(w)[c];
}

// RMSNorm of one row of at most 2048 elements (a multiple of 4) by one wave, with every load
// issued before anything is computed: the row's vectors stay in registers between the sum of
// squares and the scaling.  Same order and statements as row_sumsq_vec and the store loop of
// rmsnorm_bf16_kernel.  ``store(c, packed)`` receives vector c as four bfloat16 in 8 bytes.
template <typename Store>
__device__ __forceinline__ void rmsnorm_row_small(const f32x4* __restrict__ xv, const void* __restrict__ w,
                                                  int w_is_bf16, int nvec, int dim, float eps, int lane, Store store) {
  constexpr int UN = 8;
  f32x4 v[UN], wv[UN];
#pragma unroll
  for (int j = 0; j < UN; ++j) {
    const int c = 64 * j + lane;
    v[j] = c < nvec ? xv[c] : (f32x4){0.f, 0.f, 0.f, 0.f};
    wv[j] = c < nvec ? load_norm_w4(w, w_is_bf16, c) : (f32x4){0.f, 0.f, 0.f, 0.f};
  }
  float acc = 0.0f;
#pragma unroll
  for (int j = 0; j < UN; ++j)
#pragma unroll
    for (int e = 0; e < 4; ++e) acc = fmaf(v[j][e], v[j][e], acc);
  acc = wave_sum(acc);
  const float inv = 1.0f / sqrtf(acc / (float)dim + eps);
#pragma unroll
  for (int j = 0; j < UN; ++j) {
    const int c = 64 * j + lane;
    if (c < nvec) {
      u32x2 pk = {pack_bf16x2((v[j][0] * inv) * wv[j][0], (v[j][1] * inv) * wv[j][1]),
                  pack_bf16x2((v[j][2] * inv) * wv[j][2], (v[j][3] * inv) * wv[j][3])};
      store(c, pk);
    }
  }
}

// The launch wrappers return hipGetLastError() as int; 0 is success.
#define BW_LAUNCH_CHECK() ((int)hipGetLastError())
