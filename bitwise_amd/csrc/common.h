// Shared device helpers for the gfx950 kernels: vector types, bfloat16 conversion,
// fixed-order wave reductions.  All sources are compiled with -ffp-contract=off, so a
// multiply-add is fused only where the code says fmaf.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "layout.h"

typedef uint16_t bf16_t;  // raw bfloat16 bits
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2;

#define BW_WAVE 64

// The wave's number in its workgroup as a scalar: the compiler cannot see that threadIdx.x >> 6 is
// the same for all lanes, and everything derived from it (segments, strips, loop bounds) would
// be computed per lane and branched on per lane.  A branch around a matrix instruction must be
// scalar in particular: the matrix cores ignore the execution mask.
__device__ __forceinline__ int wave_index() { return __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6)); }

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

// exp(x) of the 32-bit path: one fixed sequence of IEEE operations (a rounding to the nearest integer,
// fused multiply-adds, multiplications by powers of two) and no library call, so that a scalar program
// on any IEEE machine gives the same bits.  x = k ln2 + r with k = rint(x * log2e), |r| <= 0.35 (ln2 in
// two parts, the high one with trailing zero bits); e^r by the Taylor polynomial of degree 7 in Horner
// form (its remainder is below a tenth of an ulp); the result scaled by 2^k in two exact steps.
// Arguments below -87 give 0 (the result would be under the smallest normal number), arguments above 89
// give +inf, NaN stays NaN; exp(0) is exactly 1.
__device__ __forceinline__ float bw_expf(float x) {
  // no branch, selects at the end: a kernel's matrix instructions must not end up under a partial execution mask
  const float xc = fminf(fmaxf(x, -87.0f), 89.0f);          // (NaN becomes -87; the selects below put it back)
  const float kf = __builtin_rintf(xc * 0x1.715476p+0f);
  float r = fmaf(kf, -0x1.62e4p-1f, xc);
  r = fmaf(kf, -0x1.7f7d1cp-20f, r);
  float p = 0x1.a01a02p-13f;
  p = fmaf(p, r, 0x1.6c16c2p-10f);
  p = fmaf(p, r, 0x1.111112p-7f);
  p = fmaf(p, r, 0x1.555556p-5f);
  p = fmaf(p, r, 0x1.555556p-3f);
  p = fmaf(p, r, 0.5f);
  p = fmaf(p, r, 1.0f);
  p = fmaf(p, r, 1.0f);
  const int k = (int)kf, k1 = k >> 1, k2 = k - k1;          // both within [-64, 64]
  float y = (p * __uint_as_float((uint32_t)(k1 + 127) << 23)) * __uint_as_float((uint32_t)(k2 + 127) << 23);
  y = x > 89.0f ? __builtin_inff() : y;
  y = !(x >= -87.0f) ? ((x != x) ? x : 0.0f) : y;
  return y;
}

// exp(x) through the hardware exp2; one fixed instruction sequence wherever it is used.
__device__ __forceinline__ float fast_exp(float x) { return __builtin_amdgcn_exp2f(x * 1.44269504088896340736f); }

// SiLU(g) * u as every bfloat16 kernel computes it: the exponential through the hardware exp2 and the quotient through
// the hardware reciprocal (the correctly rounded division is ten instructions an element, and the result is
// rounded to bfloat16 anyway); one fixed instruction sequence wherever it is used, so every route gives the same bits.
__device__ __forceinline__ float silu_times(float g, float u) { return g * __builtin_amdgcn_rcpf(1.0f + fast_exp(-g)) * u; }

// Lane exchanges from register to register (no trip through LDS).  The halves and quarters of the wave by gfx950's
// lane swaps: of (v, v) swapped, the first result holds in every lane the value of its partner or its own in the
// lower half (32: lanes 0-31; 16: the even rows of 16 lanes), the second the one in the upper half; an operation
// that commutes takes the two as they come.  Within a row of 16 lanes by data-parallel moves: l ^ 8 is a rotation
// of the row by 8, l ^ 4 the mirror image of each 8 lanes followed by that of each 4, l ^ 2 and l ^ 1
// permutations of each 4.
template <int OFF>
__device__ __forceinline__ void lane_halves(float v, float& lower, float& upper) {
  static_assert(OFF == 32 || OFF == 16, "halves of the wave or of its halves");
  typedef __attribute__((ext_vector_type(2))) unsigned u2;
  const unsigned u = __float_as_uint(v);
  const u2 r = OFF == 32 ? __builtin_amdgcn_permlane32_swap(u, u, false, false) : __builtin_amdgcn_permlane16_swap(u, u, false, false);
  lower = __uint_as_float(r[0]);
  upper = __uint_as_float(r[1]);
}

template <int OFF>
__device__ __forceinline__ float lane_xor(float v) {
  const int u = (int)__float_as_uint(v);
  if constexpr (OFF == 8) {
    return __uint_as_float((unsigned)__builtin_amdgcn_mov_dpp(u, 0x128, 0xf, 0xf, true));                // row_ror:8
  } else if constexpr (OFF == 4) {
    const int h = __builtin_amdgcn_mov_dpp(u, 0x141, 0xf, 0xf, true);                                    // row_half_mirror: l ^ 7
    return __uint_as_float((unsigned)__builtin_amdgcn_mov_dpp(h, 0x1b, 0xf, 0xf, true));                 // quad_perm [3,2,1,0]: ^ 3
  } else if constexpr (OFF == 2) {
    return __uint_as_float((unsigned)__builtin_amdgcn_mov_dpp(u, 0x4e, 0xf, 0xf, true));                 // quad_perm [2,3,0,1]
  } else {
    static_assert(OFF == 1, "1, 2, 4 or 8");
    return __uint_as_float((unsigned)__builtin_amdgcn_mov_dpp(u, 0xb1, 0xf, 0xf, true));                 // quad_perm [1,0,3,2]
  }
}

__device__ __forceinline__ int row16_min(int v) {
  v = min(v, (int)__float_as_uint(lane_xor<8>(__uint_as_float((unsigned)v))));
  v = min(v, (int)__float_as_uint(lane_xor<4>(__uint_as_float((unsigned)v))));
  v = min(v, (int)__float_as_uint(lane_xor<2>(__uint_as_float((unsigned)v))));
  v = min(v, (int)__float_as_uint(lane_xor<1>(__uint_as_float((unsigned)v))));
  return v;
}

__device__ __forceinline__ int row16_max(int v) {
  v = max(v, (int)__float_as_uint(lane_xor<8>(__uint_as_float((unsigned)v))));
  v = max(v, (int)__float_as_uint(lane_xor<4>(__uint_as_float((unsigned)v))));
  v = max(v, (int)__float_as_uint(lane_xor<2>(__uint_as_float((unsigned)v))));
  v = max(v, (int)__float_as_uint(lane_xor<1>(__uint_as_float((unsigned)v))));
  return v;
}

// Sum over a row of 16 lanes, and over the 64 lanes, by xor butterflies (offsets 32, 16, 8, 4, 2, 1).  Addition
// commutes, so every lane ends with the same bits, and the order of additions is the same for every row of every launch.
__device__ __forceinline__ float row16_sum(float v) {
  v += lane_xor<8>(v);
  v += lane_xor<4>(v);
  v += lane_xor<2>(v);
  v += lane_xor<1>(v);
  return v;
}

__device__ __forceinline__ float wave_sum(float v) {
  float a, b;
  lane_halves<32>(v, a, b);
  v = a + b;
  lane_halves<16>(v, a, b);
  v = a + b;
  return row16_sum(v);
}

__device__ __forceinline__ float row16_max(float v) {
  v = fmaxf(v, lane_xor<8>(v));
  v = fmaxf(v, lane_xor<4>(v));
  v = fmaxf(v, lane_xor<2>(v));
  v = fmaxf(v, lane_xor<1>(v));
  return v;
}

__device__ __forceinline__ float wave_max(float v) {
  float a, b;
  lane_halves<32>(v, a, b);
  v = fmaxf(a, b);
  lane_halves<16>(v, a, b);
  v = fmaxf(a, b);
  return row16_max(v);
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

// 4 norm weights (bfloat16 or 32-bit) starting at element 4c: the load leaves the bits as they
// come (8 or 16 bytes), the conversion to floats is a separate step, so that a caller can issue
// all its loads before anything waits for one.
__device__ __forceinline__ u32x4 load_norm_w_raw(const void* __restrict__ w, int is_bf16, int c) {
  if (is_bf16) {
    const u32x2 p = reinterpret_cast<const u32x2*>(w)[c];
    return (u32x4){p[0], p[1], 0u, 0u};
  }
  return reinterpret_cast<const u32x4*>(w)[c];
}

__device__ __forceinline__ f32x4 norm_w_floats(u32x4 raw, int is_bf16) {
  if (is_bf16)
    return (f32x4){__uint_as_float(raw[0] << 16), __uint_as_float(raw[0] & 0xffff0000u), __uint_as_float(raw[1] << 16),
                   __uint_as_float(raw[1] & 0xffff0000u)};
  return (f32x4){__uint_as_float(raw[0]), __uint_as_float(raw[1]), __uint_as_float(raw[2]), __uint_as_float(raw[3])};
}

__device__ __forceinline__ f32x4 load_norm_w4(const void* __restrict__ w, int is_bf16, int c) {
  return norm_w_floats(load_norm_w_raw(w, is_bf16, c), is_bf16);
}

// RMSNorm of up to R rows of at most 256 NV elements (a multiple of 4; NV vectors of four a lane) by one wave, in
// two phases: every load is issued in the first (vector indices past the row are clamped, missing rows read
// the first row, so nothing is conditional), everything is computed in the second.  Between
// them the caller may put other loads in flight: memory results are waited for in issue order,
// so what is issued later does not hold the reductions up.  rows[0] must be a row; rows[j]
// null skips row j.  The order is that of row_sumsq_vec and of the store loop of
// rmsnorm_bf16_kernel: lane l owns vectors l, l+64, ...; ``store(j, c, packed)`` receives vector
// c of row j as four bfloat16 in 8 bytes.
template <int R, int NV = 8>
struct NormRows {
  f32x4 v[R][NV];
  u32x4 w[NV];
};

template <int R, int NV = 8>
__device__ __forceinline__ void norm_rows_load(NormRows<R, NV>& nr, const f32x4* const (&rows)[R], const void* __restrict__ w,
                                               int w_is_bf16, int nvec, int lane) {
#pragma unroll
  for (int j = 0; j < NV; ++j) {
    const int c = norm_vec_index(j, lane, nvec);
    nr.w[j] = load_norm_w_raw(w, w_is_bf16, c);
#pragma unroll
    for (int i = 0; i < R; ++i) nr.v[i][j] = (rows[i] != nullptr ? rows[i] : rows[0])[c];
  }
}

template <int R, int NV = 8, typename Store>
__device__ __forceinline__ void norm_rows_finish(const NormRows<R, NV>& nr, const f32x4* const (&rows)[R], int w_is_bf16,
                                                 int nvec, int dim, float eps, int lane, Store store) {
#pragma unroll
  for (int i = 0; i < R; ++i) {
    if (rows[i] == nullptr) continue;
    float acc = 0.0f;
#pragma unroll
    for (int j = 0; j < NV; ++j) {
      const bool in = norm_vec_in_row(j, lane, nvec);
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const float x = in ? nr.v[i][j][e] : 0.0f;
        acc = fmaf(x, x, acc);
      }
    }
    acc = wave_sum(acc);
    const float inv = 1.0f / sqrtf(acc / (float)dim + eps);
#pragma unroll
    for (int j = 0; j < NV; ++j) {
      const int c = 64 * j + lane;
      if (norm_vec_in_row(j, lane, nvec)) {
        const f32x4 wv = norm_w_floats(nr.w[j], w_is_bf16);
        u32x2 pk = {pack_bf16x2((nr.v[i][j][0] * inv) * wv[0], (nr.v[i][j][1] * inv) * wv[1]),
                    pack_bf16x2((nr.v[i][j][2] * inv) * wv[2], (nr.v[i][j][3] * inv) * wv[3])};
        store(i, c, pk);
      }
    }
  }
}

// One row at once: the whole of rmsnorm_bf16_kernel for rows that fit a wave's registers.
template <int NV = 8, typename Store>
__device__ __forceinline__ void rmsnorm_row_small(const f32x4* __restrict__ xv, const void* __restrict__ w,
                                                  int w_is_bf16, int nvec, int dim, float eps, int lane, Store store) {
  NormRows<1, NV> nr;
  const f32x4* rows[1] = {xv};
  norm_rows_load<1, NV>(nr, rows, w, w_is_bf16, nvec, lane);
  norm_rows_finish<1, NV>(nr, rows, w_is_bf16, nvec, dim, eps, lane, [&](int, int c, u32x2 pk) { store(c, pk); });
}

// The operand of s_waitcnt that waits for all but the last n memory loads of the wave and for nothing else.
constexpr int vmcnt_only(int n) { return 0x0f70 | (n & 15) | ((n >> 4) << 14); }

// The launch wrappers return hipGetLastError() as int; 0 is success.
#define BW_LAUNCH_CHECK() ((int)hipGetLastError())
