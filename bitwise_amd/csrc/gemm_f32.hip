// True 32-bit matrix product: y[m][n] = sum_k x[m][k] * W[n][k], W row-major [N][K].
//
// Every output is ONE fused multiply-add chain over k = 0..K-1 starting from 0.0f, the
// order of the reference's scalar definition (src/kernels.cpp:236-244).  The tiling only
// decides which outputs share a pass over k (64x64 outputs per workgroup, 4x4 per thread,
// k staged through LDS 16 at a time); it never splits K, so a row's bits do not depend on
// the number of rows.  bfloat16 weights are widened exactly (src/kernels.cpp:77-81).
#include "common.h"
#include "api.h"

#define F32_BM 64
#define F32_BN 64
#define F32_BK 16

template <typename WT>
__global__ __launch_bounds__(256) void gemm_f32_kernel(const float* __restrict__ x, const WT* __restrict__ w,
                                                       float* __restrict__ y, int M, int N, int K, int ldx,
                                                       int ldy, int accumulate) {
  __shared__ float xs[F32_BK][F32_BM + 4];
  __shared__ float ws[F32_BK][F32_BN + 4];
  const int tid = threadIdx.x;
  const int tx = tid & 15, ty = tid >> 4;
  const int m0 = blockIdx.y * F32_BM, n0 = blockIdx.x * F32_BN;
  float acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = 0.0f;

  const int lr = tid >> 2;         // 0..63: row of the tile this thread loads
  const int lk = (tid & 3) * 4;    // 0,4,8,12: first of its four k
  for (int k0 = 0; k0 < K; k0 += F32_BK) {
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int k = k0 + lk + q;
      const int m = m0 + lr, n = n0 + lr;
      xs[lk + q][lr] = (m < M && k < K) ? x[(size_t)m * ldx + k] : 0.0f;
      float wv = 0.0f;
      if (n < N && k < K) {
        if constexpr (sizeof(WT) == 2) wv = bf16_to_f32(w[(size_t)n * K + k]);
        else wv = w[(size_t)n * K + k];
      }
      ws[lk + q][lr] = wv;
    }
    __syncthreads();
    const int kend = (K - k0) < F32_BK ? (K - k0) : F32_BK;
    for (int kk = 0; kk < kend; ++kk) {
      float a[4], b[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) a[i] = xs[kk][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) b[j] = ws[kk][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int m = m0 + ty * 4 + i;
    if (m >= M) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + tx * 4 + j;
      if (n >= N) continue;
      float* o = y + (size_t)m * ldy + n;
      *o = accumulate ? (*o + acc[i][j]) : acc[i][j];
    }
  }
}

// Prompt portions: the same chains in tiles of 128x128 outputs, 8x8 per thread (as 2x2 blocks of 4x4, 64 rows
// or columns apart, so that every LDS read is 16 bytes and free of bank conflicts), k staged through LDS 16 at a
// time in two buffers (the next stage's loads fly while this one is worked on; one barrier a stage).
// K a multiple of 16, rows 16-byte aligned.
#define F32T_BM 128
#define F32T_BN 128
#define F32T_BK 16
#define F32T_STR 132            // floats from k to k in LDS

template <typename WT>
__global__ __launch_bounds__(256) void gemm_f32_tile_kernel(const float* __restrict__ x, const WT* __restrict__ w,
                                                            float* __restrict__ y, int M, int N, int K, int ldx,
                                                            int ldy, int accumulate) {
  __shared__ __attribute__((aligned(16))) float xs[2][F32T_BK][F32T_STR];
  __shared__ __attribute__((aligned(16))) float ws[2][F32T_BK][F32T_STR];
  const int tid = threadIdx.x, tx = tid & 15, ty = tid >> 4;
  const int m0 = blockIdx.y * F32T_BM, n0 = blockIdx.x * F32T_BN;
  // loads of a stage: x rows lm and lm + 64, elements 4*lq..; W row wr, elements 8*wh.. (rows past the end are
  // clamped: what they bring is never stored)
  const int lm = tid >> 2, lq = tid & 3, wr = tid >> 1, wh = tid & 1;
  const float* xp0 = x + (size_t)min(m0 + lm, M - 1) * ldx + 4 * lq;
  const float* xp1 = x + (size_t)min(m0 + lm + 64, M - 1) * ldx + 4 * lq;
  const WT* wp = w + (size_t)min(n0 + wr, N - 1) * K + 8 * wh;
  f32x4 xr0, xr1;
  u32x4 wq0, wq1;                                          // bfloat16: 8 elements in wq0; 32-bit: 4 and 4
  auto load_stage = [&](int k0) {
    xr0 = *reinterpret_cast<const f32x4*>(xp0 + k0);
    xr1 = *reinterpret_cast<const f32x4*>(xp1 + k0);
    wq0 = *reinterpret_cast<const u32x4*>(wp + k0);
    if constexpr (sizeof(WT) == 4) wq1 = *reinterpret_cast<const u32x4*>(wp + k0 + 4);
  };
  auto store_stage = [&](int b) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      xs[b][4 * lq + i][lm] = xr0[i];
      xs[b][4 * lq + i][lm + 64] = xr1[i];
    }
    if constexpr (sizeof(WT) == 2) {                       // bfloat16 -> 32-bit: the bits, shifted (exact)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        ws[b][8 * wh + 2 * i][wr] = __uint_as_float(wq0[i] << 16);
        ws[b][8 * wh + 2 * i + 1][wr] = __uint_as_float(wq0[i] & 0xffff0000u);
      }
    } else {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        ws[b][8 * wh + i][wr] = __uint_as_float(wq0[i]);
        ws[b][8 * wh + 4 + i][wr] = __uint_as_float(wq1[i]);
      }
    }
  };
  float acc[8][8];
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[i][j] = 0.0f;
  load_stage(0);
  store_stage(0);
  __syncthreads();
  int b = 0;
  for (int k0 = 0; k0 < K; k0 += F32T_BK) {
    const bool more = k0 + F32T_BK < K;
    if (more) load_stage(k0 + F32T_BK);
#pragma unroll
    for (int kk = 0; kk < F32T_BK; ++kk) {
      const f32x4 a0 = *reinterpret_cast<const f32x4*>(&xs[b][kk][4 * ty]);
      const f32x4 a1 = *reinterpret_cast<const f32x4*>(&xs[b][kk][64 + 4 * ty]);
      const f32x4 b0 = *reinterpret_cast<const f32x4*>(&ws[b][kk][4 * tx]);
      const f32x4 b1 = *reinterpret_cast<const f32x4*>(&ws[b][kk][64 + 4 * tx]);
      const float av[8] = {a0[0], a0[1], a0[2], a0[3], a1[0], a1[1], a1[2], a1[3]};
      const float bv[8] = {b0[0], b0[1], b0[2], b0[3], b1[0], b1[1], b1[2], b1[3]};
#pragma unroll
      for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int j = 0; j < 8; ++j) acc[i][j] = fmaf(av[i], bv[j], acc[i][j]);
    }
    if (more) store_stage(b ^ 1);
    __syncthreads();
    b ^= 1;
  }
  const bool vec = (ldy & 3) == 0 && ((uintptr_t)y & 15) == 0;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int m = m0 + (i < 4 ? 4 * ty + i : 64 + 4 * ty + i - 4);
    if (m >= M) continue;
#pragma unroll
    for (int jh = 0; jh < 2; ++jh) {
      const int n = n0 + 64 * jh + 4 * tx;
      float* o = y + (size_t)m * ldy + n;
      if (vec && n + 3 < N) {
        f32x4 v = {acc[i][4 * jh], acc[i][4 * jh + 1], acc[i][4 * jh + 2], acc[i][4 * jh + 3]};
        if (accumulate) {
          const f32x4 old = *reinterpret_cast<const f32x4*>(o);
          v = (f32x4){old[0] + v[0], old[1] + v[1], old[2] + v[2], old[3] + v[3]};
        }
        *reinterpret_cast<f32x4*>(o) = v;
      } else {
#pragma unroll
        for (int j = 0; j < 4; ++j)
          if (n + j < N) o[j] = accumulate ? (o[j] + acc[i][4 * jh + j]) : acc[i][4 * jh + j];
      }
    }
  }
}

// Up to 64 rows (decoded tokens): the same chains, one per thread and block of 16 rows.  A workgroup owns 16 columns and all rows,
// thread (m, n) the output of row m and column 16 * blockIdx.x + n; its 256 threads together bring 256 elements
// of k of the 16 rows of W and of the rows of x into LDS at a time (16-byte loads; the next stage's loads fly
// while this one is worked on), widened to 32-bit there, and every thread then walks the stage in k order with
// one 16-byte read of its row of W and one of its row of x per four multiply-adds.  Few columns a workgroup,
// so that a product with few outputs still has loads in flight from many compute units.
// K a multiple of 8 (of 4 for 32-bit weights), rows 16-byte aligned.
#define F32R_NB 16

// MR blocks of 16 rows (up to 64 rows): thread (m, n) then runs the chains of rows m, m + 16, ... of its column,
// and a stage is 128 elements of k instead of 256 (the rows of x take LDS).
template <typename WT, int MR>
__global__ __launch_bounds__(256) void gemm_f32_rows_kernel(const float* __restrict__ x, const WT* __restrict__ w,
                                                            float* __restrict__ y, int M, int N, int K, int ldx,
                                                            int ldy, int accumulate) {
  constexpr int F32R_KB = MR == 1 ? 256 : 128;            // elements of k a stage
  constexpr int F32R_STRIDE = F32R_KB + 4;                 // floats from row to row in LDS: 16-byte reads of 16 rows hit 64 different banks
  constexpr int WC = sizeof(WT) == 2 ? 8 : 4;             // elements of W in a 16-byte chunk
  constexpr int WPR = F32R_KB / WC;                        // chunks in a stage's row of W
  constexpr int WJ = F32R_NB * WPR / 256;                  // chunks of W a thread and stage
  constexpr int XJ = 16 * MR * (F32R_KB / 4) / 256;        // chunks of x a thread and stage (16 * MR rows)
  extern __shared__ __attribute__((aligned(16))) float rows_lds[];   // [2][W: 16 rows | x: 16 rows] of F32R_STRIDE
  const int tid = threadIdx.x, n = tid & 15, m = tid >> 4;
  const int n0 = blockIdx.x * F32R_NB;
  // Two stages' loads are in flight while one is worked on: register sets A and B take the even and the odd stages
  // in turn.  Every load is unconditional and inside the operands (rows past N or M and k past K are clamped: what
  // they bring is never used), so that a wait for one set's loads need not be a wait for the other's.
  u32x4 wa[WJ], wb[WJ];
  f32x4 xa[XJ], xb[XJ];
  auto load_stage = [&](int k0, u32x4 (&wreg)[WJ], f32x4 (&xreg)[XJ]) {
#pragma unroll
    for (int j = 0; j < WJ; ++j) {
      const int c = tid + 256 * j, row = min(n0 + c / WPR, N - 1), k = min(k0 + (c % WPR) * WC, K - WC);
      wreg[j] = *reinterpret_cast<const u32x4*>(w + (size_t)row * K + k);
    }
#pragma unroll
    for (int j = 0; j < XJ; ++j) {
      const int c = tid + 256 * j, row = min(c / (F32R_KB / 4), M - 1), k = min(k0 + (c % (F32R_KB / 4)) * 4, K - 4);
      xreg[j] = *reinterpret_cast<const f32x4*>(x + (size_t)row * ldx + k);
    }
  };
  auto store_stage = [&](float* buf, const u32x4 (&wreg)[WJ], const f32x4 (&xreg)[XJ]) {
#pragma unroll
    for (int j = 0; j < WJ; ++j) {
      const int c = tid + 256 * j, row = c / WPR, kk = (c % WPR) * WC;
      float* dst = buf + row * F32R_STRIDE + kk;
      if constexpr (sizeof(WT) == 2) {                     // bfloat16 -> 32-bit: the bits, shifted (exact)
        *reinterpret_cast<u32x4*>(dst) = (u32x4){wreg[j][0] << 16, wreg[j][0] & 0xffff0000u, wreg[j][1] << 16, wreg[j][1] & 0xffff0000u};
        *reinterpret_cast<u32x4*>(dst + 4) = (u32x4){wreg[j][2] << 16, wreg[j][2] & 0xffff0000u, wreg[j][3] << 16, wreg[j][3] & 0xffff0000u};
      } else {
        *reinterpret_cast<u32x4*>(dst) = wreg[j];
      }
    }
#pragma unroll
    for (int j = 0; j < XJ; ++j) {
      const int c = tid + 256 * j, row = c / (F32R_KB / 4), kk = (c % (F32R_KB / 4)) * 4;
      *reinterpret_cast<f32x4*>(buf + (F32R_NB + row) * F32R_STRIDE + kk) = xreg[j];
    }
  };
  constexpr int BUF = (1 + MR) * 16 * F32R_STRIDE;         // floats of one buffer
  float acc = 0.0f;
  float accs[MR];                                          // (MR > 1)
#pragma unroll
  for (int r = 0; r < MR; ++r) accs[r] = 0.0f;
  auto work = [&](const float* buf, int k0) {              // the stage's steps of every chain, k ascending
    const int kend = (K - k0) < F32R_KB ? (K - k0) : F32R_KB;
    if (m >= M || kend <= 0) return;
    const float* wr = buf + n * F32R_STRIDE;
    const float* xr = buf + (F32R_NB + m) * F32R_STRIDE;
    if constexpr (MR > 1) {
#pragma unroll 4
      for (int kk = 0; kk < kend; kk += 4) {
        const f32x4 wv = *reinterpret_cast<const f32x4*>(wr + kk);
#pragma unroll
        for (int r = 0; r < MR; ++r) {
          const f32x4 xv = *reinterpret_cast<const f32x4*>(xr + 16 * r * F32R_STRIDE + kk);   // (rows past M: finite, never stored)
          accs[r] = fmaf(xv[0], wv[0], accs[r]);
          accs[r] = fmaf(xv[1], wv[1], accs[r]);
          accs[r] = fmaf(xv[2], wv[2], accs[r]);
          accs[r] = fmaf(xv[3], wv[3], accs[r]);
        }
      }
      return;
    }
    if (kend == F32R_KB) {
      // a whole stage: blocks of 32 steps, the operands of the next block read from LDS while this block's steps
      // run (the wave has little company on its SIMD: what hides its read latency is its own chain)
      constexpr int BLK = 8, NBLK = F32R_KB / 4 / BLK;
      f32x4 wv[2][BLK], xv[2][BLK];
#pragma unroll
      for (int i = 0; i < BLK; ++i) {
        wv[0][i] = *reinterpret_cast<const f32x4*>(wr + 4 * i);
        xv[0][i] = *reinterpret_cast<const f32x4*>(xr + 4 * i);
      }
#pragma unroll
      for (int blk = 0; blk < NBLK; ++blk) {
        if (blk + 1 < NBLK) {
#pragma unroll
          for (int i = 0; i < BLK; ++i) {
            wv[(blk + 1) & 1][i] = *reinterpret_cast<const f32x4*>(wr + 4 * (BLK * (blk + 1) + i));
            xv[(blk + 1) & 1][i] = *reinterpret_cast<const f32x4*>(xr + 4 * (BLK * (blk + 1) + i));
          }
        }
#pragma unroll
        for (int i = 0; i < BLK; ++i) {
          acc = fmaf(xv[blk & 1][i][0], wv[blk & 1][i][0], acc);
          acc = fmaf(xv[blk & 1][i][1], wv[blk & 1][i][1], acc);
          acc = fmaf(xv[blk & 1][i][2], wv[blk & 1][i][2], acc);
          acc = fmaf(xv[blk & 1][i][3], wv[blk & 1][i][3], acc);
        }
      }
      __builtin_amdgcn_sched_group_barrier(0x100, 2 * BLK, 0);
#pragma unroll
      for (int blk = 0; blk + 1 < NBLK; ++blk) {
        __builtin_amdgcn_sched_group_barrier(0x100, 2 * BLK, 0);
        __builtin_amdgcn_sched_group_barrier(0x002, 4 * BLK, 0);
      }
      __builtin_amdgcn_sched_group_barrier(0x002, 4 * BLK, 0);
      return;
    }
#pragma unroll 8
    for (int kk = 0; kk < kend; kk += 4) {               // (unrolled: the reads of the steps ahead are under way)
      const f32x4 wv = *reinterpret_cast<const f32x4*>(wr + kk);
      const f32x4 xv = *reinterpret_cast<const f32x4*>(xr + kk);
      acc = fmaf(xv[0], wv[0], acc);
      acc = fmaf(xv[1], wv[1], acc);
      acc = fmaf(xv[2], wv[2], acc);
      acc = fmaf(xv[3], wv[3], acc);
    }
  };
  float* buf0 = rows_lds;
  float* buf1 = rows_lds + BUF;
  load_stage(0, wa, xa);
  load_stage(F32R_KB, wb, xb);
  store_stage(buf0, wa, xa);
  __syncthreads();
  for (int k0 = 0; k0 < K; k0 += 2 * F32R_KB) {
    load_stage(k0 + 2 * F32R_KB, wa, xa);
    work(buf0, k0);
    store_stage(buf1, wb, xb);
    __syncthreads();
    load_stage(k0 + 3 * F32R_KB, wb, xb);
    work(buf1, k0 + F32R_KB);
    store_stage(buf0, wa, xa);
    __syncthreads();
  }
  if (n0 + n >= N) return;
#pragma unroll
  for (int r = 0; r < MR; ++r) {
    const int mr = m + 16 * r;
    if (mr >= M) continue;
    float* o = y + (size_t)mr * ldy + n0 + n;
    const float v = MR == 1 ? acc : accs[r];
    *o = accumulate ? (*o + v) : v;
  }
}

template <typename WT, int MR>
static void launch_rows_mr(const float* x, const WT* w, float* y, int M, int N, int K, int ldx, int ldy, int accumulate,
                           hipStream_t s) {
  constexpr int lds_bytes = 2 * (1 + MR) * 16 * ((MR == 1 ? 256 : 128) + 4) * (int)sizeof(float);
  static bool allowed = false;                       // more than 64 KB of dynamic LDS has to be asked for once
  if (!allowed) {
    (void)hipFuncSetAttribute((const void*)gemm_f32_rows_kernel<WT, MR>, hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes);
    allowed = true;
  }
  hipLaunchKernelGGL((gemm_f32_rows_kernel<WT, MR>), dim3((N + F32R_NB - 1) / F32R_NB), dim3(256), lds_bytes, s, x, w, y, M, N, K,
                     ldx, ldy, accumulate);
}

template <typename WT>
static void launch_rows(const float* x, const WT* w, float* y, int M, int N, int K, int ldx, int ldy, int accumulate,
                        hipStream_t s) {
  if (M <= 16) launch_rows_mr<WT, 1>(x, w, y, M, N, K, ldx, ldy, accumulate, s);
  else if (M <= 32) launch_rows_mr<WT, 2>(x, w, y, M, N, K, ldx, ldy, accumulate, s);
  else launch_rows_mr<WT, 4>(x, w, y, M, N, K, ldx, ldy, accumulate, s);
}

extern "C" int bw_gemm_f32(const float* x, const void* w, int w_is_bf16, float* y, int M, int N, int K, int ldx,
                           int ldy, int accumulate, void* stream) {
  if (M <= 0 || N <= 0) return 0;
  if (K <= 0 || ldx < K || ldy < N) return -2;
  dim3 grid((N + F32_BN - 1) / F32_BN, (M + F32_BM - 1) / F32_BM), block(256);
  hipStream_t s = (hipStream_t)stream;
  // which kernel runs depends on the shape alone, and both run the same chains
  const int wc = w_is_bf16 ? 8 : 4;
  if (M <= 64 && K % wc == 0 && ldx % 4 == 0 && ((uintptr_t)x & 15) == 0 && ((uintptr_t)w & 15) == 0) {
    if (w_is_bf16) launch_rows<bf16_t>(x, (const bf16_t*)w, y, M, N, K, ldx, ldy, accumulate, s);
    else launch_rows<float>(x, (const float*)w, y, M, N, K, ldx, ldy, accumulate, s);
    return BW_LAUNCH_CHECK();
  }
  if (M > 64 && K % F32T_BK == 0 && ldx % 4 == 0 && ((uintptr_t)x & 15) == 0 && ((uintptr_t)w & 15) == 0) {
    dim3 tgrid((N + F32T_BN - 1) / F32T_BN, (M + F32T_BM - 1) / F32T_BM);
    if (w_is_bf16)
      hipLaunchKernelGGL(gemm_f32_tile_kernel<bf16_t>, tgrid, block, 0, s, x, (const bf16_t*)w, y, M, N, K, ldx, ldy, accumulate);
    else
      hipLaunchKernelGGL(gemm_f32_tile_kernel<float>, tgrid, block, 0, s, x, (const float*)w, y, M, N, K, ldx, ldy, accumulate);
    return BW_LAUNCH_CHECK();
  }
  if (w_is_bf16)
    hipLaunchKernelGGL(gemm_f32_kernel<bf16_t>, grid, block, 0, s, x, (const bf16_t*)w, y, M, N, K, ldx, ldy, accumulate);
  else
    hipLaunchKernelGGL(gemm_f32_kernel<float>, grid, block, 0, s, x, (const float*)w, y, M, N, K, ldx, ldy, accumulate);
  return BW_LAUNCH_CHECK();
}
