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

// ------------------------------------------------------------------------------ up to 16 rows: a wave a row

// Decoded tokens, the same chains with the operands brought another way.  A workgroup owns 64 columns and all
// (up to 16) rows; wave m is row m, lane l the chain of (row m, column n0 + l).  Weights and rows travel from
// memory straight into LDS (buffer loads with LDS as destination: 8 rows of W, 128 bytes each, or 4 rows of x, 256
// bytes each, an instruction; whole cache lines, the 16-byte chunks of a row of W permuted against bank conflicts;
// a ring of stages, waits by counting loads).  The weights stay packed there: a lane reads its column's 16-byte
// chunks and widens them in registers.  A row's elements are the same for the whole wave: every lane reads the same
// address, which costs LDS one access.  Against the kernel above (every thread reads a 32-bit element of x and one
// of W from LDS for each multiply-add) a multiply-add here needs 2 bytes of W from LDS (bfloat16 weights) instead of
// 4 of W and 4 of x.  For products with at least as many blocks of 64 columns as there are compute units.
// K a multiple of a stage (64 bfloat16 or 32 32-bit elements), rows 16-byte aligned.
#define F32L_MIN_BLOCKS 256                                           // fewer blocks of 64 columns than compute units: the kernel above (16 columns a workgroup)
#define F32L_STAGES 8
#define F32L_W (64 * 128)                                             // 64 rows of W, 128 bytes each
#define F32L_X (16 * 256)                                             // 16 rows of x, up to 64 elements each
#define F32L_STAGE (F32L_W + F32L_X)

// A wave's loads of one stage (a device function rather than a lambda in the kernel: the host pass drops, without a
// word, kernel templates whose lambdas capture arrays of dependent size): LPW of W and one of x.
template <int LPW>
__device__ __forceinline__ void lanes_issue(unsigned char* lds, __amdgpu_buffer_rsrc_t rs_w, __amdgpu_buffer_rsrc_t rs_x, const int* voff,
                                            int voff_x, int wave, int nwaves, int step, int steps, int w_step, int x_step) {
  typedef __attribute__((address_space(3))) void* lds_ptr;
  unsigned char* dst = lds + (step % F32L_STAGES) * F32L_STAGE;
  unsigned char* dump = lds + F32L_STAGES * F32L_STAGE;               // where loads that bring nothing put their zeros
  const bool real = step < steps;                                     // scalar
#pragma unroll
  for (int t = 0; t < LPW; ++t) {
    const int blk = wave + t * nwaves;
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_w, (lds_ptr)(blk < 8 ? dst + blk * 1024 : dump), 16, real ? voff[t] : 0x7ffffff0,
                                             step * w_step, 0, 0);
  }
  __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_x, (lds_ptr)(wave < 4 ? dst + F32L_W + wave * 1024 : dump), 16,
                                           real ? voff_x : 0x7ffffff0, step * x_step, 0, 0);
}

// LPW: loads of W a wave issues per stage (8 in all; waves past the eighth, and what does not divide, issue loads
// outside the descriptor: no traffic, zeros into a spare KB behind the ring), so that every wave counts alike.
template <typename WT, int LPW>
__global__ __launch_bounds__(1024) void gemm_f32_lanes_kernel(const float* __restrict__ x, const WT* __restrict__ w,
                                                              float* __restrict__ y, int M, int N, int K, int ldx, int ldy,
                                                              int accumulate) {
  constexpr int EPC = 16 / (int)sizeof(WT);                           // elements in a 16-byte chunk
  constexpr int KS = 128 / (int)sizeof(WT);                           // elements of k a stage
  extern __shared__ __attribute__((aligned(16))) unsigned char lanes_lds[];   // [stages][W: 64 rows of 128 B | x: 16 rows of 256 B], 1 KB
  const int wave = wave_index(), lane = threadIdx.x & 63, nwaves = blockDim.x >> 6;
  const int n0 = blockIdx.x * 64;
  const int w_rows = min(64, N - n0);
  const __amdgpu_buffer_rsrc_t rs_w = __builtin_amdgcn_make_buffer_rsrc((void*)(w + (size_t)n0 * K), 0,
                                                                        (int)((size_t)w_rows * K * sizeof(WT)), 0x00020000);
  const __amdgpu_buffer_rsrc_t rs_x = __builtin_amdgcn_make_buffer_rsrc((void*)x, 0, (int)((((size_t)M - 1) * ldx + K) * 4), 0x00020000);
  // loads of W: lane l of a load fetches row l / 8 of its 8 rows, chunk (l % 8) ^ (row within 16 >> 1) of the row's 128 bytes
  const int lrow = lane >> 3, lslot = lane & 7;
  int voff[LPW];
#pragma unroll
  for (int t = 0; t < LPW; ++t) {
    const int blk = wave + t * nwaves;                                // which 8 rows of the 64
    const int row = 8 * blk + lrow;
    voff[t] = blk < 8 ? (int)((row * K) * (int)sizeof(WT) + 16 * (lslot ^ ((row & 15) >> 1))) : 0x7ffffff0;
  }
  // loads of x (waves 0 to 3): lane l fetches row 4 wave + l / 16, its chunk l % 16 of the stage's KS elements (rows
  // past M and, with 32-bit weights, chunks past the stage: outside, or never read)
  const int xrow = 4 * wave + (lane >> 4), xchunk = lane & 15;
  const int voff_x = (wave < 4 && xrow < M && 4 * xchunk < KS) ? (xrow * ldx + 4 * xchunk) * 4 : 0x7ffffff0;
  const int steps = K / KS;
#pragma unroll
  for (int st = 0; st < F32L_STAGES - 1; ++st) lanes_issue<LPW>(lanes_lds, rs_w, rs_x, voff, voff_x, wave, nwaves, st, steps, 128, KS * 4);
  // this lane's row of the tile: chunk j lies in slot j ^ (row within 16 >> 1)
  const int my = (lane >> 3) * 1024 + (lane & 7) * 128, swz = (lane & 15) >> 1;
  float acc = 0.0f;
  for (int step = 0; step < steps; ++step) {
    __builtin_amdgcn_s_waitcnt(vmcnt_only((LPW + 1) * (F32L_STAGES - 2)));   // all but the loads of the stages after this one have landed
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    lanes_issue<LPW>(lanes_lds, rs_w, rs_x, voff, voff_x, wave, nwaves, step + F32L_STAGES - 1, steps, 128, KS * 4);   // into the stage worked on a step ago
    const unsigned char* stage = lanes_lds + (step % F32L_STAGES) * F32L_STAGE;
    const unsigned char* xs = stage + F32L_W + wave * 256;            // the wave's row: the same address in every lane
    u32x4 v[8];                                                       // the stage's eight chunks of W, asked for at once
    f32x4 xv[KS / 4];
#pragma unroll
    for (int j = 0; j < 8; ++j) v[j] = *reinterpret_cast<const u32x4*>(stage + my + ((j ^ swz) * 16));
#pragma unroll
    for (int j = 0; j < KS / 4; ++j) xv[j] = *reinterpret_cast<const f32x4*>(xs + 16 * j);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      if constexpr (sizeof(WT) == 2) {                                // bfloat16 -> 32-bit: the bits, shifted (exact)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          acc = fmaf(xv[2 * j + (e >> 1)][2 * (e & 1)], __uint_as_float(v[j][e] << 16), acc);
          acc = fmaf(xv[2 * j + (e >> 1)][2 * (e & 1) + 1], __uint_as_float(v[j][e] & 0xffff0000u), acc);
        }
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e) acc = fmaf(xv[j][e], __uint_as_float(v[j][e]), acc);
      }
    }
    asm volatile("" ::: "memory");
  }
  __builtin_amdgcn_s_waitcnt(vmcnt_only(0));                          // the padding loads too, before the wave ends
  const int n = n0 + lane;
  if (n >= N) return;
  float* o = y + (size_t)wave * ldy + n;
  *o = accumulate ? (*o + acc) : acc;
}

template <typename WT, int LPW>
static void launch_lanes_lpw(const float* x, const WT* w, float* y, int M, int N, int K, int ldx, int ldy, int accumulate,
                             hipStream_t s) {
  constexpr int lds_bytes = F32L_STAGES * F32L_STAGE + 1024;
  static_assert((LPW + 1) * (F32L_STAGES - 2) < 64, "the wait count has six bits");
  static bool allowed = false;                       // 64 KB of dynamic LDS and more has to be asked for once
  if (!allowed) {
    (void)hipFuncSetAttribute((const void*)gemm_f32_lanes_kernel<WT, LPW>, hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes);
    allowed = true;
  }
  hipLaunchKernelGGL((gemm_f32_lanes_kernel<WT, LPW>), dim3((N + 63) / 64), dim3(64 * M), lds_bytes, s, x, w, y, M, N, K, ldx, ldy,
                     accumulate);
}

template <typename WT>
static void launch_lanes(const float* x, const WT* w, float* y, int M, int N, int K, int ldx, int ldy, int accumulate,
                         hipStream_t s) {
  switch ((8 + M - 1) / M) {                         // loads a wave and stage: 8 over the waves, rounded up
    case 8: launch_lanes_lpw<WT, 8>(x, w, y, M, N, K, ldx, ldy, accumulate, s); break;
    case 4: launch_lanes_lpw<WT, 4>(x, w, y, M, N, K, ldx, ldy, accumulate, s); break;
    case 3: launch_lanes_lpw<WT, 3>(x, w, y, M, N, K, ldx, ldy, accumulate, s); break;
    case 2: launch_lanes_lpw<WT, 2>(x, w, y, M, N, K, ldx, ldy, accumulate, s); break;
    default: launch_lanes_lpw<WT, 1>(x, w, y, M, N, K, ldx, ldy, accumulate, s); break;
  }
}

// ------------------------------------------------------------------------------ a wave a row, the row four elements a register

// Decoded tokens once more: a wave is a row and 64 columns, lane l the chain of (row, column n0 + l), weights and
// rows in an LDS ring as above (weights packed).  What is new is how a row's elements reach the multiply-adds.
// x[row][k] is the same number for every lane of the wave; read as such from LDS it costs what any read costs (LDS
// returns 128 bytes a clock whatever the addresses: above, the rows took two thirds of what LDS returned).  Here lane
// l reads the 16 bytes at element 4 * (l % 4) of a run of sixteen, so that a register holds four elements of the row,
// the same four in every quad of lanes, and the multiply-add picks its element with the quad permutation of its
// first operand (v_fmac_f32 with quad_perm [i,i,i,i]: the same fused multiply-add, the operand routed on the way
// in): sixteen elements a read instead of four.
// A workgroup is 64 columns and all rows (a chain wave a row, sharing the ring).  A block is 64 bytes of a row of W
// (four 16-byte chunks: 32 bfloat16 or 16 32-bit elements), a stage two blocks; the next block's operands are read
// from LDS while this block's chains run.  (A chain is bound by its own links: a multiply-add that waits for the one
// before it issues every 3.8 ns, and 5.3 ns with one other vector instruction a link, such as the widening of a
// bfloat16 weight, wherever that instruction stands.)
#define F32C_W (64 * 128)                                             // 64 rows of W, 128 bytes each
#define F32C_X (8 * 256)                                              // 8 rows of x, up to 64 elements each
#define F32C_STAGE (F32C_W + F32C_X)

template <int KB>
struct ChainBlock {
  f32x4 x[KB / 16];                                                   // register j of x[a]: element 16 a + 4 (lane % 4) + j of the block
  u32x4 w[4];
};

template <typename WT>
__device__ __forceinline__ void chain_read(ChainBlock<64 / (int)sizeof(WT)>& b, const unsigned char* stage, int half, int my, int swz,
                                           const unsigned char* xs) {
  constexpr int KB = 64 / (int)sizeof(WT);
#pragma unroll
  for (int a = 0; a < KB / 16; ++a) b.x[a] = *reinterpret_cast<const f32x4*>(xs + (half * KB + 16 * a) * 4);
#pragma unroll
  for (int j = 0; j < 4; ++j) b.w[j] = *reinterpret_cast<const u32x4*>(stage + my + (((4 * half + j) ^ swz) * 16));
}

// acc = fma(x of quad lane I, w, acc): v_fmac_f32 with its first operand routed through the quad permutation
// [I,I,I,I] (written out: the compiler keeps a move of its own in front of the multiply-add otherwise, which costs
// what the multiply-add costs).  The operand comes from an LDS read, never from a vector instruction just before
// (which would want two idle states in between).
template <int I>
__device__ __forceinline__ float fma_quad(float xq, float w, float acc) {
  static_assert(I >= 0 && I < 4, "a quad has four lanes");
  if constexpr (I == 0) asm("v_fmac_f32_dpp %0, %1, %2 quad_perm:[0,0,0,0] row_mask:0xf bank_mask:0xf" : "+v"(acc) : "v"(xq), "v"(w));
  else if constexpr (I == 1) asm("v_fmac_f32_dpp %0, %1, %2 quad_perm:[1,1,1,1] row_mask:0xf bank_mask:0xf" : "+v"(acc) : "v"(xq), "v"(w));
  else if constexpr (I == 2) asm("v_fmac_f32_dpp %0, %1, %2 quad_perm:[2,2,2,2] row_mask:0xf bank_mask:0xf" : "+v"(acc) : "v"(xq), "v"(w));
  else asm("v_fmac_f32_dpp %0, %1, %2 quad_perm:[3,3,3,3] row_mask:0xf bank_mask:0xf" : "+v"(acc) : "v"(xq), "v"(w));
  return acc;
}

// element k of the block: register k % 4 of x[k / 16], quad lane (k / 4) % 4
template <int K16>
__device__ __forceinline__ float chain_step(float acc, const f32x4& x, float w) {
  constexpr int I = (K16 >> 2) & 3, J = K16 & 3;
  return fma_quad<I>(x[J], w, acc);
}

// Element e of 16-byte chunk ``c`` as a 32-bit float (bfloat16: the bits, shifted: exact).
template <typename WT, int E>
__device__ __forceinline__ float chain_weight(const u32x4& c) {
  if constexpr (sizeof(WT) == 2) return __uint_as_float((E & 1) ? (c[E >> 1] & 0xffff0000u) : (c[E >> 1] << 16));
  else return __uint_as_float(c[E]);
}

// The block's chains.  A multiply-add that depends on the one before it can issue every other slot, and one whose
// weight was widened in the slot before it waits for that as well: so chunk j + 1 is widened between the multiply-adds
// of chunk j (``f`` comes in with the block's chunk 0 widened, and leaves with chunk 0 of the next block).
template <typename WT>
__device__ __forceinline__ float chain_run(float acc, const ChainBlock<64 / (int)sizeof(WT)>& b, const ChainBlock<64 / (int)sizeof(WT)>& nxt,
                                           float (&f)[16 / (int)sizeof(WT)]) {
  constexpr int EPC = 16 / (int)sizeof(WT);                           // elements a chunk
  float g[EPC];
#define BW_CHAIN_STEP(J, E, FROM, TO, SRC)                                                \
  TO[E] = chain_weight<WT, E>(SRC);                                                       \
  acc = chain_step<(EPC * J + E) & 15>(acc, b.x[(EPC * J + E) >> 4], FROM[E]);
#define BW_CHAIN_CHUNK(J, FROM, TO, SRC)                                                  \
  BW_CHAIN_STEP(J, 0, FROM, TO, SRC) BW_CHAIN_STEP(J, 1, FROM, TO, SRC) BW_CHAIN_STEP(J, 2, FROM, TO, SRC) BW_CHAIN_STEP(J, 3, FROM, TO, SRC) \
  if constexpr (EPC == 8) {                                                               \
    BW_CHAIN_STEP(J, (EPC == 8 ? 4 : 0), FROM, TO, SRC) BW_CHAIN_STEP(J, (EPC == 8 ? 5 : 1), FROM, TO, SRC)                                   \
    BW_CHAIN_STEP(J, (EPC == 8 ? 6 : 2), FROM, TO, SRC) BW_CHAIN_STEP(J, (EPC == 8 ? 7 : 3), FROM, TO, SRC)                                   \
  }
  BW_CHAIN_CHUNK(0, f, g, b.w[1])
  BW_CHAIN_CHUNK(1, g, f, b.w[2])
  BW_CHAIN_CHUNK(2, f, g, b.w[3])
  BW_CHAIN_CHUNK(3, g, f, nxt.w[0])
#undef BW_CHAIN_CHUNK
#undef BW_CHAIN_STEP
  return acc;
}

template <typename WT>
__device__ __forceinline__ void chain_first(const ChainBlock<64 / (int)sizeof(WT)>& b, float (&f)[16 / (int)sizeof(WT)]) {
  f[0] = chain_weight<WT, 0>(b.w[0]);
  f[1] = chain_weight<WT, 1>(b.w[0]);
  f[2] = chain_weight<WT, 2>(b.w[0]);
  f[3] = chain_weight<WT, 3>(b.w[0]);
  if constexpr (sizeof(WT) == 2) {
    f[4] = chain_weight<WT, 4>(b.w[0]);
    f[5] = chain_weight<WT, 5>(b.w[0]);
    f[6] = chain_weight<WT, 6>(b.w[0]);
    f[7] = chain_weight<WT, 7>(b.w[0]);
  }
}

// The loads are not the chain waves' business.  A buffer load with LDS as destination holds the wave that issues it
// for some hundred clocks (ten of them a stage were more than the stage's chains), so a workgroup has two waves more
// that do nothing else: they ask for the stages, wait for them and meet the chain waves at the stage's barrier.  A
// loader issues five loads a stage: the ten are the eight blocks of 8 rows of W and two blocks of 4 rows of x,
// dealt in turn (loads for rows the workgroup does not have go outside the descriptor: no traffic, zeros into a
// spare KB behind the ring, so that both loaders count alike).
#define F32C_LOADERS 2
#define F32C_LPL 5                                                    // loads a loader and stage

template <int STAGES>
__device__ __forceinline__ void chain_issue(unsigned char* lds, __amdgpu_buffer_rsrc_t rs_w, __amdgpu_buffer_rsrc_t rs_x, const int* voff,
                                            int loader, int step, int steps, int x_step) {
  typedef __attribute__((address_space(3))) void* lds_ptr;
  unsigned char* dst = lds + (step % STAGES) * F32C_STAGE;
  const bool real = step < steps;                                     // scalar
#pragma unroll
  for (int t = 0; t < F32C_LPL; ++t) {
    const int q = loader + F32C_LOADERS * t;                          // 0..7: W; 8, 9: x
    if (q < 8) __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_w, (lds_ptr)(dst + q * 1024), 16, real ? voff[t] : 0x7ffffff0, step * 128, 0, 0);
    else __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_x, (lds_ptr)(dst + F32C_W + (q - 8) * 1024), 16, real ? voff[t] : 0x7ffffff0,
                                                  step * x_step, 0, 0);
  }
}

template <typename WT, int STAGES>
__global__ __launch_bounds__(64 * (8 + F32C_LOADERS)) void gemm_f32_chain_kernel(const float* __restrict__ x, const WT* __restrict__ w,
                                                                                 float* __restrict__ y, int M, int N, int K, int ldx,
                                                                                 int ldy, int accumulate) {
  constexpr int KB = 64 / (int)sizeof(WT);                            // elements of k a block
  extern __shared__ __attribute__((aligned(16))) unsigned char chain_lds[];   // [stages][W: 64 rows of 128 B | x: 8 rows of 256 B]
  const int wave = wave_index(), lane = threadIdx.x & 63, rw = (int)(blockDim.x >> 6) - F32C_LOADERS;
  const int n0 = blockIdx.x * 64;
  const int m0 = blockIdx.y * rw;                                     // the workgroup's first row
  const int steps = K / (2 * KB);
  if (wave >= rw) {
    // ---- a loader
    const int loader = wave - rw;
    const int w_rows = min(64, N - n0), x_rows = min(rw, M - m0);
    const __amdgpu_buffer_rsrc_t rs_w = __builtin_amdgcn_make_buffer_rsrc((void*)(w + (size_t)n0 * K), 0,
                                                                          (int)((size_t)w_rows * K * sizeof(WT)), 0x00020000);
    const __amdgpu_buffer_rsrc_t rs_x = __builtin_amdgcn_make_buffer_rsrc((void*)(x + (size_t)m0 * ldx), 0,
                                                                          (int)((((size_t)x_rows - 1) * ldx + K) * 4), 0x00020000);
    // W: lane l of a load fetches row l / 8 of its 8 rows, chunk (l % 8) ^ (row within 16 >> 1) of the row's 128 bytes;
    // x: lane l fetches row 4 (q - 8) + l / 16 of the workgroup's, chunk l % 16 of the stage's elements (with 32-bit
    // weights a stage is 32 elements: the chunks past them lie outside)
    int voff[F32C_LPL];
#pragma unroll
    for (int t = 0; t < F32C_LPL; ++t) {
      const int q = loader + F32C_LOADERS * t;
      if (q < 8) {
        const int r = 8 * q + (lane >> 3);
        voff[t] = (int)((r * K) * (int)sizeof(WT) + 16 * ((lane & 7) ^ ((r & 15) >> 1)));
      } else {
        const int xrow = 4 * (q - 8) + (lane >> 4), xchunk = lane & 15;
        voff[t] = (xrow < x_rows && 4 * xchunk < 2 * KB) ? (xrow * ldx + 4 * xchunk) * 4 : 0x7ffffff0;
      }
    }
#pragma unroll
    for (int st = 0; st < STAGES - 1; ++st) chain_issue<STAGES>(chain_lds, rs_w, rs_x, voff, loader, st, steps, 2 * KB * 4);
    for (int step = 0; step < steps; ++step) {
      // this stage and the next have landed (the next stage's first block is read during this one's second); behind
      // the barrier every chain wave is done with the stage before, which the new loads overwrite
      __builtin_amdgcn_s_waitcnt(vmcnt_only(F32C_LPL * (STAGES - 3)));
      __builtin_amdgcn_s_barrier();
      asm volatile("" ::: "memory");
      chain_issue<STAGES>(chain_lds, rs_w, rs_x, voff, loader, step + STAGES - 1, steps, 2 * KB * 4);
    }
    __builtin_amdgcn_s_waitcnt(vmcnt_only(0));                        // the padding loads too, before the wave ends
    return;
  }
  // ---- a chain wave: row m0 + wave
  const int row = m0 + wave;
  // this lane's row of the tile: chunk j lies in slot j ^ (row within 16 >> 1); its four elements of the wave's row
  const int my = (lane >> 3) * 1024 + (lane & 7) * 128, swz = (lane & 15) >> 1;
  const int mine = F32C_W + wave * 256 + (lane & 3) * 16;
  ChainBlock<KB> even, odd;
  float f[16 / (int)sizeof(WT)];                                      // a chunk of W, widened
  float acc = 0.0f;
  for (int step = 0; step < steps; ++step) {
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    const unsigned char* stage = chain_lds + (step % STAGES) * F32C_STAGE;
    const unsigned char* next = chain_lds + ((step + 1) % STAGES) * F32C_STAGE;
    if (step == 0) {
      chain_read<WT>(even, stage, 0, my, swz, stage + mine);
      chain_first<WT>(even, f);
    }
    __builtin_amdgcn_sched_barrier(0);
    chain_read<WT>(odd, stage, 1, my, swz, stage + mine);
    __builtin_amdgcn_sched_barrier(0);
    acc = chain_run<WT>(acc, even, odd, f);
    __builtin_amdgcn_sched_barrier(0);
    chain_read<WT>(even, next, 0, my, swz, next + mine);              // (past the last stage: whatever the ring holds, unused)
    __builtin_amdgcn_sched_barrier(0);
    acc = chain_run<WT>(acc, odd, even, f);
    __builtin_amdgcn_sched_barrier(0);
    asm volatile("" ::: "memory");
  }
  const int n = n0 + lane;
  if (n >= N || row >= M) return;
  float* o = y + (size_t)row * ldy + n;
  *o = accumulate ? (*o + acc) : acc;
}

// For products with at least as many blocks of 64 columns as there are compute units and up to 8 rows: a workgroup
// a block of columns with all the rows (there it is faster than the kernels above: gate|up of 16,384 columns
// at 8 rows 26.6 us against 29.1, a head of 49,152 columns 65 against 85; with fewer columns a chain wave has a
// compute unit to itself in either kernel and both take what the chain takes).
#define F32C_STAGES 7
#define F32C_MAX_ROWS 8

template <typename WT>
static void launch_chain(const float* x, const WT* w, float* y, int M, int N, int K, int ldx, int ldy, int accumulate, hipStream_t s) {
  constexpr int lds_bytes = F32C_STAGES * F32C_STAGE + 1024;
  static_assert(F32C_LPL * (F32C_STAGES - 3) < 64, "the wait count has six bits");
  static_assert(F32C_LPL * F32C_LOADERS == 10, "eight loads of W and two of x a stage");
  static bool allowed = false;                       // 64 KB of dynamic LDS and more has to be asked for once
  if (!allowed) {
    (void)hipFuncSetAttribute((const void*)gemm_f32_chain_kernel<WT, F32C_STAGES>, hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes);
    allowed = true;
  }
  int rw = 1;
  while (rw < M) rw *= 2;                            // (1, 2, 4 or 8 chain waves)
  hipLaunchKernelGGL((gemm_f32_chain_kernel<WT, F32C_STAGES>), dim3((N + 63) / 64, 1), dim3(64 * (rw + F32C_LOADERS)), lds_bytes, s, x, w, y,
                     M, N, K, ldx, ldy, accumulate);
}

// ------------------------------------------------------------------------------ up to 64 rows on the matrix cores

// v_mfma_f32_4x4x1_16b_f32 computes, for 16 blocks of 4 x 4 outputs at once, D[r][j] = fma(A[r], B[j], D[r][j]):
// one step of k, a true 32-bit fused multiply-add with a single rounding (denormal numbers, infinities and all;
// the tests hold it against std::fma bit for bit).  A chain of them over k ascending from a zero accumulator is
// therefore the scalar chain of the definition, and it needs one element of x and one of W a lane and step where
// the vector unit needs one of each per output: the operands' way through LDS no longer bounds the product.
//
// A wave owns 4 * CG columns and up to 16 rows (MR such blocks of rows for up to 64): block (rg, cg) of the
// instruction is rows 4 rg .. 4 rg + 3 of x against columns 4 cg .. 4 cg + 3 of the wave's, RG row groups times
// CG = 16 / RG column groups; the blocks of a row group share their A operand (the instruction broadcasts it from
// the group's first block).  Lane (block, i) holds row 4 rg + i of x as A, column 4 cg + i of W as B, and the
// outputs of rows 4 rg .. 4 rg + 3 at its column.  Both operands stream through a ring in LDS that is the wave's
// own (buffer loads with LDS as destination, in whole 128-byte or 256-byte runs, the 16-byte chunks of a row
// permuted so that operand reads hit distinct banks; bfloat16 weights are widened when they are read).  Nothing is
// shared between waves, so the loop has no barrier; loads complete in issue order and every stage has the same
// number of them (stages past K are asked for outside the descriptors: zeros, no traffic), so "all but the last
// PENDING loads have landed" is the wait for the stage at hand.  K a multiple of 64.
template <typename WT, int RG, int MR>
struct F32MShape {
  static constexpr int CG = 16 / RG, NCW = 4 * CG;                  // column groups, columns a wave
  static constexpr int CBSZ = RG == 1 ? 4 : (RG == 2 ? 3 : 2);      // log2 of the blocks that share an A operand
  static constexpr int XROWS = 4 * RG * MR;                         // rows of x a stage holds
  static constexpr int WROW = 64 * (int)sizeof(WT);                 // bytes of a row of W a stage (64 steps of k)
  static constexpr int X_LOADS = XROWS / 4, W_LOADS = NCW * WROW / 1024;   // 1 KB an instruction
  static constexpr int LPW = X_LOADS + W_LOADS;
  static constexpr int XBYTES = XROWS * 256, STAGE = XBYTES + NCW * WROW;
  static constexpr int BY_COUNT = 63 / LPW + 2, BY_ROOM = 65536 / STAGE;
  static constexpr int STAGES = BY_COUNT < BY_ROOM ? (BY_COUNT < 12 ? BY_COUNT : 12) : (BY_ROOM < 12 ? BY_ROOM : 12);
  static constexpr int PENDING = LPW * (STAGES - 2);
  static_assert(STAGES >= 3 && PENDING < 64, "the ring needs three stages and the wait count has six bits");
  static_assert(MR == 1 || RG == 4, "more than 16 rows: blocks of 16");
};

template <typename WT, int RG, int MR>
__device__ __forceinline__ void f32m_issue(unsigned char* ring, __amdgpu_buffer_rsrc_t rs_x, __amdgpu_buffer_rsrc_t rs_w,
                                           const int* voff_x, const int* voff_w, int step, int steps) {
  using S = F32MShape<WT, RG, MR>;
  typedef __attribute__((address_space(3))) void* lds_ptr;
  unsigned char* dst = ring + (step % S::STAGES) * S::STAGE;
  const bool real = step < steps;                                  // scalar
#pragma unroll
  for (int t = 0; t < S::X_LOADS; ++t)
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_x, (lds_ptr)(dst + t * 1024), 16, real ? voff_x[t] : 0x7ffffff0, step * 256, 0, 0);
#pragma unroll
  for (int t = 0; t < S::W_LOADS; ++t)
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_w, (lds_ptr)(dst + S::XBYTES + t * 1024), 16, real ? voff_w[t] : 0x7ffffff0,
                                             step * S::WROW, 0, 0);
}

template <typename WT, int RG, int MR>
__global__ __launch_bounds__(64) void gemm_f32_mfma_kernel(const float* __restrict__ x, const WT* __restrict__ w,
                                                           float* __restrict__ y, int M, int N, int K, int ldx, int ldy,
                                                           int accumulate) {
  using S = F32MShape<WT, RG, MR>;
  constexpr bool BF = sizeof(WT) == 2;
  extern __shared__ __attribute__((aligned(16))) unsigned char f32m_ring[];
  const int lane = threadIdx.x, blk = lane >> 2, i = lane & 3;
  const int rg = blk / S::CG, cg = blk % S::CG;
  const int n0 = blockIdx.x * S::NCW;
  const int w_rows = min(S::NCW, N - n0);
  const __amdgpu_buffer_rsrc_t rs_w =
      __builtin_amdgcn_make_buffer_rsrc((void*)(w + (size_t)n0 * K), 0, (int)((size_t)w_rows * K * sizeof(WT)), 0x00020000);
  const __amdgpu_buffer_rsrc_t rs_x =
      __builtin_amdgcn_make_buffer_rsrc((void*)x, 0, (int)((((size_t)M - 1) * ldx + K) * sizeof(float)), 0x00020000);
  // loads: an instruction brings 1 KB: 4 rows of x (16 chunks of 4 elements each), 8 rows of bfloat16 weights (8 chunks
  // of 8 elements) or 4 rows of 32-bit ones; the lane that fills slot s of a row fetches chunk s ^ (row % 8).  Rows
  // past M or N are clamped to the last: what they bring ends in outputs that are never stored.
  int voff_x[S::X_LOADS], voff_w[S::W_LOADS];
#pragma unroll
  for (int t = 0; t < S::X_LOADS; ++t) {
    const int row = 4 * t + (lane >> 4), chunk = (lane & 15) ^ (row & 7);
    voff_x[t] = (min(row, M - 1) * ldx + 4 * chunk) * 4;
  }
#pragma unroll
  for (int t = 0; t < S::W_LOADS; ++t) {
    if constexpr (BF) {
      const int row = 8 * t + (lane >> 3), chunk = (lane & 7) ^ (row & 7);
      voff_w[t] = (min(row, w_rows - 1) * K + 8 * chunk) * 2;
    } else {
      const int row = 4 * t + (lane >> 4), chunk = (lane & 15) ^ (row & 7);
      voff_w[t] = (min(row, w_rows - 1) * K + 4 * chunk) * 4;
    }
  }
  // operand reads: this lane's row of x in every block of 16 rows, and its column's row of W
  int x_base[MR], x_swz[MR];
#pragma unroll
  for (int mr = 0; mr < MR; ++mr) {
    const int row = 16 * mr + 4 * rg + i;
    x_base[mr] = row * 256;
    x_swz[mr] = row & 7;
  }
  const int wr = 4 * cg + i;
  const int w_base = S::XBYTES + wr * S::WROW, w_swz = wr & 7;
  f32x4 acc[MR];
#pragma unroll
  for (int mr = 0; mr < MR; ++mr) acc[mr] = (f32x4){0.f, 0.f, 0.f, 0.f};
  const int steps = K / 64;
  // A stage is worked on in PH phases of CH chunks of 8 steps of k.  The operands of a phase are read from LDS
  // into one of two sets of registers while the phase before runs out of the other: an LDS read takes longer than
  // the few matrix instructions the compiler would put between it and its use.
  constexpr int CH = MR == 4 ? 2 : 4, PH = 8 / CH;
  constexpr int WQ = BF ? CH : 2 * CH;                              // 16-byte reads of W a phase
  u32x4 w_a[WQ], w_b[WQ];
  f32x4 x_a[MR][2 * CH], x_b[MR][2 * CH];
  auto read_phase = [&](const unsigned char* stage, int ph, u32x4 (&wq)[WQ], f32x4 (&xq)[MR][2 * CH]) {
#pragma unroll
    for (int c = 0; c < WQ; ++c) wq[c] = *reinterpret_cast<const u32x4*>(stage + w_base + (((ph * WQ + c) ^ w_swz) * 16));
#pragma unroll
    for (int c = 0; c < 2 * CH; ++c)
#pragma unroll
      for (int mr = 0; mr < MR; ++mr)
        xq[mr][c] = *reinterpret_cast<const f32x4*>(stage + x_base[mr] + (((ph * 2 * CH + c) ^ x_swz[mr]) * 16));
  };
  auto run_phase = [&](const u32x4 (&wq)[WQ], const f32x4 (&xq)[MR][2 * CH]) {
#pragma unroll
    for (int c = 0; c < CH; ++c) {
      float wv[8];
      if constexpr (BF) {                                           // bfloat16 -> 32-bit: the bits, shifted (exact)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          wv[2 * q] = __uint_as_float(wq[c][q] << 16);
          wv[2 * q + 1] = __uint_as_float(wq[c][q] & 0xffff0000u);
        }
      } else {
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          wv[q] = __uint_as_float(wq[2 * c][q]);
          wv[4 + q] = __uint_as_float(wq[2 * c + 1][q]);
        }
      }
#pragma unroll
      for (int e = 0; e < 8; ++e)                                   // k ascending
#pragma unroll
        for (int mr = 0; mr < MR; ++mr)
          acc[mr] = __builtin_amdgcn_mfma_f32_4x4x1f32(xq[mr][2 * c + (e >> 2)][e & 3], wv[e], acc[mr], S::CBSZ, 0, 0);
    }
  };
#pragma unroll
  for (int st = 0; st < S::STAGES - 1; ++st) f32m_issue<WT, RG, MR>(f32m_ring, rs_x, rs_w, voff_x, voff_w, st, steps);
  __builtin_amdgcn_s_waitcnt(vmcnt_only(S::PENDING));                // stage 0 has landed
  asm volatile("" ::: "memory");
  read_phase(f32m_ring, 0, w_a, x_a);
  for (int step = 0; step < steps; ++step) {
    const unsigned char* stage = f32m_ring + (step % S::STAGES) * S::STAGE;
    const unsigned char* next = f32m_ring + ((step + 1) % S::STAGES) * S::STAGE;
    // stage step - 1 has been read (its last phase was read a phase ago): it may be asked for again
    asm volatile("" ::: "memory");
    f32m_issue<WT, RG, MR>(f32m_ring, rs_x, rs_w, voff_x, voff_w, step + S::STAGES - 1, steps);
#pragma unroll
    for (int ph = 0; ph < PH; ph += 2) {
      read_phase(stage, ph + 1, w_b, x_b);
      __builtin_amdgcn_sched_barrier(0);
      run_phase(w_a, x_a);
      __builtin_amdgcn_sched_barrier(0);
      if (ph + 2 < PH) {
        read_phase(stage, ph + 2, w_a, x_a);
      } else {
        __builtin_amdgcn_s_waitcnt(vmcnt_only(S::PENDING));          // the next stage has landed (past K: zeros, unused)
        asm volatile("" ::: "memory");
        read_phase(next, 0, w_a, x_a);
      }
      __builtin_amdgcn_sched_barrier(0);
      run_phase(w_b, x_b);
      __builtin_amdgcn_sched_barrier(0);
    }
  }
  __builtin_amdgcn_s_waitcnt(vmcnt_only(0));                       // the padding loads too, before the wave ends
  const int n = n0 + 4 * cg + i;
  if (n >= N) return;
#pragma unroll
  for (int mr = 0; mr < MR; ++mr)
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int m = 16 * mr + 4 * rg + r;
      if (m >= M) continue;
      float* o = y + (size_t)m * ldy + n;
      *o = accumulate ? (*o + acc[mr][r]) : acc[mr][r];
    }
}

template <typename WT, int RG, int MR>
static void launch_f32_mfma(const float* x, const WT* w, float* y, int M, int N, int K, int ldx, int ldy, int accumulate,
                            hipStream_t s) {
  using S = F32MShape<WT, RG, MR>;
  hipLaunchKernelGGL((gemm_f32_mfma_kernel<WT, RG, MR>), dim3((N + S::NCW - 1) / S::NCW), dim3(64), S::STAGES * S::STAGE, s, x, w,
                     y, M, N, K, ldx, ldy, accumulate);
}

template <typename WT>
static void launch_f32_mfma_rows(const float* x, const WT* w, float* y, int M, int N, int K, int ldx, int ldy, int accumulate,
                                 hipStream_t s) {
  if (M <= 32) launch_f32_mfma<WT, 4, 2>(x, w, y, M, N, K, ldx, ldy, accumulate, s);
  else launch_f32_mfma<WT, 4, 4>(x, w, y, M, N, K, ldx, ldy, accumulate, s);
}

// ------------------------------------------------------------------------------ prompt portions on the matrix cores

// Tiles of 128 x 128 outputs, four waves of 64 x 64.  v_mfma_f32_32x32x1_2b_f32 is one step of k for two blocks of
// 32 x 32 outputs: D[i][j] = fma(A[i], B[j], D[i][j]), the same single-rounding multiply-add as above; with the A
// operand of the first block broadcast to the second, an instruction is 32 rows (A: lane i < 32 holds row i) against
// 64 columns (B: lane l holds column l), and a wave issues two of them a step, for its upper and lower 32 rows: two
// chains that are independent, so that neither waits for its own last result.  Every output is still one chain over k
// ascending from zero.  A lane needs two elements of x and one of W a step for 4096 multiply-adds of the wave.
// Operands come through a ring of four stages of 32 steps of k in LDS that the workgroup shares (buffer loads with
// LDS as destination, chunks permuted against bank conflicts, one barrier a stage).  K a multiple of 32.
#define F32P_BM 128
#define F32P_BN 128
#define F32P_KB 32
#define F32P_STAGES 4

template <typename WT>
struct F32PShape {
  static constexpr int XBYTES = F32P_BM * F32P_KB * 4;                        // 16 KB
  static constexpr int WROW = F32P_KB * (int)sizeof(WT);                      // 64 or 128 bytes
  static constexpr int WBYTES = F32P_BN * WROW;
  static constexpr int STAGE = XBYTES + WBYTES;
  static constexpr int X_LOADS = XBYTES / 1024 / 4, W_LOADS = WBYTES / 1024 / 4;   // per wave
  static constexpr int LPW = X_LOADS + W_LOADS;
  static constexpr int PENDING = LPW * (F32P_STAGES - 2);
};

template <typename WT>
__device__ __forceinline__ void f32p_issue(unsigned char* ring, __amdgpu_buffer_rsrc_t rs_x, __amdgpu_buffer_rsrc_t rs_w,
                                           const int* voff_x, const int* voff_w, int wave, int step, int steps) {
  using S = F32PShape<WT>;
  typedef __attribute__((address_space(3))) void* lds_ptr;
  unsigned char* dst = ring + (step % F32P_STAGES) * S::STAGE;
  const bool real = step < steps;                                  // scalar
#pragma unroll
  for (int t = 0; t < S::X_LOADS; ++t)
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_x, (lds_ptr)(dst + (wave * S::X_LOADS + t) * 1024), 16,
                                             real ? voff_x[t] : 0x7ffffff0, step * F32P_KB * 4, 0, 0);
#pragma unroll
  for (int t = 0; t < S::W_LOADS; ++t)
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_w, (lds_ptr)(dst + S::XBYTES + (wave * S::W_LOADS + t) * 1024), 16,
                                             real ? voff_w[t] : 0x7ffffff0, step * S::WROW, 0, 0);
}

typedef __attribute__((ext_vector_type(32))) float f32x32;

template <typename WT>
__global__ __launch_bounds__(256) void gemm_f32_mfma_tile_kernel(const float* __restrict__ x, const WT* __restrict__ w,
                                                                float* __restrict__ y, int M, int N, int K, int ldx, int ldy,
                                                                int accumulate) {
  using S = F32PShape<WT>;
  constexpr bool BF = sizeof(WT) == 2;
  extern __shared__ __attribute__((aligned(16))) unsigned char f32p_ring[];
  const int wave = wave_index(), lane = threadIdx.x & 63;
  const int wy = wave >> 1, wx = wave & 1;
  const int m0 = blockIdx.y * F32P_BM, n0 = blockIdx.x * F32P_BN;
  const int x_rows = min(F32P_BM, M - m0), w_rows = min(F32P_BN, N - n0);
  const __amdgpu_buffer_rsrc_t rs_x = __builtin_amdgcn_make_buffer_rsrc(
      (void*)(x + (size_t)m0 * ldx), 0, (int)((((size_t)x_rows - 1) * ldx + K) * sizeof(float)), 0x00020000);
  const __amdgpu_buffer_rsrc_t rs_w =
      __builtin_amdgcn_make_buffer_rsrc((void*)(w + (size_t)n0 * K), 0, (int)((size_t)w_rows * K * sizeof(WT)), 0x00020000);
  // loads: 1 KB an instruction.  Rows of 128 bytes (x; 32-bit weights): 8 rows, lane l fills slot l % 8 of row l / 8 with
  // chunk slot ^ (row % 8).  Rows of 64 bytes (bfloat16 weights): 16 rows, slot l % 4 of row l / 4, chunk
  // slot ^ ((row / 2) % 4).  Rows past the operand are clamped to its last: their outputs are never stored.
  int voff_x[S::X_LOADS], voff_w[S::W_LOADS];
#pragma unroll
  for (int t = 0; t < S::X_LOADS; ++t) {
    const int row = 8 * (wave * S::X_LOADS + t) + (lane >> 3), chunk = (lane & 7) ^ (row & 7);
    voff_x[t] = (min(row, x_rows - 1) * ldx + 4 * chunk) * 4;
  }
#pragma unroll
  for (int t = 0; t < S::W_LOADS; ++t) {
    if constexpr (BF) {
      const int row = 16 * (wave * S::W_LOADS + t) + (lane >> 2), chunk = (lane & 3) ^ ((row >> 1) & 3);
      voff_w[t] = (min(row, w_rows - 1) * K + 8 * chunk) * 2;
    } else {
      const int row = 8 * (wave * S::W_LOADS + t) + (lane >> 3), chunk = (lane & 7) ^ (row & 7);
      voff_w[t] = (min(row, w_rows - 1) * K + 4 * chunk) * 4;
    }
  }
  // operand reads: rows wy*64 + (lane % 32) and 32 further of x; column wx*64 + lane of W
  const int xr0 = wy * 64 + (lane & 31), xr1 = xr0 + 32;
  const int x_off0 = xr0 * 128, x_off1 = xr1 * 128, x_swz = xr0 & 7;     // (xr1 % 8 == xr0 % 8)
  const int wc = wx * 64 + lane;
  const int w_off = S::XBYTES + wc * S::WROW, w_swz = BF ? (wc >> 1) & 3 : wc & 7;
  f32x32 acc0, acc1;
#pragma unroll
  for (int r = 0; r < 32; ++r) {
    acc0[r] = 0.f;
    acc1[r] = 0.f;
  }
  const int steps = K / F32P_KB;
#pragma unroll
  for (int st = 0; st < F32P_STAGES - 1; ++st) f32p_issue<WT>(f32p_ring, rs_x, rs_w, voff_x, voff_w, wave, st, steps);
  for (int step = 0; step < steps; ++step) {
    __builtin_amdgcn_s_waitcnt(vmcnt_only(S::PENDING));
    __builtin_amdgcn_s_barrier();                                    // everyone has the stage at hand and is done with the one before
    asm volatile("" ::: "memory");
    f32p_issue<WT>(f32p_ring, rs_x, rs_w, voff_x, voff_w, wave, step + F32P_STAGES - 1, steps);
    const unsigned char* stage = f32p_ring + (step % F32P_STAGES) * S::STAGE;
#pragma unroll
    for (int c8 = 0; c8 < F32P_KB / 8; ++c8) {                        // 8 steps of k at a time
      float wv[8];
      if constexpr (BF) {
        const u32x4 raw = *reinterpret_cast<const u32x4*>(stage + w_off + ((c8 ^ w_swz) * 16));
#pragma unroll
        for (int q = 0; q < 4; ++q) {                                 // bfloat16 -> 32-bit: the bits, shifted (exact)
          wv[2 * q] = __uint_as_float(raw[q] << 16);
          wv[2 * q + 1] = __uint_as_float(raw[q] & 0xffff0000u);
        }
      } else {
#pragma unroll
        for (int h = 0; h < 2; ++h) {
          const f32x4 raw = *reinterpret_cast<const f32x4*>(stage + w_off + (((2 * c8 + h) ^ w_swz) * 16));
#pragma unroll
          for (int q = 0; q < 4; ++q) wv[4 * h + q] = raw[q];
        }
      }
      f32x4 xa[2], xb[2];
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        xa[h] = *reinterpret_cast<const f32x4*>(stage + x_off0 + (((2 * c8 + h) ^ x_swz) * 16));
        xb[h] = *reinterpret_cast<const f32x4*>(stage + x_off1 + (((2 * c8 + h) ^ x_swz) * 16));
      }
#pragma unroll
      for (int e = 0; e < 8; ++e) {                                   // k ascending; the two chains alternate
        acc0 = __builtin_amdgcn_mfma_f32_32x32x1f32(xa[e >> 2][e & 3], wv[e], acc0, 1, 0, 0);
        acc1 = __builtin_amdgcn_mfma_f32_32x32x1f32(xb[e >> 2][e & 3], wv[e], acc1, 1, 0, 0);
      }
    }
    asm volatile("" ::: "memory");
  }
  __builtin_amdgcn_s_waitcnt(vmcnt_only(0));                         // the padding loads too, before the waves end
  // lane l, register r of a block: row 8 * (r / 4) + 4 * (l / 32) + r % 4 of the 32, column l % 32 (+ 32 for the
  // second block, registers 16 to 31)
#pragma unroll
  for (int half = 0; half < 2; ++half)
#pragma unroll
    for (int r = 0; r < 32; ++r) {
      const int m = m0 + wy * 64 + 32 * half + 8 * ((r & 15) >> 2) + 4 * (lane >> 5) + (r & 3);
      const int n = n0 + wx * 64 + 32 * (r >> 4) + (lane & 31);
      if (m < M && n < N) {
        float* o = y + (size_t)m * ldy + n;
        const float v = half == 0 ? acc0[r] : acc1[r];
        *o = accumulate ? (*o + v) : v;
      }
    }
}

template <typename WT>
static void launch_f32_mfma_tiles(const float* x, const WT* w, float* y, int M, int N, int K, int ldx, int ldy, int accumulate,
                                  hipStream_t s) {
  using S = F32PShape<WT>;
  constexpr int lds_bytes = F32P_STAGES * S::STAGE;
  static bool allowed = false;                       // more than 64 KB of dynamic LDS has to be asked for once
  if (!allowed) {
    (void)hipFuncSetAttribute((const void*)gemm_f32_mfma_tile_kernel<WT>, hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes);
    allowed = true;
  }
  hipLaunchKernelGGL(gemm_f32_mfma_tile_kernel<WT>, dim3((N + F32P_BN - 1) / F32P_BN, (M + F32P_BM - 1) / F32P_BM), dim3(256),
                     lds_bytes, s, x, w, y, M, N, K, ldx, ldy, accumulate);
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
  // 17 to 64 rows, K in whole stages: the chains run on the matrix cores (offsets within x and within a wave's rows
  // of W must fit the buffer descriptors' 31 bits).  Up to 16 rows stay on the vector unit: a matrix instruction that
  // depends on the one before it issues some 40 clocks later, a vector one 4, and so few rows have too few chains
  // to fill the gap.
  if (M > 16 && M <= 64 && K % 64 == 0 && ldx % 4 == 0 && ((uintptr_t)x & 15) == 0 && ((uintptr_t)w & 15) == 0 &&
      (size_t)M * ldx * 4 < ((size_t)1 << 31) && (size_t)64 * K * 4 < ((size_t)1 << 31)) {
    if (w_is_bf16) launch_f32_mfma_rows<bf16_t>(x, (const bf16_t*)w, y, M, N, K, ldx, ldy, accumulate, s);
    else launch_f32_mfma_rows<float>(x, (const float*)w, y, M, N, K, ldx, ldy, accumulate, s);
    return BW_LAUNCH_CHECK();
  }
  // up to 8 rows, many columns, K in whole stages: a wave a row, the row four elements a register, loader waves
  if (M <= F32C_MAX_ROWS && (N + 63) / 64 >= F32L_MIN_BLOCKS && K % (w_is_bf16 ? 64 : 32) == 0 && ldx % 4 == 0 && ((uintptr_t)x & 15) == 0 &&
      ((uintptr_t)w & 15) == 0 && (size_t)64 * K * 4 < ((size_t)1 << 31) && (size_t)M * ldx * 4 < ((size_t)1 << 31)) {
    if (w_is_bf16) launch_chain<bf16_t>(x, (const bf16_t*)w, y, M, N, K, ldx, ldy, accumulate, s);
    else launch_chain<float>(x, (const float*)w, y, M, N, K, ldx, ldy, accumulate, s);
    return BW_LAUNCH_CHECK();
  }
  // up to 16 rows, many columns, K in whole stages: a wave a row, weights packed in LDS
  if (M <= 16 && (N + 63) / 64 >= F32L_MIN_BLOCKS && K % (w_is_bf16 ? 64 : 32) == 0 && ldx % 4 == 0 && ((uintptr_t)x & 15) == 0 &&
      ((uintptr_t)w & 15) == 0 && (size_t)64 * K * 4 < ((size_t)1 << 31) && (size_t)M * ldx * 4 < ((size_t)1 << 31)) {
    if (w_is_bf16) launch_lanes<bf16_t>(x, (const bf16_t*)w, y, M, N, K, ldx, ldy, accumulate, s);
    else launch_lanes<float>(x, (const float*)w, y, M, N, K, ldx, ldy, accumulate, s);
    return BW_LAUNCH_CHECK();
  }
  if (M <= 64 && K % wc == 0 && ldx % 4 == 0 && ((uintptr_t)x & 15) == 0 && ((uintptr_t)w & 15) == 0) {
    if (w_is_bf16) launch_rows<bf16_t>(x, (const bf16_t*)w, y, M, N, K, ldx, ldy, accumulate, s);
    else launch_rows<float>(x, (const float*)w, y, M, N, K, ldx, ldy, accumulate, s);
    return BW_LAUNCH_CHECK();
  }
  // prompt portions, K in whole stages: tiles on the matrix cores (the same chains)
  if (M > 64 && K % F32P_KB == 0 && ldx % 4 == 0 && ((uintptr_t)x & 15) == 0 && ((uintptr_t)w & 15) == 0 &&
      (size_t)F32P_BM * ldx * 4 < ((size_t)1 << 31) && (size_t)F32P_BN * K * 4 < ((size_t)1 << 31)) {
    if (w_is_bf16) launch_f32_mfma_tiles<bf16_t>(x, (const bf16_t*)w, y, M, N, K, ldx, ldy, accumulate, s);
    else launch_f32_mfma_tiles<float>(x, (const float*)w, y, M, N, K, ldx, ldy, accumulate, s);
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
