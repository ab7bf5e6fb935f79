// bfloat16 matrix product on the matrix cores: y[m][n] = sum_k x[m][k] * W[n][k],
// x bfloat16 [M][K], W bfloat16 row-major [N][K], 32-bit accumulation.
//
// Arithmetic, the same for every M (one row or thousands): K is cut into segments of 2048
// (a property of the weight, never of the batch).  Within a segment each 16x16 block of
// outputs is one accumulator that runs v_mfma_f32_16x16x32_bf16 over k ascending in steps
// of 32 from zero; within an instruction lane group g holds k = kk+8g..kk+8g+7.  Segment
// results are added in 32-bit left to right: y = ((p0 + p1) + p2) + ...  An output's bits
// therefore depend only on its own row of x and row of W.
//
// Two kernels run this arithmetic.  The skinny one (up to 64 rows: decode) gives every
// 16-column strip of W and every segment a wave of its own, which streams its 16 x 2048
// weights once through a ring of operand registers kept full of loads in flight; the waves
// of a strip join their segment results through LDS in segment order.  The wide one (prompt
// portions) stages 128x64 tiles of x and W through LDS (double buffered, rows padded to 144
// bytes so that 16-byte operand reads hit distinct banks) and gives each of four waves a
// 64x64 block of outputs.
//
// Epilogues: store 32-bit, store bfloat16, add into a 32-bit residual (each output owned
// by one lane: no atomics), or SwiGLU of two products (gate rows n, up rows N+n of a
// stacked weight) stored as bfloat16: h = g * (1/(1+exp(-g))) * u in 32-bit.
#include "common.h"
#include "api.h"

enum { EPI_F32 = 0, EPI_BF16 = 1, EPI_ADD_F32 = 2, EPI_SWIGLU_BF16 = 3 };

#define GEMM_SEG 2048

template <int EPI>
__device__ __forceinline__ void epilogue_store(void* __restrict__ out, size_t o, float v, float u) {
  if constexpr (EPI == EPI_F32) ((float*)out)[o] = v;
  else if constexpr (EPI == EPI_BF16) ((bf16_t*)out)[o] = f32_to_bf16(v);
  else if constexpr (EPI == EPI_ADD_F32) ((float*)out)[o] += v;
  else ((bf16_t*)out)[o] = f32_to_bf16(v * (1.0f / (1.0f + fast_exp(-v))) * u);
}

// ------------------------------------------------------------------------------ skinny

// TAIL: K is no multiple of 32, so the last step of the last segment is partly zero-filled,
// lane by lane.  Without TAIL nothing in the main loop depends on the lane: rows of W past N
// and rows of x past M are read from row 0 instead and their results thrown away, ring
// refills past the segment's end re-read its first step and are never used, and a segment
// whose step count is no multiple of D runs a few extra steps on zeros (adding exact zeros
// to an accumulator does not change its bits).
template <int WM, int EPI, int D, bool TAIL>
__global__ __launch_bounds__(256) void gemm_bf16_skinny_kernel(const bf16_t* __restrict__ x, const bf16_t* __restrict__ w,
                                                               void* __restrict__ out, int M, int N, int K, int ldx,
                                                               int ldo, int S) {
  constexpr int NB = (EPI == EPI_SWIGLU_BF16) ? 2 : 1;
  extern __shared__ float red[];   // [S][NB][WM][4][64] when S > 1
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, nwaves = blockDim.x >> 6;
  const int r = lane & 15, g = lane >> 4;
  const int n0 = blockIdx.x * 16;
  const bool n_ok = n0 + r < N;
  const bf16_t* wp[NB];
#pragma unroll
  for (int b = 0; b < NB; ++b) wp[b] = w + ((size_t)b * N + (n_ok ? n0 + r : 0)) * K + 8 * g;
  const bf16_t* xp[WM];
#pragma unroll
  for (int i = 0; i < WM; ++i) xp[i] = x + (size_t)(16 * i + r < M ? 16 * i + r : 0) * ldx + 8 * g;
  const u32x4 zero = {0u, 0u, 0u, 0u};
  f32x4 acc[NB][WM];
  for (int s = wave; s < S; s += nwaves) {
    const int k_begin = s * GEMM_SEG;
    const int k_end = (K - k_begin) < GEMM_SEG ? K : k_begin + GEMM_SEG;
#pragma unroll
    for (int b = 0; b < NB; ++b)
#pragma unroll
      for (int i = 0; i < WM; ++i) acc[b][i] = (f32x4){0.f, 0.f, 0.f, 0.f};
    u32x4 bq[D][NB], aq[D][WM];
    auto issue = [&](int d, int k) {
      // k is the same for all lanes; past the end the slot is filled from the segment's first step
      const int ks = k < k_end ? k : k_begin;
#pragma unroll
      for (int b = 0; b < NB; ++b) bq[d][b] = *reinterpret_cast<const u32x4*>(wp[b] + ks);
#pragma unroll
      for (int i = 0; i < WM; ++i) aq[d][i] = *reinterpret_cast<const u32x4*>(xp[i] + ks);
    };
#pragma unroll
    for (int d = 0; d < D; ++d) issue(d, k_begin + 32 * d);
    __builtin_amdgcn_sched_barrier(0);
    for (int k0 = k_begin; k0 < k_end; k0 += 32 * D) {
#pragma unroll
      for (int d = 0; d < D; ++d) {
        const int k = k0 + 32 * d;
        u32x4 bc[NB], ac[WM];
        bool live = k < k_end;
        if constexpr (TAIL) live = k + 8 * g < k_end && (k + 8 * g + 8 <= K);
#pragma unroll
        for (int b = 0; b < NB; ++b) bc[b] = live ? bq[d][b] : zero;
#pragma unroll
        for (int i = 0; i < WM; ++i) ac[i] = live ? aq[d][i] : zero;
        issue(d, k + 32 * D);
        // keep the refill where it is written: the scheduler would otherwise sink every load
        // to just before its use and the ring would hold nothing in flight
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int b = 0; b < NB; ++b)
#pragma unroll
          for (int i = 0; i < WM; ++i)
            acc[b][i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(ac[i]), as_bf16x8(bc[b]), acc[b][i], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    if (S > 1) {
#pragma unroll
      for (int b = 0; b < NB; ++b)
#pragma unroll
        for (int i = 0; i < WM; ++i)
#pragma unroll
          for (int q = 0; q < 4; ++q) red[(((s * NB + b) * WM + i) * 4 + q) * 64 + lane] = acc[b][i][q];
    }
  }
  if (S > 1) {
    __syncthreads();
    if (wave != 0) return;
#pragma unroll
    for (int b = 0; b < NB; ++b)
#pragma unroll
      for (int i = 0; i < WM; ++i)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          float y = red[((b * WM + i) * 4 + q) * 64 + lane];
          for (int s = 1; s < S; ++s) y += red[(((s * NB + b) * WM + i) * 4 + q) * 64 + lane];
          acc[b][i][q] = y;
        }
  }
  if (!n_ok) return;
#pragma unroll
  for (int i = 0; i < WM; ++i)
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int m = 16 * i + 4 * g + q;
      if (m < M) epilogue_store<EPI>(out, (size_t)m * ldo + n0 + r, acc[0][i][q], acc[NB - 1][i][q]);
    }
}

// ------------------------------------------------------------------------------ wide

#define WIDE_BM 128
#define WIDE_BN 128
#define WIDE_BK 64
#define WIDE_LDS_ROW 72   // bf16 elements per LDS row: 64 of data + 8 of padding (144 bytes)

template <int EPI, bool MULTI>
__global__ __launch_bounds__(256) void gemm_bf16_wide_kernel(const bf16_t* __restrict__ x, const bf16_t* __restrict__ w,
                                                             void* __restrict__ out, int M, int N, int K, int ldx,
                                                             int ldo, int m_tiles, int n_tiles) {
  // In SwiGLU mode a block covers 64 output columns: B rows 0-63 are gate rows, 64-127 up rows.
  constexpr int COLS = (EPI == EPI_SWIGLU_BF16) ? 64 : 128;
  __shared__ __attribute__((aligned(16))) bf16_t lds_a[2][WIDE_BM * WIDE_LDS_ROW];
  __shared__ __attribute__((aligned(16))) bf16_t lds_b[2][WIDE_BN * WIDE_LDS_ROW];
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int r = lane & 15, g = lane >> 4;
  const int wy = wave >> 1, wx = wave & 1;
  // Blocks that run at the same time share an n tile (its weights are fetched once from HBM);
  // consecutive block ids go to different XCDs, so ids are regrouped by XCD first.
  int bid = blockIdx.x;
  const int nblocks = m_tiles * n_tiles;
  if (nblocks % 8 == 0) bid = (bid % 8) * (nblocks / 8) + bid / 8;
  const int m0 = (bid % m_tiles) * WIDE_BM;
  const int n0 = (bid / m_tiles) * COLS;

  // this thread's share of the global -> LDS copies: rows lr + 32j, 16-byte chunk lc
  const int lr = tid >> 3, lc = tid & 7;
  const bf16_t* ga[4];
  const bf16_t* gb[4];
  bool ga_ok[4], gb_ok[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int row = lr + 32 * j;
    ga_ok[j] = m0 + row < M;
    ga[j] = x + (size_t)(ga_ok[j] ? m0 + row : 0) * ldx + lc * 8;
    int wrow;
    if constexpr (EPI == EPI_SWIGLU_BF16) wrow = (row < 64) ? n0 + row : N + n0 + row - 64;
    else wrow = n0 + row;
    const int ncol = (EPI == EPI_SWIGLU_BF16) ? n0 + (row & 63) : n0 + row;
    gb_ok[j] = ncol < N;
    gb[j] = w + (size_t)(gb_ok[j] ? wrow : 0) * K + lc * 8;
  }
  // LDS rows of this wave's four B tiles
  int brow[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    if constexpr (EPI == EPI_SWIGLU_BF16) brow[j] = (j >> 1) * 64 + 32 * wx + 16 * (j & 1);
    else brow[j] = 64 * wx + 16 * j;
  }

  f32x4 acc[4][4], tot[MULTI ? 4 : 1][MULTI ? 4 : 1];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      acc[i][j] = (f32x4){0.f, 0.f, 0.f, 0.f};
      if constexpr (MULTI) tot[i][j] = (f32x4){0.f, 0.f, 0.f, 0.f};
    }

  const u32x4 zero = {0u, 0u, 0u, 0u};
  u32x4 ra[4], rb[4];
  auto fetch = [&](int k0) {
    const bool in = k0 + lc * 8 < K;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      ra[j] = (in && ga_ok[j]) ? *reinterpret_cast<const u32x4*>(ga[j] + k0) : zero;
      rb[j] = (in && gb_ok[j]) ? *reinterpret_cast<const u32x4*>(gb[j] + k0) : zero;
    }
  };
  auto stash = [&](int buf) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      *reinterpret_cast<u32x4*>(&lds_a[buf][(lr + 32 * j) * WIDE_LDS_ROW + lc * 8]) = ra[j];
      *reinterpret_cast<u32x4*>(&lds_b[buf][(lr + 32 * j) * WIDE_LDS_ROW + lc * 8]) = rb[j];
    }
  };

  fetch(0);
  stash(0);
  __syncthreads();
  int buf = 0;
  for (int k0 = 0; k0 < K; k0 += WIDE_BK) {
    const bool more = k0 + WIDE_BK < K;
    if (more) fetch(k0 + WIDE_BK);
#pragma unroll
    for (int kk = 0; kk < 2; ++kk) {
      u32x4 fa[4], fb[4];
#pragma unroll
      for (int i = 0; i < 4; ++i)
        fa[i] = *reinterpret_cast<const u32x4*>(&lds_a[buf][(64 * wy + 16 * i + r) * WIDE_LDS_ROW + kk * 32 + g * 8]);
#pragma unroll
      for (int j = 0; j < 4; ++j)
        fb[j] = *reinterpret_cast<const u32x4*>(&lds_b[buf][(brow[j] + r) * WIDE_LDS_ROW + kk * 32 + g * 8]);
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(fa[i]), as_bf16x8(fb[j]), acc[i][j], 0, 0, 0);
    }
    if constexpr (MULTI) {
      const int kn = k0 + WIDE_BK;
      if (kn % GEMM_SEG == 0 || kn >= K) {          // a segment ends: join it to the total, left to right
        const bool first = k0 < GEMM_SEG;
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            tot[i][j] = first ? acc[i][j] : tot[i][j] + acc[i][j];
            acc[i][j] = (f32x4){0.f, 0.f, 0.f, 0.f};
          }
      }
    }
    if (more) stash(buf ^ 1);
    __syncthreads();
    buf ^= 1;
  }

#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int m = m0 + 64 * wy + 16 * i + 4 * g + q;
      if (m >= M) continue;
      if constexpr (EPI == EPI_SWIGLU_BF16) {
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          const int n = n0 + 32 * wx + 16 * j + r;
          if (n >= N) continue;
          const float gv = MULTI ? tot[MULTI ? i : 0][MULTI ? j : 0][q] : acc[i][j][q];
          const float uv = MULTI ? tot[MULTI ? i : 0][MULTI ? j + 2 : 0][q] : acc[i][j + 2][q];
          epilogue_store<EPI>(out, (size_t)m * ldo + n, gv, uv);
        }
      } else {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const int n = n0 + 64 * wx + 16 * j + r;
          if (n >= N) continue;
          const float v = MULTI ? tot[MULTI ? i : 0][MULTI ? j : 0][q] : acc[i][j][q];
          epilogue_store<EPI>(out, (size_t)m * ldo + n, v, v);
        }
      }
    }
}

// ------------------------------------------------------------------------------ launch

template <int EPI>
static int launch_gemm_bf16(const bf16_t* x, const bf16_t* w, void* out, int M, int N, int K, int ldx, int ldo,
                            hipStream_t s) {
  const int S = (K + GEMM_SEG - 1) / GEMM_SEG;
  constexpr int NB = (EPI == EPI_SWIGLU_BF16) ? 2 : 1;
  if (M <= 64) {
    const int wm = (M + 15) / 16;
    const int waves = S < 4 ? S : 4;      // one wave per SIMD: the operand ring may use up to 512 registers
    dim3 grid((N + 15) / 16), block(64 * waves);
    const size_t lds = S > 1 ? (size_t)S * NB * wm * 4 * 64 * sizeof(float) : 0;
    if (lds > 64 * 1024) return -2;
#define BW_SKINNY(WMV, DV)                                                                                         \
  if (K % 32)                                                                                                      \
    hipLaunchKernelGGL((gemm_bf16_skinny_kernel<WMV, EPI, DV, true>), grid, block, lds, s, x, w, out, M, N, K, ldx, ldo, S); \
  else                                                                                                             \
    hipLaunchKernelGGL((gemm_bf16_skinny_kernel<WMV, EPI, DV, false>), grid, block, lds, s, x, w, out, M, N, K, ldx, ldo, S);
    switch (wm) {
      case 1: BW_SKINNY(1, (NB == 2 ? 12 : 16)) break;
      case 2: BW_SKINNY(2, (NB == 2 ? 8 : 12)) break;
      case 3: BW_SKINNY(3, 8) break;
      default: BW_SKINNY(4, 8) break;
    }
#undef BW_SKINNY
  } else {
    constexpr int COLS = (EPI == EPI_SWIGLU_BF16) ? 64 : 128;
    const int m_tiles = (M + WIDE_BM - 1) / WIDE_BM, n_tiles = (N + COLS - 1) / COLS;
    dim3 grid(m_tiles * n_tiles), block(256);
    if (S > 1)
      hipLaunchKernelGGL((gemm_bf16_wide_kernel<EPI, true>), grid, block, 0, s, x, w, out, M, N, K, ldx, ldo, m_tiles, n_tiles);
    else
      hipLaunchKernelGGL((gemm_bf16_wide_kernel<EPI, false>), grid, block, 0, s, x, w, out, M, N, K, ldx, ldo, m_tiles, n_tiles);
  }
  return BW_LAUNCH_CHECK();
}

extern "C" int bw_gemm_bf16(const void* x, const void* w, void* out, int M, int N, int K, int ldx, int ldo,
                            int epilogue, void* stream) {
  if (M <= 0 || N <= 0) return 0;
  if (K <= 0 || (K % 8) || (ldx % 8) || ldx < K || ldo < N) return -2;
  if ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(w)) & 15) return -3;
  hipStream_t s = (hipStream_t)stream;
  const bf16_t* xp = (const bf16_t*)x;
  const bf16_t* wp = (const bf16_t*)w;
  switch (epilogue) {
    case EPI_F32: return launch_gemm_bf16<EPI_F32>(xp, wp, out, M, N, K, ldx, ldo, s);
    case EPI_BF16: return launch_gemm_bf16<EPI_BF16>(xp, wp, out, M, N, K, ldx, ldo, s);
    case EPI_ADD_F32: return launch_gemm_bf16<EPI_ADD_F32>(xp, wp, out, M, N, K, ldx, ldo, s);
    case EPI_SWIGLU_BF16: return launch_gemm_bf16<EPI_SWIGLU_BF16>(xp, wp, out, M, N, K, ldx, ldo, s);
  }
  return -2;
}
