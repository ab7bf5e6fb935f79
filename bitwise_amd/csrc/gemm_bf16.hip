// bfloat16 matrix product on the matrix cores: y[m][n] = sum_k x[m][k] * W[n][k],
// x bfloat16 [M][K], W bfloat16 row-major [N][K], 32-bit accumulation.
//
// Arithmetic, the same for every M (one row or thousands): each 16x16 block of outputs is
// one accumulator that runs v_mfma_f32_16x16x32_bf16 over k = 0, 32, 64, ... in ascending
// order, starting from zero; within an instruction lane group g holds k = kk+8g..kk+8g+7.
// An output's bits therefore depend only on its own row of x and row of W.  K is never
// split.  Tile shapes only decide which outputs share loads.
//
// Epilogues: store 32-bit, store bfloat16, add into a 32-bit residual (each output owned
// by one lane: no atomics), or SwiGLU of two products (gate rows n, up rows N+n of a
// stacked weight) stored as bfloat16: h = g * (1/(1+exp(-g))) * u in 32-bit.
#include "common.h"
#include "api.h"

enum { EPI_F32 = 0, EPI_BF16 = 1, EPI_ADD_F32 = 2, EPI_SWIGLU_BF16 = 3 };

__device__ __forceinline__ u32x4 load_frag(const bf16_t* __restrict__ base, int row, int rows, int ld, int k, int K) {
  u32x4 v = {0u, 0u, 0u, 0u};
  if (row < rows && k < K) v = *reinterpret_cast<const u32x4*>(base + (size_t)row * ld + k);
  return v;
}

template <int WAVES_M, int WAVES_N, int WM, int WN, int EPI>
__global__ __launch_bounds__(256) void gemm_bf16_kernel(const bf16_t* __restrict__ x, const bf16_t* __restrict__ w,
                                                        void* __restrict__ out, int M, int N, int K, int ldx,
                                                        int ldo) {
  static_assert(WAVES_M * WAVES_N == 4, "four waves per workgroup");
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int r = lane & 15, g = lane >> 4;
  const int m0 = (blockIdx.y * WAVES_M + wave / WAVES_N) * (16 * WM);
  const int n0 = (blockIdx.x * WAVES_N + wave % WAVES_N) * (16 * WN);
  if (m0 >= M || n0 >= N) return;
  constexpr int NB = (EPI == EPI_SWIGLU_BF16) ? 2 : 1;
  f32x4 acc[NB][WM][WN];
#pragma unroll
  for (int b = 0; b < NB; ++b)
#pragma unroll
    for (int i = 0; i < WM; ++i)
#pragma unroll
      for (int j = 0; j < WN; ++j) acc[b][i][j] = (f32x4){0.f, 0.f, 0.f, 0.f};

  for (int kk = 0; kk < K; kk += 32) {
    const int k = kk + 8 * g;
    u32x4 a[WM], b[NB][WN];
#pragma unroll
    for (int i = 0; i < WM; ++i) a[i] = load_frag(x, m0 + 16 * i + r, M, ldx, k, K);
#pragma unroll
    for (int j = 0; j < WN; ++j) {
      b[0][j] = load_frag(w, n0 + 16 * j + r, N, K, k, K);
      if constexpr (NB == 2) b[1][j] = load_frag(w + (size_t)N * K, n0 + 16 * j + r, N, K, k, K);
    }
#pragma unroll
    for (int bb = 0; bb < NB; ++bb)
#pragma unroll
      for (int i = 0; i < WM; ++i)
#pragma unroll
        for (int j = 0; j < WN; ++j)
          acc[bb][i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(a[i]), as_bf16x8(b[bb][j]),
                                                                  acc[bb][i][j], 0, 0, 0);
  }

  // Accumulator layout: lane (r, g) holds rows 4g..4g+3 of column r of each 16x16 block.
#pragma unroll
  for (int i = 0; i < WM; ++i)
#pragma unroll
    for (int j = 0; j < WN; ++j) {
      const int n = n0 + 16 * j + r;
      if (n >= N) continue;
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int m = m0 + 16 * i + 4 * g + q;
        if (m >= M) continue;
        const size_t o = (size_t)m * ldo + n;
        const float v = acc[0][i][j][q];
        if constexpr (EPI == EPI_F32) ((float*)out)[o] = v;
        else if constexpr (EPI == EPI_BF16) ((bf16_t*)out)[o] = f32_to_bf16(v);
        else if constexpr (EPI == EPI_ADD_F32) ((float*)out)[o] += v;
        else {
          const float u = acc[NB - 1][i][j][q];
          ((bf16_t*)out)[o] = f32_to_bf16(v * (1.0f / (1.0f + fast_exp(-v))) * u);
        }
      }
    }
}

template <int EPI>
static int launch_gemm_bf16(const bf16_t* x, const bf16_t* w, void* out, int M, int N, int K, int ldx, int ldo,
                            hipStream_t s) {
  if (M <= 16) {
    dim3 grid((N + 63) / 64, 1), block(256);
    hipLaunchKernelGGL((gemm_bf16_kernel<1, 4, 1, 1, EPI>), grid, block, 0, s, x, w, out, M, N, K, ldx, ldo);
  } else {
    dim3 grid((N + 63) / 64, (M + 63) / 64), block(256);
    hipLaunchKernelGGL((gemm_bf16_kernel<2, 2, 2, 2, EPI>), grid, block, 0, s, x, w, out, M, N, K, ldx, ldo);
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
