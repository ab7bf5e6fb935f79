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

extern "C" int bw_gemm_f32(const float* x, const void* w, int w_is_bf16, float* y, int M, int N, int K, int ldx,
                           int ldy, int accumulate, void* stream) {
  if (M <= 0 || N <= 0) return 0;
  if (K <= 0 || ldx < K || ldy < N) return -2;
  dim3 grid((N + F32_BN - 1) / F32_BN, (M + F32_BM - 1) / F32_BM), block(256);
  hipStream_t s = (hipStream_t)stream;
  if (w_is_bf16)
    hipLaunchKernelGGL(gemm_f32_kernel<bf16_t>, grid, block, 0, s, x, (const bf16_t*)w, y, M, N, K, ldx, ldy, accumulate);
  else
    hipLaunchKernelGGL(gemm_f32_kernel<float>, grid, block, 0, s, x, (const float*)w, y, M, N, K, ldx, ldy, accumulate);
  return BW_LAUNCH_CHECK();
}
