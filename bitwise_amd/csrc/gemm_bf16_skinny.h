// Part of gemm_bf16.hip (included there, after its epilogues and launch macro; not a unit of its own):
// the kernel of a wave per strip of columns and segment of K (any K, any rows up to 64).
#pragma once

// ------------------------------------------------------------------------------ skinny

// One wave per (strip of CW output columns, segment of K).  All its loads go through buffer
// descriptors with one per-lane offset fixed for the whole kernel and the step's offset in a
// scalar register, and every decision about a step (is it inside the segment?) is scalar too:
// the loop spends no vector instruction on addresses or masks.  Rows of W past N and rows of x
// past M lie outside their descriptors and read as zeros.  A ring of D operand registers keeps
// D steps of weights in flight (D = 64 holds a whole segment: nothing is refilled); the few rows
// of x come from cache a few steps ahead.
//
// CW = 8 halves the strip (lanes 8..15 repeat the columns of lanes 0..7 and their results are
// dropped): twice as many workgroups, for products with too few columns to give every compute
// unit a 16-column strip.  TAIL: K is no multiple of 32, so the last step of the last segment
// is zero-filled lane by lane past K.
template <int WM, int EPI, int D, bool TAIL, int CW>
__global__ __launch_bounds__(256) void gemm_bf16_skinny_kernel(const bf16_t* __restrict__ x, const bf16_t* __restrict__ w,
                                                               void* __restrict__ out, int M, int N, int K, int ldx,
                                                               int ldo, int S) {
  constexpr int NB = (EPI == EPI_SWIGLU_BF16) ? 2 : 1;
  constexpr int DA = D < 32 ? D : 32;             // look-ahead of the x operands (they come from cache)
  constexpr bool FULL = D * 32 >= GEMM_SEG;
  static_assert(D % DA == 0, "the x look-ahead must divide the ring depth");
  extern __shared__ float red[];   // [S][NB][WM][4][64] when S > 1
  const int wave = wave_index(), lane = threadIdx.x & 63, nwaves = blockDim.x >> 6;
  const int r = lane & 15, g = lane >> 4;
  const int c = r % CW;
  const int n0 = blockIdx.x * CW;
  // blockIdx.y: which block of 16*WM rows
  x += (size_t)blockIdx.y * (16 * WM) * ldx;
  M -= blockIdx.y * (16 * WM);
  if constexpr (EPI == EPI_F32 || EPI == EPI_ADD_F32) out = (float*)out + (size_t)blockIdx.y * (16 * WM) * ldo;
  else out = (bf16_t*)out + (size_t)blockIdx.y * (16 * WM) * ldo;
  const bool n_ok = r < CW && n0 + c < N;
  const int w_rows = min(CW, N - n0);
  __amdgpu_buffer_rsrc_t rs_w[NB];
#pragma unroll
  for (int b = 0; b < NB; ++b)
    rs_w[b] = __builtin_amdgcn_make_buffer_rsrc((void*)(w + ((size_t)b * N + n0) * K), 0, (int)((size_t)w_rows * K * 2), 0x00020000);
  const __amdgpu_buffer_rsrc_t rs_x =
      __builtin_amdgcn_make_buffer_rsrc((void*)x, 0, (int)((((size_t)M - 1) * ldx + K) * 2), 0x00020000);
  // in a half strip the lanes 8..15 point outside the descriptor: they read zeros and ask memory for nothing
  const int voff_w = r < CW ? (c * K + 8 * g) * 2 : 0x7ffffff0;
  int voff_x[WM];
#pragma unroll
  for (int i = 0; i < WM; ++i) voff_x[i] = ((16 * i + r) * ldx + 8 * g) * 2;
  const u32x4 zero = {0u, 0u, 0u, 0u};
  f32x4 acc[NB][WM];
  for (int s = wave; s < S; s += nwaves) {
    const int k_begin = s * GEMM_SEG;
    const int k_end = (K - k_begin) < GEMM_SEG ? K : k_begin + GEMM_SEG;
#pragma unroll
    for (int b = 0; b < NB; ++b)
#pragma unroll
      for (int i = 0; i < WM; ++i) acc[b][i] = (f32x4){0.f, 0.f, 0.f, 0.f};
    u32x4 bq[D][NB], aq[DA][WM];
    // k is the same for all lanes; past the end the slot is filled from the segment's first step
    auto issue_w = [&](int d, int k) {
      const int ks = k < k_end ? k : k_begin;
#pragma unroll
      for (int b = 0; b < NB; ++b) bq[d][b] = __builtin_amdgcn_raw_buffer_load_b128(rs_w[b], voff_w, ks * 2, 0);
    };
    auto issue_x = [&](int d, int k) {
      const int ks = k < k_end ? k : k_begin;
#pragma unroll
      for (int i = 0; i < WM; ++i) aq[d][i] = __builtin_amdgcn_raw_buffer_load_b128(rs_x, voff_x[i], ks * 2, 0);
    };
#pragma unroll
    for (int d = 0; d < DA; ++d) issue_x(d, k_begin + 32 * d);
#pragma unroll
    for (int d = 0; d < D; ++d) issue_w(d, k_begin + 32 * d);
    __builtin_amdgcn_sched_barrier(0);
    for (int k0 = k_begin; k0 < k_end; k0 += 32 * D) {
#pragma unroll
      for (int d = 0; d < D; ++d) {
        const int k = k0 + 32 * d;
        u32x4 bc[NB], ac[WM];
#pragma unroll
        for (int b = 0; b < NB; ++b) bc[b] = bq[d][b];
#pragma unroll
        for (int i = 0; i < WM; ++i) ac[i] = aq[d % DA][i];
        if constexpr (TAIL) {
          const bool live = k + 8 * g + 8 <= K;
#pragma unroll
          for (int b = 0; b < NB; ++b) bc[b] = live ? bc[b] : zero;
#pragma unroll
          for (int i = 0; i < WM; ++i) ac[i] = live ? ac[i] : zero;
        }
        issue_x(d % DA, k + 32 * DA);
        if constexpr (!FULL) issue_w(d, k + 32 * D);
        // keep the refill where it is written: the scheduler would otherwise sink every load
        // to just before its use and the ring would hold nothing in flight
        __builtin_amdgcn_sched_barrier(0);
        if (k < k_end) {                           // scalar: a step past the segment's end is skipped
#pragma unroll
          for (int b = 0; b < NB; ++b)
#pragma unroll
            for (int i = 0; i < WM; ++i)
              acc[b][i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(ac[i]), as_bf16x8(bc[b]), acc[b][i], 0, 0, 0);
        }
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
          if constexpr (EPI == EPI_ADD_F32) {          // the chain of additions starts at the residual
            const int m = 16 * i + 4 * g + q;
            if (n_ok && m < M) y = ((const float*)out)[(size_t)m * ldo + n0 + c] + y;
          }
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
      if (m >= M) continue;
      if (EPI == EPI_ADD_F32 && S > 1) ((float*)out)[(size_t)m * ldo + n0 + c] = acc[0][i][q];   // the residual is in already
      else epilogue_store<EPI>(out, (size_t)m * ldo + n0 + c, acc[0][i][q], acc[NB - 1][i][q]);
    }
}
