// Decode steps of up to 16 rows in bfloat16 mode: RMSNorm fused into the matrix product that
// follows it (the rows arrive as the 32-bit residual stream), and behind the product a plain
// store, a residual add, SwiGLU, or rotary encoding plus the cache write (for the stacked
// q|k|v product).  A decode step is bound by kernel count and by how many weight bytes are in
// flight, not by arithmetic; this kernel keeps the normalised rows in LDS, so that every
// outstanding memory request of a wave is a weight load, and replaces up to three launches.
//
// The arithmetic is that of the separate kernels, statement for statement, so a row's bits
// do not depend on which route ran it:
//   * RMSNorm: the sum of squares in the order of rmsnorm_bf16_kernel (lane l owns 16-byte
//     vectors l, l+64, ...; xor butterflies), inv = 1/sqrt(ss/dim + eps), bf16((x*inv)*w);
//   * product: K is at most one segment (2048) here; every 16x16 block of outputs is one
//     v_mfma_f32_16x16x32_bf16 chain over k ascending from zero;
//   * rotary: o1 = x1*c - x2*s, o2 = x2*c + x1*s on the 32-bit products, one rounding when
//     q goes to its buffer and k, v to their page slots (v transposed).
//
// Shape: a workgroup is a few strips of 16 output columns, one wave each (for q|k|v with
// rotary: the strips of one head, or one strip and its rotary partner).  Loads go out in the
// order their results are needed, because memory results are waited for in issue order: the
// rows to normalise and the positions first, then D steps of the wave's weights, which stay in
// flight while the rows are normalised into LDS (rows padded by 16 bytes so that operand reads
// hit distinct banks).  Then each wave runs its chain with A operands from LDS and B operands
// from its ring of registers.
#include "common.h"
#include "api.h"

enum { DEPI_F32 = 0, DEPI_BF16 = 1, DEPI_ADD_F32 = 2, DEPI_SWIGLU_BF16 = 3, DEPI_ROPE_KV = 4 };

#define DEC_SEG 2048

struct DecodeGemmArgs {
  const float* a;          // [M, lda] rows of the 32-bit residual stream
  const void* norm_w;      // [K]
  const bf16_t* w;         // [N (or 2N for SwiGLU), K]
  void* out;               // F32/ADD: float [M, ldo]; BF16/SWIGLU: bf16 [M, ldo]; ROPE_KV: q bf16 [M, heads*hd]
  int M, N, K, lda, ldo, norm_w_is_bf16;
  float eps;
  // rotary + cache write
  const int32_t* positions;
  const int32_t* row_seq;
  const int32_t* block_table;
  const float* cos_table;
  const float* sin_table;
  bf16_t* k_cache;
  bf16_t* v_cache;
  int heads, kv_heads, head_dim, page_size, table_stride, write_cache;
  int pairs;               // rotary: 16-wide pairs of strips a head is cut into (0: a workgroup is a whole head)
};

template <int EPI, int D>
__global__ __launch_bounds__(256) void decode_gemm_kernel(DecodeGemmArgs a) {
  constexpr int NB = (EPI == DEPI_SWIGLU_BF16) ? 2 : 1;
  constexpr bool FULL = D * 32 >= DEC_SEG;        // the ring holds a whole segment: nothing is refilled
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  const int K = a.K, M = a.M;
  const int lds_row = K + 8;                      // bf16 elements; +16 bytes keeps operand reads conflict-free
  bf16_t* xs = reinterpret_cast<bf16_t*>(smem);   // [M][lds_row]
  const int wave = wave_index(), lane = threadIdx.x & 63, nwaves = blockDim.x >> 6;
  const int r = lane & 15, g = lane >> 4;
  // rotary: a workgroup is a head (its strips in order), or, when half a head is a multiple of
  // 16, one strip of the first half and its partner in the second (workgroup p of the head:
  // strips p and p + pairs), so that twice as many workgroups share the stream
  int rope_head = 0, rope_base = 0, rope_lw = 0;
  int n0 = (blockIdx.x * nwaves + wave) * 16;
  if constexpr (EPI == DEPI_ROPE_KV) {
    if (a.pairs > 0) {
      rope_head = blockIdx.x / a.pairs;
      rope_base = 16 * (blockIdx.x % a.pairs);
      rope_lw = 32;
      n0 = rope_head * a.head_dim + rope_base + wave * (a.head_dim >> 1);
    } else {
      rope_head = blockIdx.x;
      rope_lw = a.head_dim;
    }
  }
  const bool n_ok = n0 + r < a.N;
  const int k_begin = 0, k_end = K;
  // weights through buffer descriptors that cover the strip's rows (rows past N read as zeros):
  // one per-lane offset for the whole kernel, the step's offset in a scalar register
  const int w_rows = min(16, a.N - n0);
  __amdgpu_buffer_rsrc_t rs_w[NB];
#pragma unroll
  for (int b = 0; b < NB; ++b)
    rs_w[b] = __builtin_amdgcn_make_buffer_rsrc((void*)(a.w + ((size_t)b * a.N + n0) * K), 0,
                                                (int)((size_t)(w_rows > 0 ? w_rows : 0) * K * 2), 0x00020000);
  const int voff_w = (r * K + 8 * g) * 2;

  // 1. Loads go out in the order in which their results are needed, because results are waited
  // for in issue order: first the rows to normalise (their first batch) and the positions, then
  // the weights, which stay in flight while the rows are normalised.
  constexpr int RB = 4;                            // rows a wave normalises at a time
  const int nvec = K >> 2;
  NormRows<RB> nr;
  const f32x4* nrows[RB];
#pragma unroll
  for (int i = 0; i < RB; ++i) {
    const int m = wave + i * nwaves;               // rows are dealt to the waves round robin
    nrows[i] = m < M ? reinterpret_cast<const f32x4*>(a.a + (size_t)m * a.lda) : nullptr;
  }
  if (wave < M) norm_rows_load<RB>(nr, nrows, a.norm_w, a.norm_w_is_bf16, nvec, lane);
  int r_pos[2] = {-1, -1}, r_seq[2] = {0, 0};
  if constexpr (EPI == DEPI_ROPE_KV) {
    const int lh = rope_lw >> 1;
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int e = threadIdx.x + j * blockDim.x;
      if (e < M * lh) {
        r_pos[j] = a.positions[e / lh];
        r_seq[j] = a.row_seq[e / lh];
      }
    }
  }
  __builtin_amdgcn_sched_barrier(0);
  u32x4 bq[D][NB];
  auto issue = [&](int d, int k) {
    const int ks = k < k_end ? k : k_begin;       // past the end: re-read the first step, never used
#pragma unroll
    for (int b = 0; b < NB; ++b) bq[d][b] = __builtin_amdgcn_raw_buffer_load_b128(rs_w[b], voff_w, ks * 2, 0);
  };
#pragma unroll
  for (int d = 0; d < D; ++d) issue(d, k_begin + 32 * d);
  __builtin_amdgcn_sched_barrier(0);

  // rotary epilogue: what this thread's (row, pair) items need is asked for now and used after the
  // product (at most 2 items a thread)
  int r_page[2] = {0, 0};
  float r_cos[2] = {1.f, 1.f}, r_sin[2] = {0.f, 0.f};
  if constexpr (EPI == DEPI_ROPE_KV) {
    const int half = a.head_dim >> 1, lh = rope_lw >> 1;
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int e = threadIdx.x + j * blockDim.x;
      const int pos = r_pos[j];
      if (e < M * lh && pos >= 0) {
        const int i = rope_base + e % lh;
        r_cos[j] = a.cos_table[(size_t)pos * half + i];
        r_sin[j] = a.sin_table[(size_t)pos * half + i];
        r_page[j] = a.block_table[(size_t)r_seq[j] * a.table_stride + pos / a.page_size];
      }
    }
  }

  // 2. the M rows into LDS as bfloat16, normalised
  for (int m0 = wave; m0 < M;) {
    norm_rows_finish<RB>(nr, nrows, a.norm_w_is_bf16, nvec, K, a.eps, lane, [&](int i, int c, u32x2 pk) {
      *reinterpret_cast<u32x2*>(xs + (size_t)(m0 + i * nwaves) * lds_row + 4 * c) = pk;
    });
    m0 += RB * nwaves;
    if (m0 >= M) break;
#pragma unroll
    for (int i = 0; i < RB; ++i) {
      const int m = m0 + i * nwaves;
      nrows[i] = m < M ? reinterpret_cast<const f32x4*>(a.a + (size_t)m * a.lda) : nullptr;
    }
    norm_rows_load<RB>(nr, nrows, a.norm_w, a.norm_w_is_bf16, nvec, lane);
  }
  __syncthreads();

  // 3. the product: A from LDS (rows past M read row 0; their results are thrown away), B from the ring
  const bf16_t* ap = xs + (size_t)(r < M ? r : 0) * lds_row + 8 * g;
  f32x4 acc[NB];
#pragma unroll
  for (int b = 0; b < NB; ++b) acc[b] = (f32x4){0.f, 0.f, 0.f, 0.f};
  constexpr int PA = 4;                            // A operands are read from LDS this many steps ahead
  static_assert(D % PA == 0, "the A look-ahead must divide the ring depth");
  u32x4 aq[PA];
  auto fetch_a = [&](int slot, int k) { aq[slot] = *reinterpret_cast<const u32x4*>(ap + (k < k_end ? k : k_begin)); };
#pragma unroll
  for (int j = 0; j < PA; ++j) fetch_a(j, k_begin + 32 * j);
  for (int k0 = k_begin; k0 < k_end; k0 += 32 * D) {
#pragma unroll
    for (int d = 0; d < D; ++d) {
      const int k = k0 + 32 * d;
      const u32x4 af = aq[d % PA];
      u32x4 bc[NB];
#pragma unroll
      for (int b = 0; b < NB; ++b) bc[b] = bq[d][b];
      if constexpr (!FULL) issue(d, k + 32 * D);
      fetch_a(d % PA, k + 32 * PA);
      __builtin_amdgcn_sched_barrier(0);
      if (k < k_end) {                             // scalar: a step past the segment's end is skipped
#pragma unroll
        for (int b = 0; b < NB; ++b)
          acc[b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(af), as_bf16x8(bc[b]), acc[b], 0, 0, 0);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  }

  // 4. epilogue
  if constexpr (EPI != DEPI_ROPE_KV) {
    if (!n_ok) return;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int m = 4 * g + q;
      if (m >= M) continue;
      const size_t o = (size_t)m * a.ldo + n0 + r;
      const float v = acc[0][q];
      if constexpr (EPI == DEPI_F32) ((float*)a.out)[o] = v;
      else if constexpr (EPI == DEPI_BF16) ((bf16_t*)a.out)[o] = f32_to_bf16(v);
      else if constexpr (EPI == DEPI_ADD_F32) ((float*)a.out)[o] += v;
      else {
        const float uv = acc[NB - 1][q];
        ((bf16_t*)a.out)[o] = f32_to_bf16(v * (1.0f / (1.0f + fast_exp(-v))) * uv);
      }
    }
  } else {
    // The workgroup's strips are one head or one pair of strips of it (S is 1 here); heads come
    // in the order q heads, k heads, v heads.  The 32-bit products go through LDS so that the
    // rotary pairs (i, i + hd/2), which sit in different strips, meet.
    const int hd = a.head_dim, half = hd >> 1, lw = rope_lw, lh = lw >> 1;
    __syncthreads();                               // every wave is done reading the rows
    float* os = reinterpret_cast<float*>(smem);    // [M][lw]
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int m = 4 * g + q;
      if (m < M) os[m * lw + 16 * wave + r] = acc[0][q];
    }
    __syncthreads();
    const int head = rope_head;
    const int q_dim = a.heads * hd;
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int e = threadIdx.x + j * blockDim.x;
      if (e >= M * lh) continue;
      const int m = e / lh, il = e % lh, i = rope_base + il;
      const int pos = r_pos[j];
      if (pos < 0) continue;
      const float x1 = os[m * lw + il], x2 = os[m * lw + il + lh];
      if (head < a.heads + a.kv_heads) {
        const float c = r_cos[j], s = r_sin[j];
        const float o1 = x1 * c - x2 * s;
        const float o2 = x2 * c + x1 * s;
        if (head < a.heads) {
          bf16_t* dst = (bf16_t*)a.out + (size_t)m * q_dim + (size_t)head * hd;
          dst[i] = f32_to_bf16(o1);
          dst[i + half] = f32_to_bf16(o2);
        } else if (a.write_cache) {
          bf16_t* dst = a.k_cache + (((size_t)r_page[j] * a.kv_heads + (head - a.heads)) * a.page_size + pos % a.page_size) * hd;
          dst[i] = f32_to_bf16(o1);
          dst[i + half] = f32_to_bf16(o2);
        }
      } else if (a.write_cache) {
        bf16_t* dst = a.v_cache + ((size_t)r_page[j] * a.kv_heads + (head - a.heads - a.kv_heads)) * hd * a.page_size + pos % a.page_size;
        dst[(size_t)i * a.page_size] = f32_to_bf16(x1);
        dst[(size_t)(i + half) * a.page_size] = f32_to_bf16(x2);
      }
    }
  }
}

static const size_t kMaxLds = 160 * 1024 - 1024;

template <int EPI, int D>
static int launch_decode_gemm(const DecodeGemmArgs& a, int waves, int blocks, hipStream_t s) {
  static bool raised = false;
  const size_t lds = (size_t)a.M * (a.K + 8) * sizeof(bf16_t);
  if (lds > kMaxLds) return -2;
  if (!raised) {   // more than 64 KB of dynamic LDS has to be asked for once
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(&decode_gemm_kernel<EPI, D>),
                            hipFuncAttributeMaxDynamicSharedMemorySize, (int)kMaxLds) != hipSuccess)
      return (int)hipGetLastError();
    raised = true;
  }
  hipLaunchKernelGGL((decode_gemm_kernel<EPI, D>), dim3(blocks), dim3(64 * waves), lds, s, a);
  return BW_LAUNCH_CHECK();
}

// Can the rows (M of them, K wide) live in LDS, and do the waves of a strip fit a workgroup?
static int check_decode_gemm(const DecodeGemmArgs& a) {
  if (a.M <= 0 || a.M > 16 || a.N <= 0 || a.K <= 0 || (a.K % 32)) return -2;
  if (a.K > DEC_SEG || (a.lda % 4) || a.lda < a.K) return -2;      // a row is normalised from a wave's registers
  if ((size_t)a.M * (a.K + 8) * sizeof(bf16_t) > kMaxLds) return -2;
  return 0;
}

extern "C" int bw_norm_gemm_supported(int M, int K) {
  DecodeGemmArgs a{};
  a.M = M; a.N = 16; a.K = K; a.lda = K;
  return check_decode_gemm(a) == 0;
}

extern "C" int bw_norm_gemm_bf16(const float* x, int ldx, const void* norm_w, int norm_w_is_bf16, float eps,
                                 const void* w, void* out, int ldo, int M, int N, int K, int epilogue, void* stream) {
  if (M <= 0 || N <= 0) return 0;
  DecodeGemmArgs a{};
  a.a = x; a.norm_w = norm_w; a.w = (const bf16_t*)w; a.out = out;
  a.M = M; a.N = N; a.K = K; a.lda = ldx; a.ldo = ldo; a.norm_w_is_bf16 = norm_w_is_bf16; a.eps = eps;
  const int bad = check_decode_gemm(a);
  if (bad) return bad;
  if (ldo < N) return -2;
  if ((reinterpret_cast<uintptr_t>(a.a) | reinterpret_cast<uintptr_t>(a.w)) & 15) return -3;
  const int waves = 4;                                   // strips per workgroup
  const int strips = (N + 15) / 16;
  const int blocks = (strips + waves - 1) / waves;
  hipStream_t s = (hipStream_t)stream;
  switch (epilogue) {
    case DEPI_F32: return launch_decode_gemm<DEPI_F32, 32>(a, waves, blocks, s);
    case DEPI_BF16: return launch_decode_gemm<DEPI_BF16, 32>(a, waves, blocks, s);
    case DEPI_ADD_F32: return launch_decode_gemm<DEPI_ADD_F32, 32>(a, waves, blocks, s);
    case DEPI_SWIGLU_BF16: return launch_decode_gemm<DEPI_SWIGLU_BF16, 20>(a, waves, blocks, s);
  }
  return -2;
}

extern "C" int bw_norm_qkv_rope_bf16(const float* x, int ldx, const void* norm_w, int norm_w_is_bf16, float eps,
                                     const void* w_qkv, void* q_out, const int32_t* positions,
                                     const int32_t* row_seq, const int32_t* block_table, int table_stride,
                                     const float* cos_table, const float* sin_table, void* k_cache, void* v_cache,
                                     int M, int heads, int kv_heads, int head_dim, int K, int page_size,
                                     int write_cache, void* stream) {
  if (M <= 0) return 0;
  if (head_dim % 16 || head_dim < 16 || page_size <= 0) return -4;
  const int pairs = (head_dim % 32 == 0) ? head_dim / 32 : 0;
  if (!pairs && head_dim > 64) return -4;            // a whole head per workgroup: one wave per strip, four at most
  DecodeGemmArgs a{};
  a.a = x; a.norm_w = norm_w; a.w = (const bf16_t*)w_qkv; a.out = q_out;
  a.M = M; a.N = (heads + 2 * kv_heads) * head_dim; a.K = K; a.lda = ldx; a.ldo = heads * head_dim;
  a.norm_w_is_bf16 = norm_w_is_bf16; a.eps = eps;
  a.positions = positions; a.row_seq = row_seq; a.block_table = block_table; a.cos_table = cos_table;
  a.sin_table = sin_table; a.k_cache = (bf16_t*)k_cache; a.v_cache = (bf16_t*)v_cache;
  a.heads = heads; a.kv_heads = kv_heads; a.head_dim = head_dim; a.page_size = page_size;
  a.table_stride = table_stride; a.write_cache = write_cache;
  a.pairs = pairs;
  const int bad = check_decode_gemm(a);
  if (bad) return bad;
  if ((reinterpret_cast<uintptr_t>(a.a) | reinterpret_cast<uintptr_t>(a.w)) & 15) return -3;
  if ((size_t)(pairs ? 32 : head_dim) * sizeof(float) > (size_t)(K + 8) * sizeof(bf16_t)) return -2;   // the epilogue reuses the LDS rows
  const int all_heads = heads + 2 * kv_heads;
  if (pairs) return launch_decode_gemm<DEPI_ROPE_KV, 64>(a, 2, all_heads * pairs, (hipStream_t)stream);
  return launch_decode_gemm<DEPI_ROPE_KV, 64>(a, head_dim / 16, all_heads, (hipStream_t)stream);
}
