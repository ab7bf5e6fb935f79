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
// rotary: the strips of one head, or one strip and its rotary partner).  A wave's weights stream
// through a ring of its own in LDS: buffer loads with LDS as destination, 8 rows of 128 bytes an
// instruction (whole cache lines), the 16-byte chunks of a row permuted so that operand reads hit
// distinct banks; no registers hold weights, so the ring is deep.  Loads complete in the order
// they are issued and the wait for a stage counts the loads issued after it, so everything else
// the kernel reads from memory is asked for before the ring: positions and what the rotary
// epilogue needs first (a short wait at the kernel's start), then the rows to normalise, then the
// ring's first stages, which are in flight while the rows are normalised into LDS (rows padded by
// 16 bytes so that operand reads hit distinct banks).  Then each wave runs its chain with both
// operands from LDS.  K a multiple of 64.
#include "common.h"
#include "api.h"

// in gemm_bf16.hip
int bw_norm_gemm_mid(const float* x32, int ldx32, const void* norm_w, int norm_w_is_bf16, float eps, const void* w, void* out,
                     int ldo, int M, int N, int K, int epilogue, void* stream);

int bw_norm_qkv_rope_mid(const float* x32, int ldx32, const void* norm_w, int norm_w_is_bf16, float eps, const void* w_qkv,
                         void* q_out, const int32_t* positions, const int32_t* row_seq, const int32_t* block_table,
                         int table_stride, const float* cos_table, const float* sin_table, void* k_cache, void* v_cache, int M,
                         int heads, int kv_heads, int head_dim, int K, int page_size, int write_cache, void* stream);

int bw_chain_flush_open(void* stream);

enum { DEPI_F32 = 0, DEPI_BF16 = 1, DEPI_ADD_F32 = 2, DEPI_SWIGLU_BF16 = 3, DEPI_ROPE_KV = 4 };

// (DEC_SEG, the LDS layout of the rows and the rings, and what the launchers admit: layout.h)

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

// ST: stages of a wave's ring
template <int EPI, int ST>
struct DecodeShape {
  static constexpr int NB = (EPI == DEPI_SWIGLU_BF16) ? 2 : 1;
  static constexpr int STAGES = ST;
  static constexpr int STAGE = NB * 2048;                                      // 16 rows of W, 128 bytes each, NB times
  static constexpr int LPW = 2 * NB;                                           // loads a stage
  static_assert(LPW * (STAGES - 2) < 64, "the wait count has six bits");
};

// A wave's loads of one stage of its ring (step past the end: outside the descriptors, zeros, no traffic).
template <int EPI, int ST>
__device__ __forceinline__ void decode_issue(unsigned char* ring, const __amdgpu_buffer_rsrc_t* rs_w, const int* voff_w,
                                             int step, int steps) {
  using SH = DecodeShape<EPI, ST>;
  typedef __attribute__((address_space(3))) void* lds_ptr;
  unsigned char* dst = ring + (step % SH::STAGES) * SH::STAGE;
  const bool real = step < steps;                 // scalar
#pragma unroll
  for (int b = 0; b < SH::NB; ++b)
#pragma unroll
    for (int t = 0; t < 2; ++t)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_w[b], (lds_ptr)(dst + b * 2048 + t * 1024), 16, real ? voff_w[t] : 0x7ffffff0,
                                               step * 128, 0, 0);
}

// The rows of the residual stream, normalised into LDS as bfloat16: wave ``wave`` has rows wave, wave + nwaves,
// ..., RB of them at a time.  The ring's first stages are asked for after the first batch's loads and before its
// arithmetic, so that they stay in flight meanwhile.  (A second batch, with more than RB rows a wave, is loaded
// after the ring's first stages; the compiler's wait for it also waits for those, so the caller's wait counts hold.)
template <int RB, int EPI, int ST>
__device__ __forceinline__ void decode_norm_rows(const DecodeGemmArgs& a, int wave, int nwaves, int lane, bf16_t* xs, int lds_row,
                                                 unsigned char* ring, const __amdgpu_buffer_rsrc_t* rs_w, const int* voff_w,
                                                 int steps) {
  using SH = DecodeShape<EPI, ST>;
  const int M = a.M, K = a.K, nvec = K >> 2;
  NormRows<RB> nr;
  const f32x4* nrows[RB];
#pragma unroll
  for (int i = 0; i < RB; ++i) {
    const int m = wave + i * nwaves;               // rows are dealt to the waves round robin
    nrows[i] = m < M ? reinterpret_cast<const f32x4*>(a.a + (size_t)m * a.lda) : nullptr;
  }
  if (wave < M) norm_rows_load<RB>(nr, nrows, a.norm_w, a.norm_w_is_bf16, nvec, lane);
  __builtin_amdgcn_sched_barrier(0);
#pragma unroll
  for (int st = 0; st < SH::STAGES - 1; ++st) decode_issue<EPI, ST>(ring, rs_w, voff_w, st, steps);
  __builtin_amdgcn_sched_barrier(0);
  for (int m0 = wave; m0 < M;) {
    norm_rows_finish<RB>(nr, nrows, a.norm_w_is_bf16, nvec, K, a.eps, lane, [&](int i, int c, u32x2 pk) {
      *reinterpret_cast<u32x2*>(xs + decode_norm_store_elem(m0 + i * nwaves, c, K)) = pk;
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
}

template <int EPI, int ST>
__global__ __launch_bounds__(256) void decode_gemm_kernel(DecodeGemmArgs a) {
  using SH = DecodeShape<EPI, ST>;
  constexpr int NB = SH::NB;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  const int K = a.K, M = a.M;
  const int lds_row = decode_lds_row(K);          // bf16 elements; +16 bytes keeps operand reads conflict-free
  bf16_t* xs = reinterpret_cast<bf16_t*>(smem);   // [M][lds_row], then the waves' rings
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
  // weights through buffer descriptors that cover the strip's rows (rows past N read as zeros):
  // one per-lane offset for the whole kernel, the step's offset in a scalar register
  const int w_rows = min(16, a.N - n0);
  __amdgpu_buffer_rsrc_t rs_w[NB];
#pragma unroll
  for (int b = 0; b < NB; ++b)
    rs_w[b] = __builtin_amdgcn_make_buffer_rsrc((void*)(a.w + ((size_t)b * a.N + n0) * K), 0,
                                                (int)((size_t)(w_rows > 0 ? w_rows : 0) * K * 2), 0x00020000);
  // loads: lane l fetches row l / 8 of its 8, chunk (l % 8) ^ (row within 16 >> 1) of the row's 128 bytes
  const int lrow = lane >> 3, lslot = lane & 7;
  int voff_w[2];
#pragma unroll
  for (int t = 0; t < 2; ++t) voff_w[t] = ((8 * t + lrow) * K + 8 * (lslot ^ ((8 * t + lrow) >> 1))) * 2;
  const int steps = K / 64;
  unsigned char* ring = smem + decode_ring_offset(M, K, wave, SH::STAGES, SH::STAGE);

  // 1. Everything but weights is asked for before the ring (see the head of the file).  The rotary
  // epilogue's items first: what this thread's (row, pair) items need (at most 2 items a thread).
  int r_pos[2] = {-1, -1}, r_page[2] = {0, 0};
  float r_cos[2] = {1.f, 1.f}, r_sin[2] = {0.f, 0.f};
  if constexpr (EPI == DEPI_ROPE_KV) {
    const int half = a.head_dim >> 1, lh = rope_lw >> 1;
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int e = threadIdx.x + j * blockDim.x;
      if (e < M * lh) {
        const int pos = a.positions[e / lh];
        r_pos[j] = pos;
        if (pos >= 0) {
          const int i = rope_base + e % lh;
          r_cos[j] = a.cos_table[(size_t)pos * half + i];
          r_sin[j] = a.sin_table[(size_t)pos * half + i];
          r_page[j] = a.block_table[(size_t)a.row_seq[e / lh] * a.table_stride + pos / a.page_size];
        }
      }
    }
    // these loads stay here, before the ring's: the waits in the loop count the loads issued after a stage's own,
    // and must find nothing but the ring's among them
    asm volatile("" ::: "memory");
  }
  __builtin_amdgcn_sched_barrier(0);
  // then the rows to normalise, the ring's first stages asked for between their loads and the arithmetic; a wave
  // fetches as many rows at a time as it has (four at most)
  const int rows_a_wave = (M + nwaves - 1) / nwaves;
  if (rows_a_wave <= 1) decode_norm_rows<1, EPI, ST>(a, wave, nwaves, lane, xs, lds_row, ring, rs_w, voff_w, steps);
  else if (rows_a_wave == 2) decode_norm_rows<2, EPI, ST>(a, wave, nwaves, lane, xs, lds_row, ring, rs_w, voff_w, steps);
  else if (rows_a_wave == 3) decode_norm_rows<3, EPI, ST>(a, wave, nwaves, lane, xs, lds_row, ring, rs_w, voff_w, steps);
  else decode_norm_rows<4, EPI, ST>(a, wave, nwaves, lane, xs, lds_row, ring, rs_w, voff_w, steps);
  __syncthreads();

  // 3. the product: A from the rows in LDS (rows past M read row 0; their results are thrown away), B from
  // the wave's ring.
  const bf16_t* ap = xs + decode_operand_elem(r, M, g, 0, 0, K);
  int off_w[2];
#pragma unroll
  for (int kk = 0; kk < 2; ++kk) off_w[kk] = decode_ring_operand_offset(r, g, kk);
  f32x4 acc[NB];
#pragma unroll
  for (int b = 0; b < NB; ++b) acc[b] = (f32x4){0.f, 0.f, 0.f, 0.f};
  for (int step = 0; step < steps; ++step) {
    __builtin_amdgcn_s_waitcnt(vmcnt_only(SH::LPW * (SH::STAGES - 2)));   // all but the loads of the stages after this one have landed
    asm volatile("" ::: "memory");
    const unsigned char* stage = ring + (step % SH::STAGES) * SH::STAGE;
    u32x4 fa[2], fb[2][NB];
#pragma unroll
    for (int kk = 0; kk < 2; ++kk) {
      fa[kk] = *reinterpret_cast<const u32x4*>(ap + 64 * step + 32 * kk);
#pragma unroll
      for (int b = 0; b < NB; ++b) fb[kk][b] = *reinterpret_cast<const u32x4*>(stage + b * 2048 + off_w[kk]);
    }
#pragma unroll
    for (int kk = 0; kk < 2; ++kk)
#pragma unroll
      for (int b = 0; b < NB; ++b)
        acc[b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(fa[kk]), as_bf16x8(fb[kk][b]), acc[b], 0, 0, 0);
    asm volatile("" ::: "memory");
    decode_issue<EPI, ST>(ring, rs_w, voff_w, step + SH::STAGES - 1, steps);   // into the stage of the step before
  }
  __builtin_amdgcn_s_waitcnt(vmcnt_only(0));       // the padding loads too, before LDS is used for anything else

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
        ((bf16_t*)a.out)[o] = f32_to_bf16(silu_times(v, uv));
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

static const size_t kMaxLds = DEC_MAX_LDS;

template <int EPI, int ST>
static int launch_decode_gemm(const DecodeGemmArgs& a, int waves, int blocks, hipStream_t s) {
  static bool raised = false;
  using SH = DecodeShape<EPI, ST>;
  const size_t lds = decode_lds_bytes(a.M, a.K, waves, SH::STAGES, SH::STAGE);
  if (lds > kMaxLds) return -2;
  if (!raised) {   // more than 64 KB of dynamic LDS has to be asked for once
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(&decode_gemm_kernel<EPI, ST>),
                            hipFuncAttributeMaxDynamicSharedMemorySize, (int)kMaxLds) != hipSuccess)
      return (int)hipGetLastError();
    raised = true;
  }
  (void)bw_chain_flush_open((void*)s);              // phases that wait in an open chain go first
  hipLaunchKernelGGL((decode_gemm_kernel<EPI, ST>), dim3(blocks), dim3(64 * waves), lds, s, a);
  return BW_LAUNCH_CHECK();
}

// Can the rows (M of them, K wide) live in LDS, and do the waves of a strip fit a workgroup?
static int check_decode_gemm(const DecodeGemmArgs& a) {
  return decode_gemm_admits(a.M, a.N, a.K, a.lda) ? 0 : -2;      // (a row is normalised from a wave's registers)
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
  if (ldo < N || (ldx % 4) || ldx < K) return -2;
  if ((reinterpret_cast<uintptr_t>(a.a) | reinterpret_cast<uintptr_t>(a.w)) & 15) return -3;
  // many columns: the kernel whose workgroups share the normalised rows among their strips and one ring (it alone
  // takes rows of two segments of K)
  const int mid = bw_norm_gemm_mid(x, ldx, norm_w, norm_w_is_bf16, eps, w, out, ldo, M, N, K, epilogue, stream);
  if (mid != -7) return mid;
  const int bad = check_decode_gemm(a);
  if (bad) return bad;
  const int waves = 4;                                   // strips per workgroup (their rings: 64 KB of LDS)
  const int strips = (N + 15) / 16;
  const int blocks = (strips + waves - 1) / waves;
  hipStream_t s = (hipStream_t)stream;
  switch (epilogue) {
    case DEPI_F32: return launch_decode_gemm<DEPI_F32, 8>(a, waves, blocks, s);
    case DEPI_BF16: return launch_decode_gemm<DEPI_BF16, 8>(a, waves, blocks, s);
    case DEPI_ADD_F32: return launch_decode_gemm<DEPI_ADD_F32, 8>(a, waves, blocks, s);
    case DEPI_SWIGLU_BF16: return launch_decode_gemm<DEPI_SWIGLU_BF16, 4>(a, waves, blocks, s);
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
  if ((a.lda % 4) || a.lda < K || K <= 0 || (K % 64) || M > 16) return -2;
  if ((reinterpret_cast<uintptr_t>(a.a) | reinterpret_cast<uintptr_t>(a.w)) & 15) return -3;
  if ((size_t)(pairs ? 32 : head_dim) * sizeof(float) > (size_t)(K + 8) * sizeof(bf16_t)) return -2;   // the epilogue reuses the LDS rows
  // many heads of 64: the kernel whose workgroups are a head each, four strips sharing the normalised rows and one ring
  const int mid = bw_norm_qkv_rope_mid(x, ldx, norm_w, norm_w_is_bf16, eps, w_qkv, q_out, positions, row_seq, block_table,
                                       table_stride, cos_table, sin_table, k_cache, v_cache, M, heads, kv_heads, head_dim, K,
                                       page_size, write_cache, stream);
  if (mid != -7) return mid;
  const int bad = check_decode_gemm(a);
  if (bad) return bad;
  const int all_heads = heads + 2 * kv_heads;
  if (pairs) return launch_decode_gemm<DEPI_ROPE_KV, 10>(a, 2, all_heads * pairs, (hipStream_t)stream);
  return launch_decode_gemm<DEPI_ROPE_KV, 10>(a, head_dim / 16, all_heads, (hipStream_t)stream);
}
