// Part of gemm_bf16.hip (included there, after its epilogues and launch macro; not a unit of its own):
// the tile kernels of prompt portions: the tiles' epilogue, 128 x 128 tiles from registers, 256 x 256, 128 x 128 and 128 x 256 tiles through LDS rings.
#pragma once

// ------------------------------------------------------------------------------ tile epilogue

// What a wave does with its NI x 4 accumulators (16 x 16 outputs each: rows row0 + 16 i + 4 g + q,
// columns 16 j + r of the wave's 64).  Plain epilogues: output columns col0 + 16 j + r.  SwiGLU:
// accumulators j = 0, 1 are gate columns col0 + 16 j + r, j = 2, 3 the up columns of the same outputs.
// Rotary q|k|v: the wave's 64 columns are head ``head``; accumulators j and j + 2 hold the rotary pairs
// (d, d + 32) in the same lane; q heads go to the q buffer, k heads rotated and v heads as they are to
// the row's page slot (v transposed).  ``residual_in``: the values already contain the residual.
template <int EPI, int NI>
__device__ __forceinline__ void tile_epilogue(const f32x4 (&acc)[NI][4], void* __restrict__ out, int M, int N, int ldo,
                                              int row0, int col0, int head, int r, int g, bool residual_in,
                                              const QkvRopeArgs& rp) {
  // Rotary: what the rows need from memory (position, then the page it selects) is asked for at once for all of
  // them, from addresses that are always valid, so that the waits for it are two and not two a row.
  constexpr int NR = EPI == EPI_QKV_ROPE ? NI : 1;
  int pos_all[NR][4], page_all[NR][4];
  if constexpr (EPI == EPI_QKV_ROPE) {
#pragma unroll
    for (int i = 0; i < NI; ++i)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int m = row0 + 16 * i + 4 * g + q;
        pos_all[i][q] = rp.positions[m < M ? m : M - 1];
      }
#pragma unroll
    for (int i = 0; i < NI; ++i)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int m = row0 + 16 * i + 4 * g + q;
        const int seq = rp.row_seq[m < M ? m : M - 1];
        const int pidx = (pos_all[i][q] > 0 ? pos_all[i][q] : 0) >> rp.page_shift;
        page_all[i][q] = head >= rp.heads ? rp.block_table[(size_t)seq * rp.table_stride + pidx] : 0;
      }
  }
#pragma unroll
  for (int i = 0; i < NI; ++i) {
    // Rotary: the cosines and sines of the block's four rows are asked for together, from addresses that are
    // always valid (a padding row's position counts as 0), so that their latency is paid once a block, not once a row.
    float cs[4][2], sn[4][2];
    if constexpr (EPI == EPI_QKV_ROPE) {
      if (head < rp.heads + rp.kv_heads) {
#pragma unroll
        for (int q = 0; q < 4; ++q)
#pragma unroll
          for (int j = 0; j < 2; ++j) {
            const size_t at = (size_t)(pos_all[i][q] > 0 ? pos_all[i][q] : 0) * 32 + 16 * j + r;
            cs[q][j] = rp.cos_table[at];
            sn[q][j] = rp.sin_table[at];
          }
      }
    }
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int m = row0 + 16 * i + 4 * g + q;
      if (m >= M) continue;
      if constexpr (EPI == EPI_QKV_ROPE) {
        const int pos = pos_all[i][q];
        if (head >= rp.heads + 2 * rp.kv_heads || pos < 0) continue;
        const int q_dim = rp.heads * 64;
        const size_t page = (size_t)page_all[i][q];
        const int slot = pos & (rp.page_size - 1);
        if (head < rp.heads + rp.kv_heads) {
          bf16_t* dst = head < rp.heads ? (bf16_t*)out + (size_t)m * q_dim + (size_t)head * 64
                                        : rp.k_cache + ((page * rp.kv_heads + (head - rp.heads)) * rp.page_size + slot) * 64;
          if (head < rp.heads || rp.write_cache) {
#pragma unroll
            for (int j = 0; j < 2; ++j) {
              const int d = 16 * j + r;
              const float c = cs[q][j], s = sn[q][j];
              const float x1 = acc[i][j][q], x2 = acc[i][j + 2][q];
              const float o1 = x1 * c - x2 * s;
              const float o2 = x2 * c + x1 * s;
              dst[d] = f32_to_bf16(o1);
              dst[d + 32] = f32_to_bf16(o2);
            }
          }
        } else if (rp.write_cache) {
          // values lie transposed in their page ([d][slot]).  The lane's four rows are most often four consecutive
          // slots of one page starting at a multiple of four: then the first row stores all four at once.
          bool quad = row0 + 16 * i + 4 * g + 3 < M && (pos_all[i][0] & 3) == 0;
#pragma unroll
          for (int t = 1; t < 4; ++t) quad = quad && pos_all[i][t] == pos_all[i][0] + t && page_all[i][t] == page_all[i][0];
          bf16_t* dst = rp.v_cache + (page * rp.kv_heads + (head - rp.heads - rp.kv_heads)) * 64 * rp.page_size + slot;
          if (quad) {
            if (q == 0) {
#pragma unroll
              for (int j = 0; j < 4; ++j) {
                const u32x2 four = {pack_bf16x2(acc[i][j][0], acc[i][j][1]), pack_bf16x2(acc[i][j][2], acc[i][j][3])};
                *reinterpret_cast<u32x2*>(dst + (size_t)(16 * j + r) * rp.page_size) = four;
              }
            }
          } else {
#pragma unroll
            for (int j = 0; j < 4; ++j) dst[(size_t)(16 * j + r) * rp.page_size] = f32_to_bf16(acc[i][j][q]);
          }
        }
      } else if constexpr (EPI == EPI_SWIGLU_BF16) {
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          const int n = col0 + 16 * j + r;
          if (n < N) epilogue_store<EPI>(out, (size_t)m * ldo + n, acc[i][j][q], acc[i][j + 2][q]);
        }
      } else {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const int n = col0 + 16 * j + r;
          if (n >= N) continue;
          if (EPI == EPI_ADD_F32 && residual_in) ((float*)out)[(size_t)m * ldo + n] = acc[i][j][q];
          else epilogue_store<EPI>(out, (size_t)m * ldo + n, acc[i][j][q], acc[i][j][q]);
        }
      }
    }
  }
}

// ------------------------------------------------------------------------------ wide

#define WIDE_BM 128
#define WIDE_BN 128
#define WIDE_BK 64
#define WIDE_LDS_ROW 72   // bf16 elements per LDS row: 64 of data + 8 of padding (144 bytes)

template <int EPI, bool MULTI, bool FAST>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2))) void gemm_bf16_wide_kernel(const bf16_t* __restrict__ x, const bf16_t* __restrict__ w,
                                                             void* __restrict__ out, int M, int N, int K, int ldx,
                                                             int ldo, int m_tiles, int n_tiles, QkvRopeArgs rp) {
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

  // This thread's share of the global -> LDS copies: rows lr + 32j, 16-byte chunk lc.  The loads
  // go through buffer descriptors that cover exactly the block's rows of x and of W, so a row
  // past M or N reads as zeros by itself and one 32-bit offset per operand is all a thread keeps.
  const int lr = tid >> 3, lc = tid & 7;
  const int a_rows = min(WIDE_BM, M - m0);
  const __amdgpu_buffer_rsrc_t rs_a = __builtin_amdgcn_make_buffer_rsrc(
      (void*)(x + (size_t)m0 * ldx), 0, (int)((((size_t)a_rows - 1) * ldx + K) * 2), 0x00020000);
  const int b_rows = min(COLS, N - n0);              // gate rows and up rows alike in SwiGLU mode
  const __amdgpu_buffer_rsrc_t rs_b0 =
      __builtin_amdgcn_make_buffer_rsrc((void*)(w + (size_t)n0 * K), 0, (int)((size_t)b_rows * K * 2), 0x00020000);
  const __amdgpu_buffer_rsrc_t rs_b1 = __builtin_amdgcn_make_buffer_rsrc(
      (void*)(w + ((size_t)N + n0) * K), 0, (int)((size_t)b_rows * K * 2), 0x00020000);
  const int voff_a = (lr * ldx + lc * 8) * 2, voff_b = (lr * K + lc * 8) * 2;
  // LDS rows of this wave's four B tiles
  int brow[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    if constexpr (EPI == EPI_SWIGLU_BF16) brow[j] = (j >> 1) * 64 + 32 * wx + 16 * (j & 1);
    else brow[j] = 64 * wx + 16 * j;
  }

  static_assert(!(MULTI && FAST), "the fast path is for one segment");
  constexpr bool TOT = MULTI;
  f32x4 acc[4][4], tot[TOT ? 4 : 1][TOT ? 4 : 1];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      acc[i][j] = (f32x4){0.f, 0.f, 0.f, 0.f};
      if constexpr (TOT) tot[i][j] = (f32x4){0.f, 0.f, 0.f, 0.f};
    }

  // Tiles travel global -> registers -> LDS.  A tile is asked for two steps before it is used
  // and parked in one of two register sets meanwhile, so that a load has about two steps of
  // matrix work to arrive in; it is written to LDS (two buffers) one step before its use.
  // Loads are unconditional; a chunk past K (it would read the next row) is zeroed when it is
  // written to LDS.
  const u32x4 zero = {0u, 0u, 0u, 0u};
  u32x4 ra[2][4], rb[2][4];
  auto fetch = [&](int set, int k0) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      ra[set][j] = __builtin_amdgcn_raw_buffer_load_b128(rs_a, voff_a, (32 * j * ldx + k0) * 2, 0);
      if constexpr (EPI == EPI_SWIGLU_BF16)
        rb[set][j] = __builtin_amdgcn_raw_buffer_load_b128(j < 2 ? rs_b0 : rs_b1, voff_b, (32 * (j & 1) * K + k0) * 2, 0);
      else
        rb[set][j] = __builtin_amdgcn_raw_buffer_load_b128(rs_b0, voff_b, (32 * j * K + k0) * 2, 0);
    }
  };
  auto stash = [&](int set, int buf, int k0) {
    // the loaded registers are only ever read here: writing zeros into them instead would make
    // the compiler wait for every load in flight first
    if (k0 + WIDE_BK > K) {                           // a last step that K does not fill
      const bool in = k0 + lc * 8 < K;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        *reinterpret_cast<u32x4*>(&lds_a[buf][(lr + 32 * j) * WIDE_LDS_ROW + lc * 8]) = in ? ra[set][j] : zero;
        *reinterpret_cast<u32x4*>(&lds_b[buf][(lr + 32 * j) * WIDE_LDS_ROW + lc * 8]) = in ? rb[set][j] : zero;
      }
    } else {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        *reinterpret_cast<u32x4*>(&lds_a[buf][(lr + 32 * j) * WIDE_LDS_ROW + lc * 8]) = ra[set][j];
        *reinterpret_cast<u32x4*>(&lds_b[buf][(lr + 32 * j) * WIDE_LDS_ROW + lc * 8]) = rb[set][j];
      }
    }
  };
  auto step = [&](int k0, int buf) {
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
    if constexpr (TOT) {
      const int kn = k0 + WIDE_BK;
      if (kn % GEMM_SEG == 0 || kn >= K) {          // a segment ends: join it to the total, left to right
        const bool first = k0 < GEMM_SEG;
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            if constexpr (EPI == EPI_ADD_F32) {
              if (first) {                          // the chain of additions starts at the residual
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                  const int m = m0 + 64 * wy + 16 * i + 4 * g + q, n = n0 + 64 * wx + 16 * j + r;
                  tot[i][j][q] = (m < M && n < N) ? ((const float*)out)[(size_t)m * ldo + n] : 0.0f;
                }
              }
              tot[i][j] = tot[i][j] + acc[i][j];
            } else {
              tot[i][j] = first ? acc[i][j] : tot[i][j] + acc[i][j];
            }
            acc[i][j] = (f32x4){0.f, 0.f, 0.f, 0.f};
          }
      }
    }
  };

  fetch(0, 0);
  fetch(1, WIDE_BK);
  stash(0, 0, 0);
  __syncthreads();
  if constexpr (FAST) {
    // K is a multiple of 128: every step is whole, and a step's body is one straight run of
    // instructions that the scheduler is told how to interleave, so that the LDS traffic and the
    // global loads hide behind the matrix instructions of the same wave:
    //   8 operand reads (first half of the step);
    //   8 x [2 matrix instructions, 1 operand read (second half), 1 global load (the tile after next)];
    //   8 x [2 matrix instructions, 1 LDS write (the next tile, loaded a step ago)].
    // (What then bounds the kernel is how many bytes of tile loads a compute unit can keep in
    // flight: about 45 KB, which at the latency of the L2 is a little more than the 64 KB a step
    // of two resident workgroups asks for.)
    auto fast_step = [&](int k0, int set_fetch, int buf) {
      const int set_stash = set_fetch ^ 1;
      fetch(set_fetch, k0 + 2 * WIDE_BK);             // past K: outside the descriptors, zeros, never used
      u32x4 fa[2][4], fb[2][4];
#pragma unroll
      for (int kk = 0; kk < 2; ++kk) {
#pragma unroll
        for (int i = 0; i < 4; ++i)
          fa[kk][i] = *reinterpret_cast<const u32x4*>(&lds_a[buf][(64 * wy + 16 * i + r) * WIDE_LDS_ROW + kk * 32 + g * 8]);
#pragma unroll
        for (int j = 0; j < 4; ++j)
          fb[kk][j] = *reinterpret_cast<const u32x4*>(&lds_b[buf][(brow[j] + r) * WIDE_LDS_ROW + kk * 32 + g * 8]);
      }
#pragma unroll
      for (int kk = 0; kk < 2; ++kk)
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
          for (int j = 0; j < 4; ++j)
            acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(fa[kk][i]), as_bf16x8(fb[kk][j]), acc[i][j], 0, 0, 0);
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        *reinterpret_cast<u32x4*>(&lds_a[buf ^ 1][(lr + 32 * j) * WIDE_LDS_ROW + lc * 8]) = ra[set_stash][j];
        *reinterpret_cast<u32x4*>(&lds_b[buf ^ 1][(lr + 32 * j) * WIDE_LDS_ROW + lc * 8]) = rb[set_stash][j];
      }
      __builtin_amdgcn_sched_group_barrier(0x100, 8, 0);
#pragma unroll
      for (int t = 0; t < 8; ++t) {
        __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
      }
#pragma unroll
      for (int t = 0; t < 8; ++t) {
        __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);
        __builtin_amdgcn_sched_group_barrier(0x200, 1, 0);
      }
      __syncthreads();
    };
    for (int k0 = 0; k0 < K; k0 += 2 * WIDE_BK) {
      fast_step(k0, 0, 0);
      fast_step(k0 + WIDE_BK, 1, 1);
    }
  } else
  // steps in pairs, so that register sets and buffers are named at compile time
  for (int k0 = 0; k0 < K; k0 += 2 * WIDE_BK) {
    fetch(0, k0 + 2 * WIDE_BK);
    step(k0, 0);
    stash(1, 1, k0 + WIDE_BK);
    __syncthreads();
    if (k0 + WIDE_BK >= K) break;
    fetch(1, k0 + 3 * WIDE_BK);
    step(k0 + WIDE_BK, 1);
    stash(0, 0, k0 + 2 * WIDE_BK);
    __syncthreads();
  }

  if constexpr (TOT) {
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) acc[i][j] = tot[TOT ? i : 0][TOT ? j : 0];
  }
  tile_epilogue<EPI, 4>(acc, out, M, N, ldo, m0 + 64 * wy, n0 + (EPI == EPI_SWIGLU_BF16 ? 32 : 64) * wx, (n0 >> 6) + wx, r, g,
                        TOT, rp);
}

// ------------------------------------------------------------------------------ big tiles

// 256 x 256 outputs a workgroup (256 x 128 of SwiGLU: 128 gate and 128 up rows of W), steps of 64
// along K, eight waves of 128 x 64 outputs each.  A compute unit can keep only so many bytes of
// loads in flight, so what it computes per byte it loads decides how busy its matrix cores are:
// this tile computes twice as much per byte as the 128 x 128 one.  Tiles travel from memory straight
// into LDS (buffer loads with LDS as their destination: no registers, no LDS write instructions).
// One load instruction of a wave brings 8 rows of a step, 128 bytes each (whole cache lines), into
// 1 KB of LDS, lane l's 16 bytes to 16 * l.  Which 16 bytes of its row a lane fetches is permuted:
// slot c' of row r (r counted within its block of 16 rows) holds the row's chunk c' ^ (r >> 1), so
// that the 16 lanes that read one chunk of 16 different rows as a matrix operand hit 16 different
// groups of banks.  LDS is a ring of five slots of 32 KB, filled in the order A0 B0 A1 B1 A2 ... (a
// step's tile of x, then its tile of W): while the waves work on step s, B(s+1) and A(s+2) are in
// flight and A(s+1) has landed or is landing, so the memory pipe never runs dry at a step's edge;
// one barrier a step.  Rows past M or N lie outside the buffer descriptors.  K a multiple of 64 and
// one segment; for products with enough tiles to go round.
#define BIG_BM 256
#define BIG_SLOT (32 * 1024)
#define BIG_SLOTS 5
#define BIG_WAIT_ALL 0x0f70     // s_waitcnt vmcnt(0) alone
#define BIG_WAIT_BUT_4 0x0f74   // s_waitcnt vmcnt(4): all but the wave's last four loads have landed

template <int EPI>
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(2, 2))) void gemm_bf16_big_kernel(
    const bf16_t* __restrict__ x, const bf16_t* __restrict__ w, void* __restrict__ out, int M, int N, int K, int ldx,
    int ldo, int m_tiles, int n_tiles, QkvRopeArgs rp, size_t seg_stride) {
  constexpr bool GLU = EPI == EPI_SWIGLU_BF16;
  constexpr int COLS = GLU ? 128 : 256;
  extern __shared__ __attribute__((aligned(16))) unsigned char big_lds[];   // [5 slots][32 KB]
  // gridDim.y > 1: workgroup (tile, y) works on segment y of K alone and leaves its sums at out + y * seg_stride
  // elements (a residual add's segments, joined in order by add_segments_kernel afterwards)
  const int k_base = (int)blockIdx.y * GEMM_SEG;
  if (gridDim.y > 1) out = (void*)((float*)out + (size_t)blockIdx.y * seg_stride);
  const int wave = wave_index(), lane = threadIdx.x & 63;
  const int r = lane & 15, g = lane >> 4;
  const int wy = wave >> 2, wx = wave & 3;
  int bid = blockIdx.x;
  const int nblocks = m_tiles * n_tiles;
  if (nblocks % 8 == 0) bid = (bid % 8) * (nblocks / 8) + bid / 8;      // an n tile's workgroups share an XCD
  const int m0 = (bid % m_tiles) * BIG_BM;
  const int n0 = (bid / m_tiles) * COLS;

  // this wave's loads of a stage: rows 32*wave .. 32*wave + 31 of A's 256 and of B's 256, four loads of 8 rows each
  const int a_rows = min(BIG_BM, M - m0), b_rows = min(COLS, N - n0);
  const __amdgpu_buffer_rsrc_t rs_a = __builtin_amdgcn_make_buffer_rsrc(
      (void*)(x + (size_t)m0 * ldx), 0, (int)((((size_t)a_rows - 1) * ldx + K) * 2), 0x00020000);
  // SwiGLU: B rows 0-127 are gate rows n0.., 128-255 the up rows N + n0..
  const bool up = GLU && wave >= 4;
  const __amdgpu_buffer_rsrc_t rs_b = __builtin_amdgcn_make_buffer_rsrc(
      (void*)(w + ((size_t)(up ? N : 0) + n0) * K), 0, (int)((size_t)b_rows * K * 2), 0x00020000);
  const int b_row0 = GLU ? 32 * (wave & 3) : 32 * wave;
  const int lrow = lane >> 3, lslot = lane & 7;
  int voff_a[4], voff_b[4];
#pragma unroll
  for (int t = 0; t < 4; ++t) {
    const int r16 = (8 * t + lrow) & 15;                    // the row within its block of 16
    const int chunk = lslot ^ (r16 >> 1);
    voff_a[t] = ((32 * wave + 8 * t + lrow) * ldx + 8 * chunk) * 2;
    voff_b[t] = ((b_row0 + 8 * t + lrow) * K + 8 * chunk) * 2;
  }
  typedef __attribute__((address_space(3))) void* lds_ptr;
  // load number n of the ring: A of step n / 2 (n even) or B of it (n odd), into slot n % 5
  auto issue_a = [&](int step) {
    unsigned char* dst = big_lds + ((2 * step) % BIG_SLOTS) * BIG_SLOT + (4 * wave) * 1024;
#pragma unroll
    for (int t = 0; t < 4; ++t)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_a, (lds_ptr)(dst + t * 1024), 16, voff_a[t], k_base * 2 + step * 128, 0, 0);
  };
  auto issue_b = [&](int step) {
    unsigned char* dst = big_lds + ((2 * step + 1) % BIG_SLOTS) * BIG_SLOT + (4 * wave) * 1024;
#pragma unroll
    for (int t = 0; t < 4; ++t)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_b, (lds_ptr)(dst + t * 1024), 16, voff_b[t], k_base * 2 + step * 128, 0, 0);
  };

  f32x4 acc[8][4];
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = (f32x4){0.f, 0.f, 0.f, 0.f};
  // the wave's operands: A row blocks 8*wy + i; B row blocks 4*wx + j, or in SwiGLU mode gate blocks
  // 2*wx, 2*wx + 1 (j = 0, 1) and up blocks 8 + 2*wx, 8 + 2*wx + 1 (j = 2, 3).  A block of 16 rows is
  // 2 KB; lane (g, r) wants row r, chunk 4*kk + g: slot (4*kk + g) ^ (r >> 1) of that row.
  const int row_off = (r >> 3) * 1024 + (r & 7) * 128;
  int slot_off[2];
#pragma unroll
  for (int kk = 0; kk < 2; ++kk) slot_off[kk] = row_off + (((4 * kk + g) ^ (r >> 1)) * 16);
  const int a_frag = (8 * wy) * 2048, b_frag = (GLU ? 2 * wx : 4 * wx) * 2048;
  auto b_off = [&](int j) { return GLU ? ((j & 1) + 8 * (j >> 1)) * 2048 : j * 2048; };

  const int steps = gridDim.y > 1 ? ((K - k_base) < GEMM_SEG ? K - k_base : GEMM_SEG) / 64 : K / 64;
  issue_a(0);
  issue_b(0);
  if (steps > 1) issue_a(1);
  for (int step = 0; step < steps; ++step) {
    // A(step) and B(step) have landed (only A(step + 1), the wave's last four loads, may still be in
    // flight), for every wave; and every wave is done with the slots of the step before, which the
    // next loads overwrite
    if (step + 1 < steps) __builtin_amdgcn_s_waitcnt(BIG_WAIT_BUT_4);
    else __builtin_amdgcn_s_waitcnt(BIG_WAIT_ALL);
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    if (step + 1 < steps) issue_b(step + 1);
    if (step + 2 < steps) issue_a(step + 2);
    const unsigned char* a_slot = big_lds + ((2 * step) % BIG_SLOTS) * BIG_SLOT + a_frag;
    const unsigned char* b_slot = big_lds + ((2 * step + 1) % BIG_SLOTS) * BIG_SLOT + b_frag;
    __builtin_amdgcn_sched_barrier(0);
    // A step is 24 operand reads (per half of the step: 4 of B, 8 of A) and 64 matrix instructions,
    // written in the order they are needed and then interleaved explicitly: the reads of a pair of A
    // blocks (and, at the half's end, of the next half's B blocks) are issued while the 8 matrix
    // instructions of the pair before run, so that no matrix instruction waits for LDS.
    u32x4 fb[2][4], fa[2][2];
    auto read_b = [&](int kk) {
#pragma unroll
      for (int j = 0; j < 4; ++j) fb[kk][j] = *reinterpret_cast<const u32x4*>(b_slot + b_off(j) + slot_off[kk]);
    };
    auto read_a = [&](int kk, int pair) {
#pragma unroll
      for (int t = 0; t < 2; ++t)
        fa[pair & 1][t] = *reinterpret_cast<const u32x4*>(a_slot + (2 * pair + t) * 2048 + slot_off[kk]);
    };
    auto multiply = [&](int kk, int pair) {
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int j = 0; j < 4; ++j)
          acc[2 * pair + t][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(fa[pair & 1][t]), as_bf16x8(fb[kk][j]),
                                                                         acc[2 * pair + t][j], 0, 0, 0);
    };
    read_b(0);
    read_a(0, 0);
#pragma unroll
    for (int kk = 0; kk < 2; ++kk)
#pragma unroll
      for (int pair = 0; pair < 4; ++pair) {
        if (pair < 3) read_a(kk, pair + 1);
        else if (kk == 0) {
          read_b(1);
          read_a(1, 0);
        }
        multiply(kk, pair);
      }
    __builtin_amdgcn_sched_group_barrier(0x100, 6, 0);
#pragma unroll
    for (int kk = 0; kk < 2; ++kk) {
#pragma unroll
      for (int pair = 0; pair < 3; ++pair) {
        __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x008, 4, 0);
      }
      if (kk == 0) {
#pragma unroll
        for (int t = 0; t < 6; ++t) {
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
          __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        }
        __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);
      } else {
        __builtin_amdgcn_sched_group_barrier(0x008, 8, 0);
      }
    }
    __builtin_amdgcn_sched_barrier(0);
    asm volatile("" ::: "memory");
  }
  if constexpr (EPI == EPI_QKV_ROPE) {
    // What the rows of the tile need from memory is fetched once for the workgroup, into the ring (free now), not
    // by every lane for each of its rows: position and page of each of the 256 rows (a thread a row), then the
    // rows' cosines and sines (16-byte loads; a row of 32 + 32 floats, 36 apart against bank conflicts).
    constexpr int CS = 36;
    __builtin_amdgcn_s_waitcnt(BIG_WAIT_ALL);
    __syncthreads();                                                // every wave is done with the ring
    int* pos_lds = reinterpret_cast<int*>(big_lds);                 // [256]
    int* page_lds = pos_lds + BIG_BM;                               // [256]
    float* cos_lds = reinterpret_cast<float*>(page_lds + BIG_BM);   // [256][CS]
    float* sin_lds = cos_lds + BIG_BM * CS;                         // [256][CS]
    const int first_head = n0 >> 6;
    const bool any_cache = first_head + 4 > rp.heads;               // some of the tile's four heads are k or v heads
    const bool any_rotary = first_head < rp.heads + rp.kv_heads;
    if (threadIdx.x < BIG_BM) {
      const int m = m0 + (int)threadIdx.x;
      const int mm = m < M ? m : M - 1;
      const int pos = rp.positions[mm];
      int page = 0;
      if (any_cache) page = rp.block_table[(size_t)rp.row_seq[mm] * rp.table_stride + ((pos > 0 ? pos : 0) >> rp.page_shift)];
      pos_lds[threadIdx.x] = m < M ? pos : -1;
      page_lds[threadIdx.x] = page;
    }
    __syncthreads();
    if (any_rotary) {
      const int row = threadIdx.x >> 1, part = threadIdx.x & 1;     // 16 cosines and 16 sines of a row a thread
      const int pos = pos_lds[row];
      const size_t at = (size_t)(pos > 0 ? pos : 0) * 32 + 16 * part;
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        *reinterpret_cast<f32x4*>(cos_lds + row * CS + 16 * part + 4 * t) = *reinterpret_cast<const f32x4*>(rp.cos_table + at + 4 * t);
        *reinterpret_cast<f32x4*>(sin_lds + row * CS + 16 * part + 4 * t) = *reinterpret_cast<const f32x4*>(rp.sin_table + at + 4 * t);
      }
    }
    __syncthreads();
    const int head = first_head + wx;
    if (head >= rp.heads + 2 * rp.kv_heads) return;
    const int q_dim = rp.heads * 64;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int lrow0 = 128 * wy + 16 * i + 4 * g;                  // the lane's four rows of the block, within the tile
      int pos4[4], page4[4];
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        pos4[q] = pos_lds[lrow0 + q];
        page4[q] = page_lds[lrow0 + q];
      }
      if (head < rp.heads + rp.kv_heads) {
        if (head >= rp.heads && !rp.write_cache) continue;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int pos = pos4[q];
          if (pos < 0) continue;
          const int m = m0 + lrow0 + q;
          bf16_t* dst = head < rp.heads
                            ? (bf16_t*)out + (size_t)m * q_dim + (size_t)head * 64
                            : rp.k_cache + (((size_t)page4[q] * rp.kv_heads + (head - rp.heads)) * rp.page_size + (pos & (rp.page_size - 1))) * 64;
#pragma unroll
          for (int j = 0; j < 2; ++j) {
            const int d = 16 * j + r;
            const float c = cos_lds[(lrow0 + q) * CS + d], sn = sin_lds[(lrow0 + q) * CS + d];
            const float x1 = acc[i][j][q], x2 = acc[i][j + 2][q];
            dst[d] = f32_to_bf16(x1 * c - x2 * sn);
            dst[d + 32] = f32_to_bf16(x2 * c + x1 * sn);
          }
        }
      } else if (rp.write_cache) {
        // values lie transposed in their page ([d][slot]).  The lane's four rows are most often four consecutive
        // slots of one page starting at a multiple of four: then all four are stored at once.
        bool quad = pos4[0] >= 0 && (pos4[0] & 3) == 0;
#pragma unroll
        for (int t = 1; t < 4; ++t) quad = quad && pos4[t] == pos4[0] + t && page4[t] == page4[0];
        const int vh = head - rp.heads - rp.kv_heads;
        if (quad) {
          bf16_t* dst = rp.v_cache + ((size_t)page4[0] * rp.kv_heads + vh) * 64 * rp.page_size + (pos4[0] & (rp.page_size - 1));
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const u32x2 four = {pack_bf16x2(acc[i][j][0], acc[i][j][1]), pack_bf16x2(acc[i][j][2], acc[i][j][3])};
            *reinterpret_cast<u32x2*>(dst + (size_t)(16 * j + r) * rp.page_size) = four;
          }
        } else {
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            if (pos4[q] < 0) continue;
            bf16_t* dst = rp.v_cache + ((size_t)page4[q] * rp.kv_heads + vh) * 64 * rp.page_size + (pos4[q] & (rp.page_size - 1));
#pragma unroll
            for (int j = 0; j < 4; ++j) dst[(size_t)(16 * j + r) * rp.page_size] = f32_to_bf16(acc[i][j][q]);
          }
        }
      }
    }
  } else {
    if constexpr (GLU) {
      // Whole rows of the tile leave as 16-byte stores: the waves put their outputs into the ring (free now) as the tile
      // lies in memory, [256 rows][128 columns] with 16 bytes between rows, and the threads then store a row's 256 bytes
      // sixteen lanes wide.  (Two bytes a lane straight from the accumulators were 64 stores a wave, each of them four
      // pieces of 32 bytes.)  Outputs that are not 16-byte aligned take the element-wise way below.
      constexpr int TROW = 128 * 2 + 16;
      const bool wide = (reinterpret_cast<uintptr_t>(out) & 15) == 0 && (ldo & 7) == 0 && (N & 7) == 0;
      if (wide) {
        __syncthreads();                                              // every wave is done with the ring
#pragma unroll
        for (int i = 0; i < 8; ++i)
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            unsigned char* row = big_lds + (128 * wy + 16 * i + 4 * g + q) * TROW + (32 * wx + r) * 2;
#pragma unroll
            for (int j = 0; j < 2; ++j)
              *reinterpret_cast<bf16_t*>(row + 32 * j) = f32_to_bf16(silu_times(acc[i][j][q], acc[i][j + 2][q]));
          }
        __syncthreads();
        const int chunk = threadIdx.x & 15, row0 = threadIdx.x >> 4;
        const int n = n0 + 8 * chunk;
#pragma unroll
        for (int pass = 0; pass < 8; ++pass) {
          const int row = row0 + 32 * pass, m = m0 + row;
          if (m < M && n < N)
            *reinterpret_cast<u32x4*>((bf16_t*)out + (size_t)m * ldo + n) = *reinterpret_cast<const u32x4*>(big_lds + row * TROW + 16 * chunk);
        }
        return;
      }
    }
    tile_epilogue<EPI, 8>(acc, out, M, N, ldo, m0 + 128 * wy, n0 + (GLU ? 32 : 64) * wx, (n0 >> 6) + wx, r, g, false, rp);
  }
}

// ------------------------------------------------------------------------------ 128 x 128 tiles through an LDS ring

// 128 x 128 outputs a workgroup (128 x 64 of SwiGLU: 64 gate and 64 up rows of W), steps of 64 along K, eight waves
// of 64 x 32 outputs each, for prompt portions whose product has too few tiles of 256 x 256 to go round.  Tiles
// travel as in the big-tile kernel (buffer loads with LDS as destination, 8 rows of 128 bytes an instruction, chunks
// permuted against bank conflicts); a stage is a step's tiles of x and W (32 KB), the ring has four, a wave issues
// four loads a stage, and "all but the last 8 have landed" is the wait for the stage at hand; one barrier a step.
// A residual add over several segments of K adds each finished segment into the output (the chain of additions
// starts at the residual, segments in order); the other epilogues join the segments' sums left to right in
// registers.  K a multiple of 64.
#define T128_STAGE (32 * 1024)
#define T128_STAGES 4

__device__ __forceinline__ void t128_issue(unsigned char* lds, __amdgpu_buffer_rsrc_t rs_a, __amdgpu_buffer_rsrc_t rs_b,
                                           const int* voff_a, const int* voff_b, int wave, int step, int steps,
                                           int k_base) {
  typedef __attribute__((address_space(3))) void* lds_ptr;
  unsigned char* dst = lds + (step % T128_STAGES) * T128_STAGE + (2 * wave) * 1024;
  const bool real = step < steps;                                     // scalar; past K: outside the descriptors
#pragma unroll
  for (int t = 0; t < 2; ++t) {
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_a, (lds_ptr)(dst + t * 1024), 16, real ? voff_a[t] : 0x7ffffff0,
                                             k_base * 2 + step * 128, 0, 0);
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_b, (lds_ptr)(dst + 16 * 1024 + t * 1024), 16, real ? voff_b[t] : 0x7ffffff0,
                                             k_base * 2 + step * 128, 0, 0);
  }
}

template <int EPI>
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(2, 2))) void gemm_bf16_tile128_kernel(
    const bf16_t* __restrict__ x, const bf16_t* __restrict__ w, void* __restrict__ out, int M, int N, int K, int ldx,
    int ldo, int m_tiles, int n_tiles, QkvRopeArgs rp, size_t seg_stride) {
  constexpr bool GLU = EPI == EPI_SWIGLU_BF16;
  constexpr bool ROPE = EPI == EPI_QKV_ROPE;           // waves of 32 x 64 outputs: a head's 64 columns in one wave
  // gridDim.y > 1: workgroup (tile, y) works on segment y of K alone and leaves its sums at out + y * seg_stride
  // elements (a residual add's segments, joined in order by add_segments_kernel afterwards)
  const int k_base = (int)blockIdx.y * GEMM_SEG;
  if (gridDim.y > 1) out = (void*)((float*)out + (size_t)blockIdx.y * seg_stride);
  constexpr int NI = ROPE ? 2 : 4, NJ = ROPE ? 4 : 2;
  constexpr int COLS = GLU ? 64 : 128;
  extern __shared__ __attribute__((aligned(16))) unsigned char t128_lds[];   // [4 stages][x 16 KB | W 16 KB]
  const int wave = wave_index(), lane = threadIdx.x & 63;
  const int r = lane & 15, g = lane >> 4;
  const int wy = ROPE ? wave >> 1 : wave >> 2, wx = ROPE ? wave & 1 : wave & 3;
  int bid = blockIdx.x;
  const int nblocks = m_tiles * n_tiles;
  if (nblocks % 8 == 0) bid = (bid % 8) * (nblocks / 8) + bid / 8;      // an n tile's workgroups share an XCD
  const int m0 = (bid % m_tiles) * 128;
  const int n0 = (bid / m_tiles) * COLS;
  // this wave's loads of a stage: rows 16*wave .. 16*wave + 15 of x's 128 and of W's 128 (SwiGLU: W rows 0-63 of
  // the tile are gate rows n0.., 64-127 the up rows N + n0..)
  const int a_rows = min(128, M - m0), b_rows = min(COLS, N - n0);
  const __amdgpu_buffer_rsrc_t rs_a = __builtin_amdgcn_make_buffer_rsrc(
      (void*)(x + (size_t)m0 * ldx), 0, (int)((((size_t)a_rows - 1) * ldx + K) * 2), 0x00020000);
  const bool up = GLU && wave >= 4;
  const __amdgpu_buffer_rsrc_t rs_b = __builtin_amdgcn_make_buffer_rsrc(
      (void*)(w + ((size_t)(up ? N : 0) + n0) * K), 0, (int)((size_t)b_rows * K * 2), 0x00020000);
  const int b_row0 = GLU ? 16 * (wave & 3) : 16 * wave;
  const int lrow = lane >> 3, lslot = lane & 7;
  int voff_a[2], voff_b[2];
#pragma unroll
  for (int t = 0; t < 2; ++t) {
    const int r16 = 8 * t + lrow;
    const int chunk = lslot ^ (r16 >> 1);
    voff_a[t] = ((16 * wave + r16) * ldx + 8 * chunk) * 2;
    voff_b[t] = ((b_row0 + r16) * K + 8 * chunk) * 2;
  }
  f32x4 acc[NI][NJ], tot[NI][NJ];
#pragma unroll
  for (int i = 0; i < NI; ++i)
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
      acc[i][j] = (f32x4){0.f, 0.f, 0.f, 0.f};
      tot[i][j] = (f32x4){0.f, 0.f, 0.f, 0.f};
    }
  // operands: x row blocks 4*wy + i; W row blocks 2*wx + j, or in SwiGLU mode gate block wx (j = 0) and up block 4 + wx
  const int row_off = (r >> 3) * 1024 + (r & 7) * 128;
  int slot_off[2];
#pragma unroll
  for (int kk = 0; kk < 2; ++kk) slot_off[kk] = row_off + (((4 * kk + g) ^ (r >> 1)) * 16);
  const int a_frag = (NI * wy) * 2048;
  const int b_frag = 16 * 1024 + (GLU ? wx : NJ * wx) * 2048;
  constexpr int b_step = GLU ? 4 * 2048 : 2048;                        // from the wave's first W block to its second
  const int steps = gridDim.y > 1 ? ((K - k_base) < GEMM_SEG ? K - k_base : GEMM_SEG) / 64 : K / 64;
#pragma unroll
  for (int st = 0; st < T128_STAGES - 1; ++st) t128_issue(t128_lds, rs_a, rs_b, voff_a, voff_b, wave, st, steps, k_base);
  for (int step = 0; step < steps; ++step) {
    __builtin_amdgcn_s_waitcnt(vmcnt_only(4 * (T128_STAGES - 2)));
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    t128_issue(t128_lds, rs_a, rs_b, voff_a, voff_b, wave, step + T128_STAGES - 1, steps, k_base);   // into the stage worked on a step ago
    const unsigned char* stage = t128_lds + (step % T128_STAGES) * T128_STAGE;
    __builtin_amdgcn_sched_barrier(0);
    // 12 operand reads and 16 matrix instructions a step, the second half's reads under the first half's products
    u32x4 fa[2][NI], fb[2][NJ];
#pragma unroll
    for (int kk = 0; kk < 2; ++kk) {
#pragma unroll
      for (int j = 0; j < NJ; ++j) fb[kk][j] = *reinterpret_cast<const u32x4*>(stage + b_frag + j * b_step + slot_off[kk]);
#pragma unroll
      for (int i = 0; i < NI; ++i) fa[kk][i] = *reinterpret_cast<const u32x4*>(stage + a_frag + i * 2048 + slot_off[kk]);
    }
#pragma unroll
    for (int kk = 0; kk < 2; ++kk)
#pragma unroll
      for (int i = 0; i < NI; ++i)
#pragma unroll
        for (int j = 0; j < NJ; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(fa[kk][i]), as_bf16x8(fb[kk][j]), acc[i][j], 0, 0, 0);
    __builtin_amdgcn_sched_group_barrier(0x100, 6, 0);
#pragma unroll
    for (int t = 0; t < 6; ++t) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
    }
    __builtin_amdgcn_sched_group_barrier(0x008, 10, 0);
    __builtin_amdgcn_sched_barrier(0);
    asm volatile("" ::: "memory");
    if constexpr (EPI == EPI_ADD_F32) {
      const int kn = (step + 1) * 64;
      if (kn % GEMM_SEG == 0 && step + 1 < steps) {    // a segment ends before the last: add it into the output now
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
          for (int j = 0; j < 2; ++j) {
#pragma unroll
            for (int q = 0; q < 4; ++q) {
              const int m = m0 + 64 * wy + 16 * i + 4 * g + q, n = n0 + 32 * wx + 16 * j + r;
              if (m < M && n < N) ((float*)out)[(size_t)m * ldo + n] += acc[i][j][q];
            }
            acc[i][j] = (f32x4){0.f, 0.f, 0.f, 0.f};
          }
      }
    } else {
      const int kn = (step + 1) * 64;
      if (kn % GEMM_SEG == 0 && step + 1 < steps) {    // a segment ends before the last: joined left to right
#pragma unroll
        for (int i = 0; i < NI; ++i)
#pragma unroll
          for (int j = 0; j < NJ; ++j) {
            tot[i][j] = kn == GEMM_SEG ? acc[i][j] : tot[i][j] + acc[i][j];
            acc[i][j] = (f32x4){0.f, 0.f, 0.f, 0.f};
          }
      }
    }
  }
  if (EPI != EPI_ADD_F32 && steps > GEMM_SEG / 64) {
#pragma unroll
    for (int i = 0; i < NI; ++i)
#pragma unroll
      for (int j = 0; j < NJ; ++j) acc[i][j] = tot[i][j] + acc[i][j];
  }
  if constexpr (ROPE) {
    tile_epilogue<EPI, NI>(acc, out, M, N, ldo, m0 + 32 * wy, n0 + 64 * wx, (n0 >> 6) + wx, r, g, false, rp);
  } else {
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int m = m0 + 64 * wy + 16 * i + 4 * g + q;
      if (m >= M) continue;
      if constexpr (GLU) {
        const int n = n0 + 16 * wx + r;
        if (n < N) epilogue_store<EPI>(out, (size_t)m * ldo + n, acc[i][0][q], acc[i][1][q]);
      } else {
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          const int n = n0 + 32 * wx + 16 * j + r;
          if (n < N) epilogue_store<EPI>(out, (size_t)m * ldo + n, acc[i][j][q], acc[i][j][q]);
        }
      }
    }
  }
}

// ------------------------------------------------------------------------------ 128 x 256 tiles through an LDS ring

// 128 rows x 256 columns a workgroup (128 of SwiGLU: 128 gate and 128 up rows of W), eight waves of 64 x 64 outputs:
// a step pulls 48 KB for twice the 128 x 128 tile's products (which pulls 32), and a wave's 64 accumulators leave room
// for the sums of the segments before, so that a K of several segments, which the 256 x 256 kernel does not take,
// runs on these where there are enough of them.  Three stages of 48 KB (x 16 KB | W 32 KB); a wave issues six loads a
// stage.  Plain, residual, SwiGLU and (one segment, heads of 64) rotary epilogues; segments joined left to right in registers (a residual add's chain
// starts at the residual, which is read when the first segment ends).  K a multiple of 64.
#define T256_STAGE (48 * 1024)
#define T256_STAGES 3

template <int EPI>
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(2, 2))) void gemm_bf16_tile256_kernel(
    const bf16_t* __restrict__ x, const bf16_t* __restrict__ w, void* __restrict__ out, int M, int N, int K, int ldx,
    int ldo, int m_tiles, int n_tiles, QkvRopeArgs rp, size_t seg_stride) {
  constexpr bool GLU = EPI == EPI_SWIGLU_BF16;
  constexpr int COLS = GLU ? 128 : 256;
  extern __shared__ __attribute__((aligned(16))) unsigned char t256_lds[];   // [3 stages][x 16 KB | W 32 KB]
  // gridDim.y > 1: workgroup (tile, y) works on segment y of K alone and leaves its sums at out + y * seg_stride
  // elements (a residual add's segments, joined in order by add_segments_kernel afterwards)
  const int k_base = (int)blockIdx.y * GEMM_SEG, k_all = K;
  if (gridDim.y > 1) {
    out = (void*)((float*)out + (size_t)blockIdx.y * seg_stride);
    K = min(GEMM_SEG, K - k_base);
  }
  const int wave = wave_index(), lane = threadIdx.x & 63;
  const int r = lane & 15, g = lane >> 4;
  const int wy = wave >> 2, wx = wave & 3;
  int bid = blockIdx.x;
  const int nblocks = m_tiles * n_tiles;
  if (nblocks % 8 == 0) bid = (bid % 8) * (nblocks / 8) + bid / 8;      // an n tile's workgroups share an XCD
  const int m0 = (bid % m_tiles) * 128;
  const int n0 = (bid / m_tiles) * COLS;
  // this wave's loads of a stage: rows 16*wave .. 16*wave + 15 of x's 128 and rows 32*wave .. 32*wave + 31 of W's 256
  // (SwiGLU: W rows 0-127 of the tile are gate rows n0.., 128-255 the up rows N + n0..)
  const int a_rows = min(128, M - m0), b_rows = min(COLS, N - n0);
  const __amdgpu_buffer_rsrc_t rs_a = __builtin_amdgcn_make_buffer_rsrc(
      (void*)(x + (size_t)m0 * ldx), 0, (int)((((size_t)a_rows - 1) * ldx + k_all) * 2), 0x00020000);
  const bool up = GLU && wave >= 4;
  const __amdgpu_buffer_rsrc_t rs_b = __builtin_amdgcn_make_buffer_rsrc(
      (void*)(w + ((size_t)(up ? N : 0) + n0) * k_all), 0, (int)((size_t)b_rows * k_all * 2), 0x00020000);
  const int b_row0 = GLU ? 32 * (wave & 3) : 32 * wave;
  const int lrow = lane >> 3, lslot = lane & 7;
  int voff_a[2], voff_b[4];
#pragma unroll
  for (int t = 0; t < 4; ++t) {
    const int r16 = (8 * t + lrow) & 15;                    // the row within its block of 16
    const int chunk = lslot ^ (r16 >> 1);
    if (t < 2) voff_a[t] = ((16 * wave + 8 * t + lrow) * ldx + 8 * chunk) * 2;
    voff_b[t] = ((b_row0 + 8 * t + lrow) * k_all + 8 * chunk) * 2;
  }
  typedef __attribute__((address_space(3))) void* lds_ptr;
  const int steps = K / 64;
  auto issue = [&](int step) {
    unsigned char* dst = t256_lds + (step % T256_STAGES) * T256_STAGE;
    const bool real = step < steps;                                     // scalar; past K: outside the descriptors
#pragma unroll
    for (int t = 0; t < 2; ++t)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_a, (lds_ptr)(dst + (2 * wave + t) * 1024), 16, real ? voff_a[t] : 0x7ffffff0,
                                               k_base * 2 + step * 128, 0, 0);
#pragma unroll
    for (int t = 0; t < 4; ++t)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_b, (lds_ptr)(dst + 16 * 1024 + (4 * wave + t) * 1024), 16,
                                               real ? voff_b[t] : 0x7ffffff0, k_base * 2 + step * 128, 0, 0);
  };
  f32x4 acc[4][4], tot[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      acc[i][j] = (f32x4){0.f, 0.f, 0.f, 0.f};
      tot[i][j] = (f32x4){0.f, 0.f, 0.f, 0.f};
    }
  // operands: x row blocks 4*wy + i; W row blocks 4*wx + j, or in SwiGLU mode gate blocks 2*wx, 2*wx + 1 (j = 0, 1)
  // and up blocks 8 + 2*wx, 8 + 2*wx + 1 (j = 2, 3)
  const int row_off = (r >> 3) * 1024 + (r & 7) * 128;
  int slot_off[2];
#pragma unroll
  for (int kk = 0; kk < 2; ++kk) slot_off[kk] = row_off + (((4 * kk + g) ^ (r >> 1)) * 16);
  const int a_frag = (4 * wy) * 2048;
  const int b_frag = 16 * 1024 + (GLU ? 2 * wx : 4 * wx) * 2048;
  auto b_off = [&](int j) { return GLU ? ((j & 1) + 8 * (j >> 1)) * 2048 : j * 2048; };
#pragma unroll
  for (int st = 0; st < T256_STAGES - 1; ++st) issue(st);
  for (int step = 0; step < steps; ++step) {
    __builtin_amdgcn_s_waitcnt(vmcnt_only(6 * (T256_STAGES - 2)));
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    issue(step + T256_STAGES - 1);                                      // into the stage worked on a step ago
    const unsigned char* stage = t256_lds + (step % T256_STAGES) * T256_STAGE;
    __builtin_amdgcn_sched_barrier(0);
    // 16 operand reads and 32 matrix instructions a step, the second half's reads under the first half's products
    u32x4 fa[2][4], fb[2][4];
#pragma unroll
    for (int kk = 0; kk < 2; ++kk) {
#pragma unroll
      for (int j = 0; j < 4; ++j) fb[kk][j] = *reinterpret_cast<const u32x4*>(stage + b_frag + b_off(j) + slot_off[kk]);
#pragma unroll
      for (int i = 0; i < 4; ++i) fa[kk][i] = *reinterpret_cast<const u32x4*>(stage + a_frag + i * 2048 + slot_off[kk]);
    }
#pragma unroll
    for (int kk = 0; kk < 2; ++kk)
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(fa[kk][i]), as_bf16x8(fb[kk][j]), acc[i][j], 0, 0, 0);
    __builtin_amdgcn_sched_group_barrier(0x100, 8, 0);
#pragma unroll
    for (int t = 0; t < 8; ++t) {
      __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
    }
    __builtin_amdgcn_sched_group_barrier(0x008, 16, 0);
    __builtin_amdgcn_sched_barrier(0);
    asm volatile("" ::: "memory");
    const int kn = (step + 1) * 64;
    if (kn % GEMM_SEG == 0 && kn < K) {                // a segment ends before the last: joined left to right
      if (EPI == EPI_ADD_F32 && kn == GEMM_SEG) {      // the chain of a residual add starts at the residual
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
          for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int q = 0; q < 4; ++q) {
              const int m = m0 + 64 * wy + 16 * i + 4 * g + q, n = n0 + 64 * wx + 16 * j + r;
              tot[i][j][q] = (m < M && n < N) ? ((const float*)out)[(size_t)m * ldo + n] : 0.0f;
            }
      }
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          tot[i][j] = (EPI != EPI_ADD_F32 && kn == GEMM_SEG) ? acc[i][j] : tot[i][j] + acc[i][j];
          acc[i][j] = (f32x4){0.f, 0.f, 0.f, 0.f};
        }
    }
  }
  if (K > GEMM_SEG) {
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) acc[i][j] = tot[i][j] + acc[i][j];
  }
  // (a residual add of several segments has the residual in its sums; of one segment the epilogue adds it)
  tile_epilogue<EPI, 4>(acc, out, M, N, ldo, m0 + 64 * wy, n0 + (GLU ? 32 : 64) * wx, (n0 >> 6) + wx, r, g,
                        EPI == EPI_ADD_F32 && K > GEMM_SEG, rp);
}

template <int EPI>
static int launch_tile256(const bf16_t* x, const bf16_t* w, void* out, int M, int N, int K, int ldx, int ldo, hipStream_t s,
                          const QkvRopeArgs& rp = QkvRopeArgs{}, int segments = 1, size_t seg_stride = 0) {
  constexpr int COLS256 = (EPI == EPI_SWIGLU_BF16) ? 128 : 256;
  const int mt = (M + 127) / 128, nt = (N + COLS256 - 1) / COLS256;
  static bool allowed = false;                   // more than 64 KB of dynamic LDS has to be asked for once
  if (!allowed) {
    (void)hipFuncSetAttribute((const void*)gemm_bf16_tile256_kernel<EPI>, hipFuncAttributeMaxDynamicSharedMemorySize,
                              T256_STAGES * T256_STAGE);
    allowed = true;
  }
  BW_LAUNCH((gemm_bf16_tile256_kernel<EPI>), dim3(mt * nt, segments), dim3(512), T256_STAGES * T256_STAGE, s, x, w, out, M, N, K, ldx,
                     ldo, mt, nt, rp, seg_stride);
  return BW_LAUNCH_CHECK();
}
