// Part of gemm_bf16.hip (included there, after its epilogues and launch macro; not a unit of its own):
// the kernels of decode steps and short portions: up to 64 rows through LDS (with RMSNorm, SwiGLU, rotation and cache write), and the residual adds of up to 16 rows.
#pragma once

// ------------------------------------------------------------------------------ up to 64 rows, through LDS

// All rows (NRB blocks of 16: up to 16, 32 or 64 rows) x 64 columns a workgroup (32 of SwiGLU: 32 gate
// and 32 up rows of W), steps of 64 along K.  The rows of x come into LDS once per workgroup and serve
// all its strips; weights and x travel as in the big-tile kernel (buffer loads with LDS as destination,
// 8 rows of 128 bytes an instruction, whole cache lines; chunks permuted against bank conflicts), and
// since no registers hold them the ring can be deep: eight stages, so up to seven steps of weights are
// in flight while one is worked on.  Every wave issues the same number of loads a stage (LPW: its share
// of the weights and of x, padded with loads from outside the descriptors, which cost no memory
// traffic), in order, so "all but the last (stages - 2) * LPW have landed" is the wait for the stage at hand;
// stages past K are asked for outside the descriptors too, to keep that count fixed.  One barrier a
// step: behind it every wave has the stage at hand and is done with the one before.
// Plain epilogues: four waves, wave w owns strip w and all blocks of rows.  SwiGLU: wave (s, h) owns
// gate and up strip s for half h of the row blocks (with one block of rows the waves of the second
// half only load and normalise: their products are of rows that do not exist and go nowhere).
// K a multiple of 64, one segment.

// NORM: the rows arrive as the 32-bit residual stream and are normalised (RMSNorm, the statements of
// rmsnorm_bf16_kernel) into LDS by the workgroup itself, all of K at once (up to 16 rows, K one segment);
// the ring then holds weights only, and its first stages are in flight while the rows are normalised.
// NARROW (plain epilogues, at least two blocks of rows): 32 columns a workgroup, the waves arranged as for SwiGLU
// (strip s, half h of the row blocks), for products with so few columns that 64 a workgroup would leave most
// compute units idle.
// EIGHT (17 rows or more): eight waves, wave (s, b) owns strip s for one block of the rows (narrow and SwiGLU tiles;
// with two blocks of rows half the waves only load) or for half of them (64 columns), and a stage is four steps of 64
// along K (two where a step has 64 rows of W): what a compute unit pulls grows with its waves and with the bytes
// between two barriers (64 rows of the output projection: 29 KB a microsecond with four waves and a stage a step,
// 55 with eight and four steps).  K in whole stages.
// (MidShape, the numbers that follow from these choices, is in layout.h)

// Residual add over several segments of K, a workgroup per tile and segment (gridDim.y segments): where the
// segments' sums meet (device scratch, [tile][segment][wave][block of rows][lane] x 16 bytes) and the tiles'
// counters (zero before and after every launch).
struct MidSplitArgs {
  float* scratch;
  int* counters;
};

// What the NORM variant needs beside the product's operands.
struct MidNormArgs {
  const float* x32;      // [M, ldx32] rows of the residual stream
  const void* norm_w;    // [K]
  int ldx32, norm_w_is_bf16;
  float eps;
  int row_step;          // bytes of LDS a step of 64 along K of the normalised rows takes: 2048 (16 rows), or 1024
                         // (8 rows: rows of up to two segments of K, which are normalised a wave a row)
};

// What a phase of a chain is asked with: the operands of bw_norm_gemm_mid / bw_norm_qkv_rope_mid, or of the kernels for
// up to 16 rows and few columns.
struct MidCall {
  const bf16_t* w;
  void* out;
  int M, N, K, ldo;
  MidNormArgs na;
  QkvRopeArgs rp;
};
struct RowsCall {
  const bf16_t* x;
  const bf16_t* w;
  void* out;
  int M, N, K, ldx, ldo, S;
};
enum ChainKind {
  CK_QKV_NARROW, CK_QKV_WIDE, CK_GLU, CK_F32, CK_BURST_ADD, CK_STREAM_ADD_8_8, CK_STREAM_ADD_8_16, CK_STREAM_ADD_16_8,
  CK_STREAM_ADD_16_16
};
// Which phase a variant of the kernel for up to 64 rows is; -1: it does not run as a phase.
template <int EPI, int NRB, bool NORM, bool NARROW, bool EIGHT>
constexpr int mid_chain_kind() {
  if (!NORM || !EIGHT || NRB != 1) return -1;
  if (EPI == EPI_QKV_ROPE) return NARROW ? CK_QKV_NARROW : CK_QKV_WIDE;
  if (NARROW) return -1;
  if (EPI == EPI_SWIGLU_BF16) return CK_GLU;
  if (EPI == EPI_F32) return CK_F32;
  return -1;
}
template <int EPI, int CW, int XR>
constexpr int stream_chain_kind() {
  if (EPI != EPI_ADD_F32) return -1;
  if (CW == 8) return XR == 8 ? CK_STREAM_ADD_8_8 : CK_STREAM_ADD_8_16;
  return XR == 8 ? CK_STREAM_ADD_16_8 : CK_STREAM_ADD_16_16;
}

// Where a wave's loads of a stage go and come from.  A load is 8 rows of one step of 64 along K (1 KB): of x, block
// ``id % (2 NRB)`` of step ``id / (2 NRB)`` of the stage for the wave's id-th load; of W likewise (SwiGLU with eight
// waves: the first four waves take the gate rows, the others the up rows, so that a wave's loads share a descriptor).
template <int EPI, int NRB, bool NORM, bool NARROW, bool EIGHT>
struct MidLoads {
  using S = MidShape<EPI, NRB, NORM, NARROW, EIGHT>;
  int voff_a[S::A_LOADS > 0 ? S::A_LOADS : 1], voff_b[S::B_LOADS];   // byte offsets in x (0x7ffffff0: a padding load) and in the tile's rows of W
  int dst_a[S::A_LOADS > 0 ? S::A_LOADS : 1], dst_b[S::B_LOADS];     // byte offsets in the stage
};

// A wave's loads of one stage of the ring: its share of the rows of x and of W, LPW instructions.
template <int EPI, int NRB, bool NORM, bool NARROW, bool EIGHT>
__device__ __forceinline__ void mid_issue(unsigned char* lds, __amdgpu_buffer_rsrc_t rs_a, __amdgpu_buffer_rsrc_t rs_b,
                                          const MidLoads<EPI, NRB, NORM, NARROW, EIGHT>& ld, int step, int steps, int k_base) {
  using S = MidShape<EPI, NRB, NORM, NARROW, EIGHT>;
  typedef __attribute__((address_space(3))) void* lds_ptr;
  unsigned char* dst = lds + mid_stage_offset<S>(step);
  const bool real = step < steps;                                     // scalar
  const int k_off = (k_base + step * S::SUB * 64) * 2;
#pragma unroll
  for (int t = 0; t < S::A_LOADS; ++t)                                // (a padding load's zeros go behind the ring)
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_a, (lds_ptr)(ld.dst_a[t] >= 0 ? dst + ld.dst_a[t] : lds + mid_padding_offset<S>()), 16,
                                             real ? ld.voff_a[t] : 0x7ffffff0, k_off, 0, 0);
#pragma unroll
  for (int t = 0; t < S::B_LOADS; ++t)
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_b, (lds_ptr)(dst + ld.dst_b[t]), 16, real ? ld.voff_b[t] : 0x7ffffff0, k_off, 0, 0);
}

// The NORM variant's rows: wave ``wave`` normalises rows wave, wave + 4, ... (RB of them at most) into LDS, the
// ring's first stages asked for between the rows' loads and the arithmetic.
template <int RB, int NV, int EPI, int NRB, bool NARROW, bool EIGHT>
__device__ __forceinline__ void mid_norm_rows(const MidNormArgs& na, int M, int K, int wave, int lane, unsigned char* rows_lds,
                                              unsigned char* mid_lds, __amdgpu_buffer_rsrc_t rs_a, __amdgpu_buffer_rsrc_t rs_b,
                                              const MidLoads<EPI, NRB, true, NARROW, EIGHT>& ld, int steps, int k_base) {
  using S = MidShape<EPI, NRB, true, NARROW, EIGHT>;
  const int nvec = K >> 2;
  NormRows<RB, NV> nr;
  const f32x4* nrows[RB];
#pragma unroll
  for (int i = 0; i < RB; ++i) {
    const int m = mid_norm_row_of(wave, i, S::NW);
    nrows[i] = m < M ? reinterpret_cast<const f32x4*>(na.x32 + (size_t)m * na.ldx32) : nullptr;
  }
  norm_rows_load<RB>(nr, nrows, na.norm_w, na.norm_w_is_bf16, nvec, lane);
  __builtin_amdgcn_sched_barrier(0);
#pragma unroll
  for (int st = 0; st < S::STAGES - 1; ++st) mid_issue<EPI, NRB, true, NARROW, EIGHT>(mid_lds, rs_a, rs_b, ld, st, steps, k_base);
  __builtin_amdgcn_sched_barrier(0);
  unsigned char* rl = rows_lds;
  const int nw = S::NW, row_step = na.row_step;
  norm_rows_finish<RB>(nr, nrows, na.norm_w_is_bf16, nvec, K, na.eps, lane, [=](int i, int c, u32x2 pk) {
    // vector c = elements 4c..4c+3 of row m: step c / 16, 16-byte chunk (c % 16) / 2 of the step, its half c % 2
    const int m = mid_norm_row_of(wave, i, nw);
    *reinterpret_cast<u32x2*>(rl + mid_norm_store_offset(c, m, row_step)) = pk;
  });
}

// The same for a workgroup that is a phase of a launch of several: the rows were written earlier in this launch,
// maybe on another die, so they are loaded at device scope (through a descriptor over all rows), after the ring's
// first stages and after the wait for the phase that wrote them.  The statements that follow the loads are the same.
template <int RB, int NV, int NW>
__device__ __forceinline__ void mid_norm_rows_dev(const MidNormArgs& na, int M, int K, int wave, int lane, unsigned char* rows_lds) {
  const int nvec = K >> 2;
  NormRows<RB, NV> nr;
  const f32x4* nrows[RB];
  int row_off[RB];
#pragma unroll
  for (int i = 0; i < RB; ++i) {
    const int m = mid_norm_row_of(wave, i, NW);
    nrows[i] = m < M ? reinterpret_cast<const f32x4*>(na.x32 + (size_t)m * na.ldx32) : nullptr;
    row_off[i] = (m < M ? m : mid_norm_row_of(wave, 0, NW)) * na.ldx32 * 4;
  }
  const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc((void*)na.x32, 0, (int)((((size_t)M - 1) * na.ldx32 + K) * 4), 0x00020000);
#pragma unroll
  for (int j = 0; j < NV; ++j) {
    const int c = norm_vec_index(j, lane, nvec);
    nr.w[j] = load_norm_w_raw(na.norm_w, na.norm_w_is_bf16, c);
#pragma unroll
    for (int i = 0; i < RB; ++i)
      nr.v[i][j] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(rs, row_off[i] + 16 * c, 0, 16));
  }
  unsigned char* rl = rows_lds;
  const int row_step = na.row_step;
  norm_rows_finish<RB>(nr, nrows, na.norm_w_is_bf16, nvec, K, na.eps, lane, [=](int i, int c, u32x2 pk) {
    const int m = mid_norm_row_of(wave, i, NW);
    *reinterpret_cast<u32x2*>(rl + mid_norm_store_offset(c, m, row_step)) = pk;
  });
}

// CH: the workgroup is one of a phase of a launch of several (ChainCtx): the ring's first stages are asked for before
// the wait for the phase before, the rows to normalise after it, and rows and outputs travel at device scope.
template <int EPI, int NRB, bool NORM, bool NARROW, bool EIGHT, bool CH>
__device__ __forceinline__ void mid_body(const bf16_t* __restrict__ x, const bf16_t* __restrict__ w, void* __restrict__ out, int M, int N,
                                         int K, int ldx, int ldo, MidNormArgs na, QkvRopeArgs rp, MidSplitArgs sp, const ChainCtx& cc) {
  static_assert(!CH || NORM, "as a phase: the variants that normalise their rows");
  using S = MidShape<EPI, NRB, NORM, NARROW, EIGHT>;
  constexpr bool GLU = S::GLU;
  constexpr int COLS = S::COLS, NI = S::NI, NJ = S::NJ, THREADS = 64 * S::NW;
  if constexpr (!NORM) {
    // cc.gz > 1: a prompt portion of a few blocks of 16 * NRB rows in one launch, workgroup (tile, segment, z) the
    // rows of block z (a residual add's segments meet in scratch cells of their own for every block and tile)
    if (cc.gz > 1) {
      const int first = cc.bz * 16 * NRB;
      x += (size_t)first * ldx;
      if constexpr (EPI == EPI_QKV_ROPE) {
        rp.positions += first;
        rp.row_seq += first;
        out = (void*)((bf16_t*)out + (size_t)first * rp.heads * rp.head_dim);
      } else if constexpr (EPI == EPI_BF16 || EPI == EPI_SWIGLU_BF16) {
        out = (void*)((bf16_t*)out + (size_t)first * ldo);
      } else {
        out = (void*)((float*)out + (size_t)first * ldo);
      }
      M = min(16 * NRB, M - first);
    }
  }
  extern __shared__ __attribute__((aligned(16))) unsigned char mid_lds[];   // [8 stages][x: NRB * 2 KB | W: 8 KB], 1 KB for padding loads; NORM: then the rows, 2 KB a step
  const int wave = wave_index(), lane = threadIdx.x & 63;
  const int r = lane & 15, g = lane >> 4;
  // rotary epilogue: a workgroup has PAIRS whole rotary pairs (i, i + head size / 2) of one head, 32 or (narrow
  // tiles) 16: the pairs' first columns as the first half of its tile's rows of W, their second columns as the second
  constexpr bool ROPE = EPI == EPI_QKV_ROPE;
  constexpr bool RN = S::ROPE_NARROW;
  constexpr int PAIRS = RN ? 16 : 32, PSH = RN ? 4 : 5;              // rotary pairs of a row in this tile
  const int hd = ROPE ? rp.head_dim : 64, half = hd >> 1;
  const int tiles_per_head = half / PAIRS;
  const int head = ROPE ? cc.bx / tiles_per_head : 0;
  const int pair0 = ROPE ? PAIRS * (cc.bx % tiles_per_head) : 0;   // the tile's first pair within the head
  const int n0 = ROPE ? head * hd : cc.bx * COLS;
  const int b_rows = ROPE ? hd : min(COLS, N - n0);
  const __amdgpu_buffer_rsrc_t rs_a = __builtin_amdgcn_make_buffer_rsrc(
      (void*)x, 0, NORM ? 0 : (int)((((size_t)M - 1) * ldx + K) * 2), 0x00020000);
  // SwiGLU: W rows 0-31 of the tile are gate rows n0.., 32-63 the up rows N + n0..; a wave's loads are all of one kind
  const int lrow = lane >> 3, lslot = lane & 7;
  // which 1 KB of a stage this wave's t-th load of W is: block ``blk`` (8 rows) of step ``sub`` of the stage
  auto b_load = [&](int t, int& sub, int& blk) { mid_b_load<S>(wave, t, sub, blk); };
  int sub0, blk0;
  b_load(0, sub0, blk0);
  const bool up = GLU && blk0 >= 4;                                  // (all of a wave's loads are of one kind)
  const __amdgpu_buffer_rsrc_t rs_b = __builtin_amdgcn_make_buffer_rsrc(
      (void*)(w + ((size_t)(up ? N : 0) + n0) * K), 0, (int)((size_t)b_rows * K * 2), 0x00020000);
  MidLoads<EPI, NRB, NORM, NARROW, EIGHT> ld;
#pragma unroll
  for (int t = 0; t < S::A_LOADS; ++t) {
    int sub, block;
    const bool is_load = mid_a_load<S, NRB>(wave, t, sub, block);    // past the stage's blocks: a padding load
    const int row = block * 8 + lrow;                                // of the NRB * 16 rows of x
    const int chunk = lslot ^ ((row & 15) >> 1);
    ld.voff_a[t] = is_load ? (row * ldx + 8 * chunk + 64 * sub) * 2 : 0x7ffffff0;
    ld.dst_a[t] = is_load ? mid_a_dst<S>(sub, block) : -1;
  }
  if constexpr (S::A_LOADS == 0) {
    ld.voff_a[0] = 0;
    ld.dst_a[0] = -1;
  }
#pragma unroll
  for (int t = 0; t < S::B_LOADS; ++t) {
    int sub, blk;
    b_load(t, sub, blk);
    const int row = blk * 8 + lrow;                                  // of the tile's rows of W
    const int chunk = lslot ^ ((row & 15) >> 1);
    const int w_row = ROPE ? (row < PAIRS ? pair0 + row : half + pair0 + row - PAIRS) : (GLU ? row & 31 : row);
    ld.voff_b[t] = (w_row * K + 8 * chunk + 64 * sub) * 2;
    ld.dst_b[t] = mid_b_dst<S>(sub, blk);
  }
  // cc.gy > 1: this workgroup works on one segment of K (the residual add's split, below); else on all of K,
  // segment after segment, each segment's sums joined to those before it when it ends
  const int k_base = cc.by * GEMM_SEG;
  const int steps = (cc.gy > 1 ? ((K - k_base) < GEMM_SEG ? K - k_base : GEMM_SEG) / 64 : K / 64) / S::SUB;   // stages
  f32x4 acc[NI][NJ], tot[NI][NJ];
#pragma unroll
  for (int i = 0; i < NI; ++i)
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
      acc[i][j] = (f32x4){0.f, 0.f, 0.f, 0.f};
      tot[i][j] = (f32x4){0.f, 0.f, 0.f, 0.f};
    }
  // lane (g, r) wants row r of a block of 16 rows (2 KB), chunk 4*kk + g: slot (4*kk + g) ^ (r >> 1) of that row
  int slot_off[2];
#pragma unroll
  for (int kk = 0; kk < 2; ++kk) slot_off[kk] = mid_operand_offset(r, g, kk);
  const int strip = wave % S::STRIPS;                                 // of the tile's output columns
  const int a_block0 = mid_first_block<S>(wave);                      // first block of 16 rows this wave works on
  const bool computing = a_block0 < NRB;                              // (more groups of waves than blocks of rows: the others only load)

  // Rotary epilogue (the stacked q|k|v product, heads of 64: the workgroup's columns are a head, or 16 pairs of
  // one): what this thread's (row, pair) items need, cosine, sine and page, hangs on the row's position.
  constexpr int ITEMS = EPI == EPI_QKV_ROPE ? (16 * NRB * PAIRS + THREADS - 1) / THREADS : 1;   // (row, pair) items a thread: 16 * NRB rows x PAIRS
  int r_pos[ITEMS], r_page[ITEMS];
  float r_cos[ITEMS], r_sin[ITEMS];
  if constexpr (EPI == EPI_QKV_ROPE) {
    // the positions are asked for first of all; what depends on them (two loads in a row cost two trips to memory)
    // is asked for once the ring is under way
#pragma unroll
    for (int j = 0; j < ITEMS; ++j) {
      const int e = threadIdx.x + j * THREADS;
      r_pos[j] = e < M * PAIRS ? rp.positions[e >> PSH] : -1;
    }
    asm volatile("" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);
  }
  // A residual add without a meeting of segments: the outputs' old values are asked for before the ring (older than its
  // loads, so the loop's waits cover them); asked for at the end they were one more trip to memory.
  constexpr bool OLD_FIRST = EPI == EPI_ADD_F32 && !NORM;
  float old_out[OLD_FIRST ? NI : 1][4];
  if constexpr (OLD_FIRST) {
    const int n = n0 + 16 * strip + r;
#pragma unroll
    for (int i = 0; i < NI; ++i)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int m = 16 * (a_block0 + i) + 4 * g + q;
        old_out[i][q] = (cc.gy == 1 && computing && m < M && n < N) ? ((const float*)out)[(size_t)m * ldo + n] : 0.0f;
      }
    asm volatile("" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);
  }
  unsigned char* rows_lds = mid_lds + S::RING;
  if constexpr (NORM && CH) {
    // as a phase: the weights depend on nothing, the rows on the phase before
#pragma unroll
    for (int st = 0; st < S::STAGES - 1; ++st) mid_issue<EPI, NRB, NORM, NARROW, EIGHT>(mid_lds, rs_a, rs_b, ld, st, steps, k_base);
    asm volatile("" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);
    chain_wait<CH>(cc);
    if (wave < M) {
      const int rows_a_wave = mid_norm_rows_a_wave(M, S::NW);
      if (mid_norm_vectors_a_lane(K) == 16) mid_norm_rows_dev<1, 16, S::NW>(na, M, K, wave, lane, rows_lds);
      else if (rows_a_wave == 1) mid_norm_rows_dev<1, 8, S::NW>(na, M, K, wave, lane, rows_lds);
      else mid_norm_rows_dev<2, 8, S::NW>(na, M, K, wave, lane, rows_lds);
    }
  } else if constexpr (NORM) {
    // the rows to normalise are asked for before the ring (loads complete in the order they are issued: the
    // wait for the rows must not be a wait for weights); wave w takes rows w, w + 4, ...: as many at a time as
    // there are (a slot without a row would fetch a row for nothing)
    if (wave < M) {
      const int rows_a_wave = mid_norm_rows_a_wave(M, S::NW);         // EIGHT: at most 2 (rows w and w + 8), else at most 4
      if (mid_norm_vectors_a_lane(K) == 16)                           // (rows of two segments: by the launch no more than a row a wave)
        mid_norm_rows<1, 16, EPI, NRB, NARROW, EIGHT>(na, M, K, wave, lane, rows_lds, mid_lds, rs_a, rs_b, ld, steps, k_base);
      else if (rows_a_wave == 1) mid_norm_rows<1, 8, EPI, NRB, NARROW, EIGHT>(na, M, K, wave, lane, rows_lds, mid_lds, rs_a, rs_b, ld, steps, k_base);
      else if (rows_a_wave == 2) mid_norm_rows<2, 8, EPI, NRB, NARROW, EIGHT>(na, M, K, wave, lane, rows_lds, mid_lds, rs_a, rs_b, ld, steps, k_base);
      else if constexpr (!EIGHT) {
        if (rows_a_wave == 3) mid_norm_rows<3, 8, EPI, NRB, NARROW, EIGHT>(na, M, K, wave, lane, rows_lds, mid_lds, rs_a, rs_b, ld, steps, k_base);
        else mid_norm_rows<4, 8, EPI, NRB, NARROW, EIGHT>(na, M, K, wave, lane, rows_lds, mid_lds, rs_a, rs_b, ld, steps, k_base);
      }
    }
    if (wave >= M) {                                                   // a wave without rows still feeds the ring
#pragma unroll
      for (int st = 0; st < S::STAGES - 1; ++st) mid_issue<EPI, NRB, NORM, NARROW, EIGHT>(mid_lds, rs_a, rs_b, ld, st, steps, k_base);
    }
    // rows past M stay as LDS holds them: their products are never stored
  } else {
#pragma unroll
    for (int st = 0; st < S::STAGES - 1; ++st) mid_issue<EPI, NRB, NORM, NARROW, EIGHT>(mid_lds, rs_a, rs_b, ld, st, steps, k_base);
  }
  if constexpr (EPI == EPI_QKV_ROPE) {
    // These loads are younger than the ring's first stages: the loop's waits ("all but the last PENDING loads have
    // landed") ask for a little more than the stage at hand until these have landed too, never for less.
    asm volatile("" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int j = 0; j < ITEMS; ++j) {
      const int e = threadIdx.x + j * THREADS;
      const int pos = r_pos[j];
      r_page[j] = 0;
      r_cos[j] = 1.f;
      r_sin[j] = 0.f;
      if (pos >= 0) {
        r_cos[j] = rp.cos_table[(size_t)pos * half + pair0 + (e & (PAIRS - 1))];
        r_sin[j] = rp.sin_table[(size_t)pos * half + pair0 + (e & (PAIRS - 1))];
        r_page[j] = rp.block_table[(size_t)rp.row_seq[e >> PSH] * rp.table_stride + (pos >> rp.page_shift)];
      }
    }
    asm volatile("" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);
  }
  for (int step = 0; step < steps; ++step) {
    __builtin_amdgcn_s_waitcnt(vmcnt_only(S::PENDING));
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    mid_issue<EPI, NRB, NORM, NARROW, EIGHT>(mid_lds, rs_a, rs_b, ld, step + S::STAGES - 1, steps, k_base);   // into the stage worked on a step ago
    const unsigned char* stage = mid_lds + mid_stage_offset<S>(step);
    if (computing) {
#pragma unroll
      for (int sub = 0; sub < S::SUB; ++sub) {
        const unsigned char* at = stage + sub * S::STEP_BYTES;         // this step of 64 along K
#pragma unroll
        for (int kk = 0; kk < 2; ++kk) {
          u32x4 fa[NI], fb[NJ];
#pragma unroll
          for (int i = 0; i < NI; ++i)
            fa[i] = *reinterpret_cast<const u32x4*>(NORM ? rows_lds + mid_norm_read_offset(step * S::SUB + sub, a_block0 + i, na.row_step, r, g, kk)
                                                         : at + (a_block0 + i) * 2048 + slot_off[kk]);
#pragma unroll
          for (int j = 0; j < NJ; ++j) fb[j] = *reinterpret_cast<const u32x4*>(at + mid_b_read_offset<S>(strip, j, r, g, kk));
#pragma unroll
          for (int i = 0; i < NI; ++i)
#pragma unroll
            for (int j = 0; j < NJ; ++j)
              acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(fa[i]), as_bf16x8(fb[j]), acc[i][j], 0, 0, 0);
        }
        if constexpr (!NORM || EIGHT) {
          const int kn = (step * S::SUB + sub + 1) * 64;
          if (kn % GEMM_SEG == 0 && kn < K && cc.gy == 1) {          // a segment ends before the last: left to right
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
    }
    asm volatile("" ::: "memory");
  }
  if constexpr (!NORM || EIGHT) {
    if (K > GEMM_SEG && cc.gy == 1) {                               // the last segment joins the others
#pragma unroll
      for (int i = 0; i < NI; ++i)
#pragma unroll
        for (int j = 0; j < NJ; ++j) acc[i][j] = tot[i][j] + acc[i][j];
    }
  }
  if constexpr (EPI == EPI_QKV_ROPE) {
    // The rotary pairs (i, i + 32) sit in different waves: the 32-bit products meet in LDS.  Heads come in the
    // order q heads, k heads, v heads; q rotated to its buffer, k rotated and v as it is to the row's page slot.
    __builtin_amdgcn_s_waitcnt(vmcnt_only(0));                       // the padding loads have landed: LDS is free
    __syncthreads();
    float* os = reinterpret_cast<float*>(mid_lds);                    // [M][2 * PAIRS]: a row's first halves of the pairs, then the second
#pragma unroll
    for (int i = 0; i < NI; ++i)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int m = 16 * (a_block0 + i) + 4 * g + q;
        if (m < M) os[m * 2 * PAIRS + 16 * strip + r] = acc[i][0][q];
      }
    __syncthreads();
#pragma unroll
    for (int j = 0; j < ITEMS; ++j) {
      const int e = threadIdx.x + j * THREADS;
      const int pos = r_pos[j];
      if (e >= M * PAIRS || pos < 0) continue;
      const int m = e >> PSH, ip = e & (PAIRS - 1), i = pair0 + ip;
      const float x1 = os[m * 2 * PAIRS + ip], x2 = os[m * 2 * PAIRS + ip + PAIRS];
      if (head < rp.heads + rp.kv_heads) {
        const float c = r_cos[j], sn = r_sin[j];
        const float o1 = x1 * c - x2 * sn;
        const float o2 = x2 * c + x1 * sn;
        bf16_t* dst = nullptr;
        if (head < rp.heads) dst = (bf16_t*)out + (size_t)m * rp.heads * hd + (size_t)head * hd;
        else if (rp.write_cache)
          dst = rp.k_cache + (((size_t)r_page[j] * rp.kv_heads + (head - rp.heads)) * rp.page_size + (pos & (rp.page_size - 1))) * hd;
        if (dst != nullptr) {
          st_bf16<CH>(dst + i, f32_to_bf16(o1));
          st_bf16<CH>(dst + i + half, f32_to_bf16(o2));
        }
      } else if (rp.write_cache) {
        bf16_t* dst = rp.v_cache + ((size_t)r_page[j] * rp.kv_heads + (head - rp.heads - rp.kv_heads)) * hd * rp.page_size +
                      (pos & (rp.page_size - 1));
        st_bf16<CH>(dst + (size_t)i * rp.page_size, f32_to_bf16(x1));
        st_bf16<CH>(dst + (size_t)(i + half) * rp.page_size, f32_to_bf16(x2));
      }
    }
  } else {
    const int n = n0 + 16 * strip + r;
    if constexpr (EPI == EPI_ADD_F32 && !NORM) {
      const int nseg = cc.gy;
      if (nseg > 1) {
        // Every segment's workgroup leaves its sums in device scratch (stores of device scope: they write through,
        // and each wave waits below until its own are acknowledged, so they are in memory, not in this die's L2,
        // before the barrier) and counts itself in; the one that finds all others counted in adds all segments'
        // sums to the residual in segment order, every one of them read back from the scratch (its own too) with
        // device-scope loads issued after the barrier behind the count.  The counter is back at zero when the
        // kernel ends.
        const int cell = S::NW * NI * 1024;                          // bytes of a workgroup's sums: [wave][i][lane] x 16
        const int tile_id = (int)(cc.bz * cc.gx + cc.bx);   // (block of rows, tile of columns)
        const __amdgpu_buffer_rsrc_t rs_s = __builtin_amdgcn_make_buffer_rsrc(
            (void*)((unsigned char*)sp.scratch + (size_t)tile_id * nseg * cell), 0, nseg * cell, 0x00020000);
        const int mine = (wave * NI) * 1024 + lane * 16;
#pragma unroll
        for (int i = 0; i < NI; ++i)
          __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, acc[i][0]), rs_s, mine + i * 1024, cc.by * cell, 16);
        __builtin_amdgcn_s_waitcnt(vmcnt_only(0));                   // this wave's stores have been acknowledged
        __syncthreads();                                             // also: every wave is done with the ring, whose first word is the flag now
        int* is_last = reinterpret_cast<int*>(mid_lds);
        if (threadIdx.x == 0) *is_last = atomicAdd(&sp.counters[tile_id], 1) == nseg - 1;
        __syncthreads();
        if (!*is_last) return;
        if (threadIdx.x == 0) sp.counters[tile_id] = 0;
#pragma unroll
        for (int i = 0; i < NI; ++i) {
          f32x4 y;
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            const int m = 16 * (a_block0 + i) + 4 * g + q;
            y[q] = (m < M && n < N) ? ((const float*)out)[(size_t)m * ldo + n] : 0.0f;   // the chain starts at the residual
          }
          for (int sg = 0; sg < nseg; ++sg)
            y = y + __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(rs_s, mine + i * 1024, sg * cell, 16));
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            const int m = 16 * (a_block0 + i) + 4 * g + q;
            if (m < M && n < N) ((float*)out)[(size_t)m * ldo + n] = y[q];
          }
        }
        return;
      }
    }
    if (n >= N) return;
#pragma unroll
    for (int i = 0; i < NI; ++i)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int m = 16 * (a_block0 + i) + 4 * g + q;
        if (m >= M) continue;
        if constexpr (OLD_FIRST) ((float*)out)[(size_t)m * ldo + n] = old_out[i][q] + acc[i][0][q];
        else epilogue_store<EPI, CH>(out, (size_t)m * ldo + n, acc[i][0][q], acc[i][NJ - 1][q]);
      }
  }
}

template <int EPI, int NRB, bool NORM, bool NARROW, bool EIGHT>
__global__ __launch_bounds__((64 * MidShape<EPI, NRB, NORM, NARROW, EIGHT>::NW)) void gemm_bf16_mid_kernel(
    const bf16_t* __restrict__ x, const bf16_t* __restrict__ w, void* __restrict__ out, int M, int N, int K, int ldx, int ldo,
    MidNormArgs na, QkvRopeArgs rp, MidSplitArgs sp) {
  mid_body<EPI, NRB, NORM, NARROW, EIGHT, false>(x, w, out, M, N, K, ldx, ldo, na, rp, sp, launch_ctx());
}


template <int EPI, int NRB, bool NORM, bool NARROW, bool EIGHT>
static int launch_mid_waves(const bf16_t* x, const bf16_t* w, void* out, int M, int N, int K, int ldx, int ldo, int wgs, hipStream_t s,
                            const MidNormArgs& na, const QkvRopeArgs& rp, int segments, const MidSplitArgs& sp, int row_blocks) {
  using S = MidShape<EPI, NRB, NORM, NARROW, EIGHT>;
  static bool allowed = false;                       // more than 64 KB of dynamic LDS has to be asked for once
  const int lds_bytes = NORM ? mid_norm_lds_bytes(S::RING, K, na.row_step) : S::RING;
  if (lds_bytes > BW_LDS_LIMIT) return -2;
  if (!allowed) {
    (void)hipFuncSetAttribute((const void*)gemm_bf16_mid_kernel<EPI, NRB, NORM, NARROW, EIGHT>, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    allowed = true;
  }
  if (chain_is_open()) {
    constexpr int kind = mid_chain_kind<EPI, NRB, NORM, NARROW, EIGHT>();
    if constexpr (kind >= 0) {
      if (segments == 1 && row_blocks == 1 && (size_t)M * na.ldx32 * 4 < ((size_t)1 << 31))
        return chain_record_mid(kind, MidCall{w, out, M, N, K, ldo, na, rp}, wgs, lds_bytes, s);
    }
  }
  BW_LAUNCH((gemm_bf16_mid_kernel<EPI, NRB, NORM, NARROW, EIGHT>), dim3(wgs, segments, row_blocks), dim3(64 * S::NW), lds_bytes, s, x, w, out, M, N, K, ldx, ldo, na, rp, sp);
  return BW_LAUNCH_CHECK();
}

template <int EPI, int NRB, bool NORM, bool NARROW = false>
static int launch_mid(const bf16_t* x, const bf16_t* w, void* out, int M, int N, int K, int ldx, int ldo, int wgs, hipStream_t s,
                      const MidNormArgs& na = MidNormArgs{}, const QkvRopeArgs& rp = QkvRopeArgs{}, int segments = 1,
                      const MidSplitArgs& sp = MidSplitArgs{}, int row_blocks = 1) {
  // 17 rows or more, or rows normalised in the kernel (a row a wave sooner done than two), K in whole stages: the
  // eight-wave variant (the same bits)
  if constexpr (NORM || NRB >= 2) {
    if (K % (64 * MidShape<EPI, NRB, NORM, NARROW, true>::SUB) == 0)
      return launch_mid_waves<EPI, NRB, NORM, NARROW, true>(x, w, out, M, N, K, ldx, ldo, wgs, s, na, rp, segments, sp, row_blocks);
  }
  return launch_mid_waves<EPI, NRB, NORM, NARROW, false>(x, w, out, M, N, K, ldx, ldo, wgs, s, na, rp, segments, sp, row_blocks);
}

// RMSNorm of up to 16 rows of the residual stream + product with many columns in one kernel; -7: not this shape.
int bw_norm_gemm_mid(const float* x32, int ldx32, const void* norm_w, int norm_w_is_bf16, float eps, const void* w, void* out,
                     int ldo, int M, int N, int K, int epilogue, void* stream) {
  const int cols = epilogue == EPI_SWIGLU_BF16 ? 32 : 64;
  const int wgs = (N + cols - 1) / cols;
  // (rows of two segments of K: eight of them at most, a row a wave, sixteen vectors a lane; LDS holds 8-row blocks)
  if (!mid_norm_admits(M, K, wgs)) return -7;
  MidNormArgs na{x32, norm_w, ldx32, norm_w_is_bf16, eps, mid_norm_row_step(K)};
  const bf16_t* wp = (const bf16_t*)w;
  hipStream_t s = (hipStream_t)stream;
  switch (epilogue) {
    case EPI_F32: return launch_mid<EPI_F32, 1, true>(nullptr, wp, out, M, N, K, 0, ldo, wgs, s, na);
    case EPI_BF16: return launch_mid<EPI_BF16, 1, true>(nullptr, wp, out, M, N, K, 0, ldo, wgs, s, na);
    case EPI_ADD_F32: return launch_mid<EPI_ADD_F32, 1, true>(nullptr, wp, out, M, N, K, 0, ldo, wgs, s, na);
    case EPI_SWIGLU_BF16: return launch_mid<EPI_SWIGLU_BF16, 1, true>(nullptr, wp, out, M, N, K, 0, ldo, wgs, s, na);
  }
  return -7;
}

// Whether bw_norm_gemm_mid takes rows of this width that the other fused kernels do not (wider than a segment of K).
extern "C" int bw_norm_gemm_wide_supported(int M, int N, int K, int cols) {
  return cols > 0 && K > GEMM_SEG && mid_norm_admits(M, K, (N + cols - 1) / cols);
}

#define ROPE_NARROW_BELOW 256

// The stacked q|k|v product of up to 64 normalised rows with rotation and cache write in its epilogue, for heads of
// 64 and at least 64 of them (a workgroup a head); -7: not this shape.
static int launch_qkv_rope_mid(const bf16_t* x, int ldx, const bf16_t* w_qkv, void* q_out, int M, int K, const QkvRopeArgs& rp,
                               hipStream_t s) {
  const int all_heads = rp.heads + 2 * rp.kv_heads, hd = rp.head_dim;
  const int wide_tiles = all_heads * (hd / 64);         // workgroups with 32 pairs each
  if (K % 64 || hd % 64 || wide_tiles < 64 || (size_t)M * ldx * 2 >= ((size_t)1 << 31)) return -7;
  const int N = all_heads * hd, ldo = rp.heads * hd;
  if (M > 64) {
    // a short prompt portion: blocks of 64 rows in one launch, while all of them fit the chip at once
    const int zb = (M + 63) / 64;
    if (wide_tiles * zb > 512) return -7;
    if (2 * wide_tiles * zb <= 256 && wide_tiles < ROPE_NARROW_BELOW)      // (half heads only while they leave compute units idle)
      return launch_mid<EPI_QKV_ROPE, 4, false, true>(x, w_qkv, q_out, M, N, K, ldx, ldo, 2 * wide_tiles, s, MidNormArgs{}, rp, 1,
                                                      MidSplitArgs{}, zb);
    return launch_mid<EPI_QKV_ROPE, 4, false>(x, w_qkv, q_out, M, N, K, ldx, ldo, wide_tiles, s, MidNormArgs{}, rp, 1, MidSplitArgs{}, zb);
  }
  if (wide_tiles < ROPE_NARROW_BELOW) {                // fewer workgroups than compute units: 16 pairs a workgroup
    if (M <= 16) return launch_mid<EPI_QKV_ROPE, 1, false, true>(x, w_qkv, q_out, M, N, K, ldx, ldo, 2 * wide_tiles, s, MidNormArgs{}, rp);
    if (M <= 32) return launch_mid<EPI_QKV_ROPE, 2, false, true>(x, w_qkv, q_out, M, N, K, ldx, ldo, 2 * wide_tiles, s, MidNormArgs{}, rp);
    return launch_mid<EPI_QKV_ROPE, 4, false, true>(x, w_qkv, q_out, M, N, K, ldx, ldo, 2 * wide_tiles, s, MidNormArgs{}, rp);
  }
  if (M <= 16) return launch_mid<EPI_QKV_ROPE, 1, false>(x, w_qkv, q_out, M, N, K, ldx, ldo, wide_tiles, s, MidNormArgs{}, rp);
  if (M <= 32) return launch_mid<EPI_QKV_ROPE, 2, false>(x, w_qkv, q_out, M, N, K, ldx, ldo, wide_tiles, s, MidNormArgs{}, rp);
  return launch_mid<EPI_QKV_ROPE, 4, false>(x, w_qkv, q_out, M, N, K, ldx, ldo, wide_tiles, s, MidNormArgs{}, rp);
}

// RMSNorm of up to 16 rows + the stacked q|k|v product + rotation + cache write in one kernel, for heads of 64
// and at least 64 of them (a workgroup a head); -7: not this shape.
int bw_norm_qkv_rope_mid(const float* x32, int ldx32, const void* norm_w, int norm_w_is_bf16, float eps, const void* w_qkv,
                         void* q_out, const int32_t* positions, const int32_t* row_seq, const int32_t* block_table,
                         int table_stride, const float* cos_table, const float* sin_table, void* k_cache, void* v_cache, int M,
                         int heads, int kv_heads, int head_dim, int K, int page_size, int write_cache, void* stream) {
  const int all_heads = heads + 2 * kv_heads;
  const int wide_tiles = all_heads * (head_dim / 64);
  if (head_dim % 64 || !mid_norm_admits(M, K, wide_tiles)) return -7;        // as in bw_norm_gemm_mid
  MidNormArgs na{x32, norm_w, ldx32, norm_w_is_bf16, eps, mid_norm_row_step(K)};
  if (page_size <= 0 || (page_size & (page_size - 1))) return -5;
  QkvRopeArgs rp{positions, row_seq, block_table, cos_table, sin_table, (bf16_t*)k_cache, (bf16_t*)v_cache,
                 heads, kv_heads, page_size, table_stride, write_cache, __builtin_ctz((unsigned)page_size), head_dim};
  if (wide_tiles < ROPE_NARROW_BELOW)
    return launch_mid<EPI_QKV_ROPE, 1, true, true>(nullptr, (const bf16_t*)w_qkv, q_out, M, all_heads * head_dim, K, 0,
                                                   heads * head_dim, 2 * wide_tiles, (hipStream_t)stream, na, rp);
  return launch_mid<EPI_QKV_ROPE, 1, true>(nullptr, (const bf16_t*)w_qkv, q_out, M, all_heads * head_dim, K, 0, heads * head_dim,
                                           wide_tiles, (hipStream_t)stream, na, rp);
}

// ------------------------------------------------------------------------------ up to 16 rows, few columns

// The skinny kernel's division of work (a wave per strip of CW columns and segment of K; the waves of
// a strip join their segment sums through LDS in segment order) with the loads of the kernel above:
// every wave owns a ring of STREAM_STAGES stages in LDS, a stage being a step's 64 elements of its CW
// rows of W and of the 16 rows of x, fetched by buffer loads with LDS as destination in whole cache
// lines; LPW loads a stage, so "all but the last LPW * (stages - 2)" is the wait for the stage at
// hand.  Nothing is shared between waves, so the loop has no barrier.  K a multiple of 64.
// XR: rows of x a stage holds, 16, or 8 where there are no more than 8 (lanes that stand for rows 8 to 15 read rows
// 0 to 7 again; their products go nowhere): a load less a stage, so more stages of W in flight.
// DEPTH: loads a wave keeps in flight, 24, or fewer for a workgroup of more than four waves (a product of five to eight
// segments of K: a wave a segment, all at once, where four waves would take the segments in two turns; the rings of
// eight waves fit the compute unit's LDS only if they are shallower).
template <int CW, int XR = 16, int DEPTH = 24>
struct StreamShape {
  static constexpr int A_LOADS = XR / 8, B_LOADS = CW / 8, LPW = A_LOADS + B_LOADS;
  static constexpr int A_BYTES = A_LOADS * 1024;
  static constexpr int STAGE = A_BYTES + B_LOADS * 1024;            // x: XR rows of 128 bytes, then W
  static constexpr int STAGES = DEPTH / LPW + 2;
  static constexpr int RING = STAGES * STAGE;
  static_assert(LPW * (STAGES - 2) == DEPTH, "the wait for a stage counts DEPTH loads in flight");
};
#define STREAM_DEPTH_MANY(CW) ((CW) == 16 ? 15 : 14)               // (with 8 rows of x a stage: seven and nine stages)

// A wave's loads of one stage of its ring (a device function rather than a lambda in the kernel: the
// host pass drops, without a word, kernel templates whose lambdas capture arrays of dependent size).
// DO_X, DO_W: which of the stage's loads (a phase of a launch of several asks for the weights of its first stages
// before the rows); DEV: x at device scope.
template <int CW, int XR, bool DO_X = true, bool DO_W = true, bool DEV = false, int DEPTH = 24>
__device__ __forceinline__ void stream_issue(unsigned char* ring, __amdgpu_buffer_rsrc_t rs_x, __amdgpu_buffer_rsrc_t rs_w,
                                             const int* voff_x, const int* voff_w, int step, int steps, int k_begin) {
  using SH = StreamShape<CW, XR, DEPTH>;
  typedef __attribute__((address_space(3))) void* lds_ptr;
  unsigned char* dst = ring + (step % SH::STAGES) * SH::STAGE;
  const bool real = step < steps;                                  // scalar; past the segment: outside the descriptors
  const int soff = (k_begin + step * 64) * 2;
  if constexpr (DO_X) {
#pragma unroll
    for (int t = 0; t < SH::A_LOADS; ++t)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_x, (lds_ptr)(dst + t * 1024), 16, real ? voff_x[t] : 0x7ffffff0, soff, 0, DEV ? 16 : 0);
  }
  if constexpr (DO_W) {
#pragma unroll
    for (int t = 0; t < SH::B_LOADS; ++t)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_w, (lds_ptr)(dst + SH::A_BYTES + t * 1024), 16, real ? voff_w[t] : 0x7ffffff0, soff, 0, 0);
  }
}

// CH: as a phase of a launch of several (ChainCtx): x and the outputs' old values were written by the phase before, so a
// wave asks for the weights of its first segment's first stages, waits, and asks for their rows of x then (loads
// complete in the order they are issued: until the ring has turned once the wait for a stage lets fewer loads stay in
// flight); x, old values and outputs travel at device scope.
template <int EPI, int CW, int XR, bool CH, int DEPTH = 24>
__device__ __forceinline__ void stream_body(const bf16_t* __restrict__ x, const bf16_t* __restrict__ w, void* __restrict__ out, int M, int N,
                                            int K, int ldx, int ldo, int S, const ChainCtx& cc) {
  using SH = StreamShape<CW, XR, DEPTH>;
  extern __shared__ __attribute__((aligned(16))) unsigned char stream_lds[];   // [waves][ring], then [S][4][64] floats when S > 1
  const int wave = wave_index(), lane = threadIdx.x & 63, nwaves = cc.waves;
  const int r = lane & 15, g = lane >> 4;
  const int c = r % CW;
  const int n0 = cc.bx * CW;
  const bool n_ok = r < CW && n0 + c < N;
  const int w_rows = min(CW, N - n0);
  const __amdgpu_buffer_rsrc_t rs_w =
      __builtin_amdgcn_make_buffer_rsrc((void*)(w + (size_t)n0 * K), 0, (int)((size_t)w_rows * K * 2), 0x00020000);
  const __amdgpu_buffer_rsrc_t rs_x =
      __builtin_amdgcn_make_buffer_rsrc((void*)x, 0, (int)((((size_t)M - 1) * ldx + K) * 2), 0x00020000);
  // loads: lane l fetches row l / 8 of its 8, chunk (l % 8) ^ (row within 16 >> 1) of the row's 128 bytes
  const int lrow = lane >> 3, lslot = lane & 7;
  int voff_x[2], voff_w[SH::B_LOADS];
#pragma unroll
  for (int t = 0; t < 2; ++t) voff_x[t] = ((8 * t + lrow) * ldx + 8 * (lslot ^ ((8 * t + lrow) >> 1))) * 2;
#pragma unroll
  for (int t = 0; t < SH::B_LOADS; ++t) voff_w[t] = ((8 * t + lrow) * K + 8 * (lslot ^ ((8 * t + lrow) >> 1))) * 2;
  // operand reads: lane (g, r) wants row r (of W: r % CW), chunk 4*kk + g: slot (4*kk + g) ^ (row >> 1)
  int off_x[2], off_w[2];
  const int rx = XR == 8 ? (r & 7) : r;                              // the row of x this lane reads
#pragma unroll
  for (int kk = 0; kk < 2; ++kk) {
    off_x[kk] = (rx >> 3) * 1024 + (rx & 7) * 128 + (((4 * kk + g) ^ (rx >> 1)) * 16);
    off_w[kk] = SH::A_BYTES + (c >> 3) * 1024 + (c & 7) * 128 + (((4 * kk + g) ^ (c >> 1)) * 16);
  }
  unsigned char* ring = stream_lds + wave * SH::RING;
  float* red = reinterpret_cast<float*>(stream_lds + nwaves * SH::RING);
  // A residual add: the wave that stores asks for its outputs' old values before anything else (loads older than
  // the ring's, so every wait below covers them); asked for at the end they were one more trip to memory.
  float old_out[4] = {0.f, 0.f, 0.f, 0.f};
  auto ask_old = [&]() {
    if constexpr (EPI == EPI_ADD_F32) {
      if (wave == 0 && n_ok) {
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int m = 4 * g + q;
          if (m < M) old_out[q] = ld_f32<CH>((const float*)out + (size_t)m * ldo + n0 + c);
        }
      }
      asm volatile("" ::: "memory");
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  if constexpr (!CH) ask_old();
  f32x4 acc = {0.f, 0.f, 0.f, 0.f};
  for (int s = wave; s < S; s += nwaves) {
    const int k_begin = s * GEMM_SEG;
    const int steps = ((K - k_begin) < GEMM_SEG ? K - k_begin : GEMM_SEG) / 64;
    acc = (f32x4){0.f, 0.f, 0.f, 0.f};
    const bool first_turn = CH && s == wave;                       // (scalar) the segment whose x had to wait
    if (first_turn) {
#pragma unroll
      for (int st = 0; st < SH::STAGES - 1; ++st) stream_issue<CW, XR, false, true, CH, DEPTH>(ring, rs_x, rs_w, voff_x, voff_w, st, steps, k_begin);
      asm volatile("" ::: "memory");
      __builtin_amdgcn_sched_barrier(0);
      chain_wait<CH>(cc);
      ask_old();
#pragma unroll
      for (int st = 0; st < SH::STAGES - 1; ++st) stream_issue<CW, XR, true, false, CH, DEPTH>(ring, rs_x, rs_w, voff_x, voff_w, st, steps, k_begin);
    } else {
#pragma unroll
      for (int st = 0; st < SH::STAGES - 1; ++st) stream_issue<CW, XR, true, true, CH, DEPTH>(ring, rs_x, rs_w, voff_x, voff_w, st, steps, k_begin);
    }
    for (int step = 0; step < steps; ++step) {
      // the stage at hand has landed when all but the loads of the stages after it have: 24, or, while x of the
      // first stages was asked for behind their weights, what is left of x (B_LOADS fewer a stage) and what came since
      if (first_turn && step < SH::STAGES - 2) __builtin_amdgcn_s_waitcnt(vmcnt_only(SH::A_LOADS * (SH::STAGES - 2)));
      else __builtin_amdgcn_s_waitcnt(vmcnt_only(DEPTH));
      asm volatile("" ::: "memory");
      const unsigned char* stage = ring + (step % SH::STAGES) * SH::STAGE;
      u32x4 fa[2], fb[2];
#pragma unroll
      for (int kk = 0; kk < 2; ++kk) {
        fa[kk] = *reinterpret_cast<const u32x4*>(stage + off_x[kk]);
        fb[kk] = *reinterpret_cast<const u32x4*>(stage + off_w[kk]);
      }
#pragma unroll
      for (int kk = 0; kk < 2; ++kk)
        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(fa[kk]), as_bf16x8(fb[kk]), acc, 0, 0, 0);
      // the reads above are done (their values were used) before the stage is asked for again
      asm volatile("" ::: "memory");
      stream_issue<CW, XR, true, true, CH, DEPTH>(ring, rs_x, rs_w, voff_x, voff_w, step + SH::STAGES - 1, steps, k_begin);
    }
    __builtin_amdgcn_s_waitcnt(0x0f70);                            // the padding loads too, before the ring is reused
    if (S > 1) {
#pragma unroll
      for (int q = 0; q < 4; ++q) red[(s * 4 + q) * 64 + lane] = acc[q];
    }
  }
  if (S > 1) {
    __syncthreads();
    if (wave != 0) return;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      float y = red[q * 64 + lane];
      if constexpr (EPI == EPI_ADD_F32) {            // the chain of additions starts at the residual
        const int m = 4 * g + q;
        if (n_ok && m < M) y = old_out[q] + y;
      }
      for (int s = 1; s < S; ++s) y += red[(s * 4 + q) * 64 + lane];
      acc[q] = y;
    }
  }
  if (!n_ok) return;
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    const int m = 4 * g + q;
    if (m >= M) continue;
    if constexpr (EPI == EPI_ADD_F32) {
      // (several segments: the residual is in already; one: old + sum, the addition of the store that reads)
      st_f32<CH>((float*)out + (size_t)m * ldo + n0 + c, S > 1 ? acc[q] : old_out[q] + acc[q]);
    } else {
      epilogue_store<EPI, CH>(out, (size_t)m * ldo + n0 + c, acc[q], acc[q]);
    }
  }
}

template <int EPI, int CW, int XR = 16, int DEPTH = 24>
__global__ __launch_bounds__(DEPTH == 24 ? 256 : 512) void gemm_bf16_stream_kernel(const bf16_t* __restrict__ x, const bf16_t* __restrict__ w,
                                                                                   void* __restrict__ out, int M, int N, int K, int ldx,
                                                                                   int ldo, int S) {
  stream_body<EPI, CW, XR, false, DEPTH>(x, w, out, M, N, K, ldx, ldo, S, launch_ctx());
}

// Five to eight segments of K and no more than 8 rows: a wave a segment, all at once, with shallower rings.
template <int EPI, int CW>
static int launch_stream_many(const bf16_t* x, const bf16_t* w, void* out, int M, int N, int K, int ldx, int ldo, int S, hipStream_t s) {
  constexpr int DEPTH = STREAM_DEPTH_MANY(CW);
  using SH = StreamShape<CW, 8, DEPTH>;
  const size_t lds_bytes = (size_t)S * SH::RING + (size_t)S * 4 * 64 * sizeof(float);
  if (S < 5 || S > 8 || lds_bytes > BW_LDS_LIMIT - 256) return -7;
  static bool allowed = false;                       // more than 64 KB of dynamic LDS has to be asked for once
  if (!allowed) {
    (void)hipFuncSetAttribute((const void*)gemm_bf16_stream_kernel<EPI, CW, 8, DEPTH>, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    allowed = true;
  }
  BW_LAUNCH((gemm_bf16_stream_kernel<EPI, CW, 8, DEPTH>), dim3((N + CW - 1) / CW), dim3(64 * S), lds_bytes, s, x, w, out, M, N, K, ldx, ldo, S);
  return BW_LAUNCH_CHECK();
}

template <int EPI, int CW, int XR>
static int launch_stream_rows(const bf16_t* x, const bf16_t* w, void* out, int M, int N, int K, int ldx, int ldo, int S, hipStream_t s) {
  using SH = StreamShape<CW, XR>;
  if constexpr (XR == 8) {
    const int rc = launch_stream_many<EPI, CW>(x, w, out, M, N, K, ldx, ldo, S, s);
    if (rc != -7) return rc;
  }
  const int waves = S < 4 ? S : 4;
  const size_t lds_bytes = (size_t)waves * SH::RING + (S > 1 ? (size_t)S * 4 * 64 * sizeof(float) : 0);
  if (lds_bytes > 160 * 1024) return -2;
  static bool allowed = false;                       // more than 64 KB of dynamic LDS has to be asked for once
  if (!allowed) {
    (void)hipFuncSetAttribute((const void*)gemm_bf16_stream_kernel<EPI, CW, XR>, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    allowed = true;
  }
  if (chain_is_open()) {
    constexpr int kind = stream_chain_kind<EPI, CW, XR>();
    if constexpr (kind >= 0) return chain_record_rows(kind, RowsCall{x, w, out, M, N, K, ldx, ldo, S}, (N + CW - 1) / CW, waves, (int)lds_bytes, s);
  }
  BW_LAUNCH((gemm_bf16_stream_kernel<EPI, CW, XR>), dim3((N + CW - 1) / CW), dim3(64 * waves), lds_bytes, s, x, w, out, M, N,
                     K, ldx, ldo, S);
  return BW_LAUNCH_CHECK();
}

template <int EPI, int CW>
static int launch_stream(const bf16_t* x, const bf16_t* w, void* out, int M, int N, int K, int ldx, int ldo, int S, hipStream_t s) {
  // (how many rows a stage holds changes no bit: the chain of a row is the same statements on the same values)
  if (M <= 8) return launch_stream_rows<EPI, CW, 8>(x, w, out, M, N, K, ldx, ldo, S, s);
  return launch_stream_rows<EPI, CW, 16>(x, w, out, M, N, K, ldx, ldo, S, s);
}

// ------------------------------------------------------------------------------ up to 16 rows, few columns, one segment

// A product so small that a ring would never fill (the output projection of a decode step: 8 MB of
// weights for 256 compute units): a workgroup of four waves takes 8 columns, and everything it needs,
// all of its 8 rows of W and the 16 rows of x, is asked for at once, straight into LDS, wave w asking for
// the steps w, w + 4, ... of K; nothing waits for a ring slot, so the whole weight is in flight within
// the kernel's first hundred nanoseconds.  Loads land in the order they were asked for: when every
// wave's q-th step has landed, steps 4q .. 4q + 3 are there, and wave 0 runs them through the one chain
// of the workgroup's 16 x 16 block while the later ones are still on their way.  The stage layout and
// the chain are the stream kernel's: the same bits.  K a multiple of 64, at most BURST_STEPS steps.
#define BURST_STEPS 32
#define BURST_STAGE 3072                                           // x: 16 rows of 128 bytes, then 8 rows of W

// CH: as a phase of a launch of several (ChainCtx): all the weights are asked for, then the wait for the phase before,
// then the old values and x at device scope; a wave's q-th step is there when all but its last 2 * (7 - q) loads are.
template <int EPI, bool CH>
__device__ __forceinline__ void burst_body(const bf16_t* __restrict__ x, const bf16_t* __restrict__ w, void* __restrict__ out, int M, int N,
                                           int K, int ldx, int ldo, const ChainCtx& cc) {
  extern __shared__ __attribute__((aligned(16))) unsigned char burst_lds[];   // [BURST_STEPS][BURST_STAGE]
  typedef __attribute__((address_space(3))) void* lds_ptr;
  const int wave = wave_index(), lane = threadIdx.x & 63;
  const int r = lane & 15, g = lane >> 4;
  const int c = r & 7;
  const int n0 = cc.bx * 8;
  const bool n_ok = r < 8 && n0 + c < N;
  const int w_rows = min(8, N - n0);
  const __amdgpu_buffer_rsrc_t rs_w =
      __builtin_amdgcn_make_buffer_rsrc((void*)(w + (size_t)n0 * K), 0, (int)((size_t)w_rows * K * 2), 0x00020000);
  const __amdgpu_buffer_rsrc_t rs_x =
      __builtin_amdgcn_make_buffer_rsrc((void*)x, 0, (int)((((size_t)M - 1) * ldx + K) * 2), 0x00020000);
  const int lrow = lane >> 3, lslot = lane & 7;
  int voff_x[2];
#pragma unroll
  for (int t = 0; t < 2; ++t) voff_x[t] = ((8 * t + lrow) * ldx + 8 * (lslot ^ ((8 * t + lrow) >> 1))) * 2;
  const int voff_w = (lrow * K + 8 * (lslot ^ (lrow >> 1))) * 2;
  const int steps = K / 64;
  // A residual add: the wave that stores asks for its outputs' old values before anything else (older than its loads
  // of the steps, so every wait below covers them); asked for at the end they were one more trip to memory.
  float old_out[4] = {0.f, 0.f, 0.f, 0.f};
  auto ask_old = [&]() {
    if constexpr (EPI == EPI_ADD_F32) {
      if (wave == 0 && n_ok) {
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int m = 4 * g + q;
          if (m < M) old_out[q] = ld_f32<CH>((const float*)out + (size_t)m * ldo + n0 + c);
        }
      }
      asm volatile("" ::: "memory");
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  // eight steps a wave, whatever K: those past K are asked for outside the descriptors (no traffic, zeros), so
  // that the counts below are the same for every wave
  if constexpr (CH) {
#pragma unroll
    for (int i = 0; i < BURST_STEPS / 4; ++i) {
      const int st = wave + 4 * i;
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_w, (lds_ptr)(burst_lds + st * BURST_STAGE + 2048), 16, st < steps ? voff_w : 0x7ffffff0, st * 128, 0, 0);
    }
    asm volatile("" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);
    chain_wait<CH>(cc);
    ask_old();
#pragma unroll
    for (int i = 0; i < BURST_STEPS / 4; ++i) {
      const int st = wave + 4 * i;
      const bool real = st < steps;                                // scalar
#pragma unroll
      for (int t = 0; t < 2; ++t)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_x, (lds_ptr)(burst_lds + st * BURST_STAGE + t * 1024), 16, real ? voff_x[t] : 0x7ffffff0, st * 128, 0, 16);
    }
  } else {
    ask_old();
#pragma unroll
    for (int i = 0; i < BURST_STEPS / 4; ++i) {
      const int st = wave + 4 * i;
      const bool real = st < steps;                                  // scalar
      unsigned char* dst = burst_lds + st * BURST_STAGE;
#pragma unroll
      for (int t = 0; t < 2; ++t)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_x, (lds_ptr)(dst + t * 1024), 16, real ? voff_x[t] : 0x7ffffff0, st * 128, 0, 0);
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_w, (lds_ptr)(dst + 2048), 16, real ? voff_w : 0x7ffffff0, st * 128, 0, 0);
    }
  }
  int off_x[2], off_w[2];
#pragma unroll
  for (int kk = 0; kk < 2; ++kk) {
    off_x[kk] = (r >> 3) * 1024 + (r & 7) * 128 + (((4 * kk + g) ^ (r >> 1)) * 16);
    off_w[kk] = 2048 + c * 128 + (((4 * kk + g) ^ (c >> 1)) * 16);
  }
  f32x4 acc = {0.f, 0.f, 0.f, 0.f};
  auto run_steps = [&](int q) {                                     // steps 4q .. 4q + 3 of the chain (wave 0)
    for (int step = 4 * q; step < 4 * q + 4 && step < steps; ++step) {
      const unsigned char* stage = burst_lds + step * BURST_STAGE;
      u32x4 fa[2], fb[2];
#pragma unroll
      for (int kk = 0; kk < 2; ++kk) {
        fa[kk] = *reinterpret_cast<const u32x4*>(stage + off_x[kk]);
        fb[kk] = *reinterpret_cast<const u32x4*>(stage + off_w[kk]);
      }
#pragma unroll
      for (int kk = 0; kk < 2; ++kk)
        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(fa[kk]), as_bf16x8(fb[kk]), acc, 0, 0, 0);
    }
  };
  // the wave's q-th step has landed when all but its last 3 * (7 - q) loads have
#define BURST_ROUND(Q, WAIT)                                   \
  if (4 * (Q) < steps) {                                       \
    __builtin_amdgcn_s_waitcnt(WAIT);                          \
    __builtin_amdgcn_s_barrier();                              \
    asm volatile("" ::: "memory");                             \
    if (wave == 0) run_steps(Q);                               \
  }
  BURST_ROUND(0, vmcnt_only(CH ? 14 : 21))
  BURST_ROUND(1, vmcnt_only(CH ? 12 : 18))
  BURST_ROUND(2, vmcnt_only(CH ? 10 : 15))
  BURST_ROUND(3, vmcnt_only(CH ? 8 : 12))
  BURST_ROUND(4, vmcnt_only(CH ? 6 : 9))
  BURST_ROUND(5, vmcnt_only(CH ? 4 : 6))
  BURST_ROUND(6, vmcnt_only(CH ? 2 : 3))
  BURST_ROUND(7, vmcnt_only(0))
#undef BURST_ROUND
  __builtin_amdgcn_s_waitcnt(vmcnt_only(0));                        // the padding loads too, before the wave ends
  if (wave != 0 || !n_ok) return;
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    const int m = 4 * g + q;
    if (m >= M) continue;
    if constexpr (EPI == EPI_ADD_F32) st_f32<CH>((float*)out + (size_t)m * ldo + n0 + c, old_out[q] + acc[q]);
    else epilogue_store<EPI, CH>(out, (size_t)m * ldo + n0 + c, acc[q], acc[q]);
  }
}

template <int EPI>
__global__ __launch_bounds__(256) void gemm_bf16_burst_kernel(const bf16_t* __restrict__ x, const bf16_t* __restrict__ w,
                                                              void* __restrict__ out, int M, int N, int K, int ldx, int ldo) {
  burst_body<EPI, false>(x, w, out, M, N, K, ldx, ldo, launch_ctx());
}

template <int EPI>
static int launch_burst(const bf16_t* x, const bf16_t* w, void* out, int M, int N, int K, int ldx, int ldo, hipStream_t s) {
  static bool allowed = false;                       // more than 64 KB of dynamic LDS has to be asked for once
  if (!allowed) {
    (void)hipFuncSetAttribute((const void*)gemm_bf16_burst_kernel<EPI>, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    allowed = true;
  }
  if (chain_is_open()) {
    if constexpr (EPI == EPI_ADD_F32) return chain_record_rows(CK_BURST_ADD, RowsCall{x, w, out, M, N, K, ldx, ldo, 1}, (N + 7) / 8, 4, BURST_STEPS * BURST_STAGE, s);
  }
  BW_LAUNCH((gemm_bf16_burst_kernel<EPI>), dim3((N + 7) / 8), dim3(256), BURST_STEPS * BURST_STAGE, s, x, w, out, M, N, K,
                     ldx, ldo);
  return BW_LAUNCH_CHECK();
}
