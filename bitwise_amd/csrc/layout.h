// Index arithmetic of the kernels that normalise rows into LDS in front of a matrix product, as plain functions
// that compile for the host too: which shapes a launcher admits, how many bytes of LDS it asks for, where a lane
// stores and reads there, and which vector of a row a lane loads from memory.  The kernels call these functions
// and nothing else for those addresses, so a host program can walk every admitted shape, wave, lane and step and
// check each offset against the launch's own sizes (tests/layout_sweep.cpp does, with the compiler's address and
// undefined-behaviour checks switched on).  No HIP header is needed to include this file.
#pragma once

#include <stddef.h>

#if defined(__HIPCC__)
#define BW_HD __host__ __device__ __forceinline__
#else
#define BW_HD inline
#endif

enum { EPI_F32 = 0, EPI_BF16 = 1, EPI_ADD_F32 = 2, EPI_SWIGLU_BF16 = 3, EPI_QKV_ROPE = 4 };

#define GEMM_SEG 2048                 // a segment of K: sums of different segments are joined left to right
#define BW_LDS_LIMIT (160 * 1024)     // bytes of LDS a workgroup of gfx950 may ask for

// ------------------------------------------------------------------------------ rows held in a wave's registers

// Lane ``lane`` owns the 16-byte vectors lane, lane + 64, ... of a row of ``nvec`` vectors; its j-th register
// holds vector 64 j + lane, or, past the row's end, the row's last vector again (loaded so that no load is
// conditional, never used).
BW_HD int norm_vec_index(int j, int lane, int nvec) {
  const int c = 64 * j + lane;
  return c < nvec ? c : nvec - 1;
}
BW_HD bool norm_vec_in_row(int j, int lane, int nvec) { return 64 * j + lane < nvec; }

// ------------------------------------------------------------------------------ gemm_bf16_mid_kernel

// The shape of gemm_bf16_mid_kernel's workgroup and ring for one set of template arguments (see the kernel).
template <int EPI, int NRB, bool NORM, bool NARROW = false, bool EIGHT = false>
struct MidShape {
  static constexpr bool GLU = EPI == EPI_SWIGLU_BF16;
  static constexpr bool HALVES = GLU || NARROW;                     // waves are (strip, half of the row blocks)
  static constexpr int NW = EIGHT ? 8 : 4;                          // waves
  static constexpr int COLS = HALVES ? 32 : 64;                     // output columns a workgroup
  static constexpr int B_ROWS = NARROW ? 32 : 64;                   // rows of W a step (SwiGLU: 32 gate, 32 up)
  static constexpr int SUB = EIGHT ? (B_ROWS == 64 ? (NORM || NRB == 4 ? 1 : 2) : (NORM ? 2 : 4)) : 1;   // steps of 64 along K a stage (NORM: weights only)
  static constexpr int STRIPS = COLS / 16, GROUPS = NW / STRIPS;    // wave = (strip of the columns, group of the row blocks)
  static constexpr int A_LOADS = NORM ? 0 : (SUB * 2 * NRB + NW - 1) / NW; // per wave and stage: 8 rows of x each
  static constexpr int B_LOADS = SUB * B_ROWS / 8 / NW;             // 8 rows of W each
  static constexpr int LPW = A_LOADS + B_LOADS;
  static constexpr int A_BYTES = NORM ? 0 : NRB * 2048, STEP_BYTES = A_BYTES + B_ROWS * 128, STAGE = SUB * STEP_BYTES;
  static constexpr int NI = NRB >= GROUPS ? NRB / GROUPS : 1;       // blocks of rows a wave works on (fewer blocks than groups: waves that only load)
  static constexpr int NJ = GLU ? 2 : 1;
  static constexpr bool ROPE_NARROW = NARROW && EPI == EPI_QKV_ROPE;  // a workgroup = 16 rotary pairs of a head
  // 17 rows or more: a ring of at most 72 KB, so that two workgroups share a compute unit and one's first loads
  // and epilogue lie under the other's steps (products with more workgroups than compute units: gate|up 17.2 ->
  // 16.0 us, the 8B shape's 53 -> 50 and its down projection 37 -> 35; the others unchanged); never fewer than 3
  static constexpr int FIT0 = (NORM || NRB < 2 ? 150 : 72) * 1024 / STAGE;
  static constexpr int FIT = FIT0 < 3 ? 3 : FIT0;
  static constexpr int STAGES = EIGHT ? (NORM ? 8 : (FIT > 6 ? 6 : FIT))
                                      : (ROPE_NARROW && NRB <= 2 ? 16 : 8);   // (half the weights a stage: twice the stages, where they fit)
  static constexpr int PENDING = LPW * (STAGES - 2);                // loads that may still be in flight at a step's start
  static constexpr int RING = STAGES * STAGE + 1024;                // and 1 KB where padding loads put their zeros
  static_assert(PENDING < 64, "the wait count has six bits");
  static_assert(STAGES >= 3, "a stage at hand, one landing, one asked for");
  static_assert(!NORM || NRB == 1, "rows are normalised in the kernel only up to 16 of them");
  static_assert(!NARROW || (!GLU && (EPI == EPI_QKV_ROPE || NRB >= 2)), "narrow tiles: plain epilogues of 17 rows or more, or the rotary one");
  static_assert(!EIGHT || NORM || (NRB >= 2 && (SUB * 2 * NRB) % NW == 0), "eight waves: 17 rows or more, or rows normalised in the kernel");
};

// A block of 16 rows of one step of 64 along K is 2 KB: rows 0-7 then rows 8-15, 128 bytes a row, the row's eight
// 16-byte chunks permuted by the row's number so that the operand reads of a wave hit distinct banks.  Lane
// (g = lane / 16, r = lane % 16) of a matrix instruction wants row r, chunk 4 kk + g for the half step kk.
BW_HD int mid_operand_offset(int r, int g, int kk) {
  return (r >> 3) * 1024 + (r & 7) * 128 + (((4 * kk + g) ^ (r >> 1)) * 16);
}

// The ring: stage ``step % STAGES``; a load is 8 rows of one step of 64 along K (1 KB).  Of x: block ``id % (2 NRB)``
// of step ``id / (2 NRB)`` of the stage for the wave's t-th load (ids past the stage's blocks are padding loads, whose
// zeros go behind the ring); of W likewise (SwiGLU with eight waves: the first four waves take the gate rows, the
// others the up rows, so that a wave's loads share a descriptor).  A step's bytes: the blocks of x, then those of W.
template <class S> BW_HD int mid_stage_offset(int step) { return (step % S::STAGES) * S::STAGE; }
template <class S> BW_HD int mid_padding_offset() { return S::STAGES * S::STAGE; }
template <class S, int NRB> BW_HD bool mid_a_load(int wave, int t, int& sub, int& block) {
  const int id = wave * S::A_LOADS + t;
  sub = id / (2 * NRB);
  block = id % (2 * NRB);
  return id < S::SUB * 2 * NRB;
}
template <class S> BW_HD int mid_a_dst(int sub, int block) { return sub * S::STEP_BYTES + block * 1024; }
template <class S> BW_HD void mid_b_load(int wave, int t, int& sub, int& blk) {
  constexpr int PER_STEP = S::B_ROWS / 8;
  if (S::NW == 8 && S::GLU) {                                        // waves 0-3: the gate rows, 4-7: the up rows
    const int id = (wave & 3) * S::B_LOADS + t;
    sub = id / (PER_STEP / 2);
    blk = id % (PER_STEP / 2) + (PER_STEP / 2) * (wave >> 2);
  } else {
    const int id = wave * S::B_LOADS + t;
    sub = id / PER_STEP;
    blk = id % PER_STEP;
  }
}
template <class S> BW_HD int mid_b_dst(int sub, int blk) { return sub * S::STEP_BYTES + S::A_BYTES + blk * 1024; }
// a wave's operand reads of W inside a step: its (gate) strip, the up strip 4 KB further
template <class S> BW_HD int mid_b_read_offset(int strip, int j, int r, int g, int kk) {
  return S::A_BYTES + strip * 2048 + j * 4096 + mid_operand_offset(r, g, kk);
}
// which block of 16 rows a wave starts at, and whether it has rows to work on at all (waves beyond the blocks of
// rows only load)
template <class S> BW_HD int mid_first_block(int wave) { return S::NI * (wave / S::STRIPS); }

// NORM variant: what the launcher admits.  Rows of one segment of K: up to 16 of them (LDS holds blocks of 16 rows,
// 2048 bytes a step).  Rows of up to two segments: up to 8, a row a wave, blocks of 8 rows, 1024 bytes a step.
// ``tiles``: workgroups of the launch (the kernel is for products with at least 64).
BW_HD bool mid_norm_admits(int M, int K, int tiles) {
  if (M < 1 || M > 16 || K < 64 || K % 64 || tiles < 64) return false;
  if (K > GEMM_SEG && (M > 8 || K > 2 * GEMM_SEG || K % 128)) return false;
  return true;
}
BW_HD int mid_norm_row_step(int K) { return K > GEMM_SEG ? 1024 : 2048; }

// Which rows a wave normalises: rows wave, wave + NW, ..., as many at a time as the rows need (a slot without a row
// would fetch a row for nothing); and how many 16-byte vectors of a row a lane holds: 8 (rows of one segment), or
// 16 (rows of two, which by the admission above are at most a row a wave of the eight-wave variant).
BW_HD int mid_norm_row_of(int wave, int i, int nw) { return wave + i * nw; }
BW_HD int mid_norm_rows_a_wave(int M, int nw) { return (M + nw - 1) / nw; }
BW_HD int mid_norm_vectors_a_lane(int K) { return K > GEMM_SEG ? 16 : 8; }

// Where vector c (elements 4c..4c+3 as four bfloat16, 8 bytes) of row m goes, relative to the rows' area: step
// c / 16, chunk (c % 16) / 2 of the step permuted as above, half c % 2 of the chunk.
BW_HD int mid_norm_store_offset(int c, int m, int row_step) {
  return (c >> 4) * row_step + (m >> 3) * 1024 + (m & 7) * 128 + ((((c & 15) >> 1) ^ ((m & 15) >> 1)) * 16) + (c & 1) * 8;
}

// Where lane (g, r) reads its 16 bytes of step ``k_step`` (of 64 along K) for the half step kk, relative to the rows' area.
BW_HD int mid_norm_read_offset(int k_step, int a_block, int row_step, int r, int g, int kk) {
  return k_step * row_step + a_block * 2048 + mid_operand_offset(r, g, kk);
}

// Bytes of LDS of a NORM launch: the ring, then the rows (8-row blocks: the reads of rows 8 to 15, which do not
// exist, end a block further).
BW_HD int mid_norm_lds_bytes(int ring, int K, int row_step) {
  return ring + (K / 64) * row_step + (row_step == 1024 ? 1024 : 0);
}

// ------------------------------------------------------------------------------ decode_gemm_kernel (fused_decode.hip)

#define DEC_SEG 2048
#define DEC_MAX_LDS (BW_LDS_LIMIT - 1024)

// LDS: [M rows of K + 8 bfloat16 (16 bytes of padding: operand reads hit distinct banks)] rounded up to 16 bytes,
// then a ring of ``stages`` stages of ``stage_bytes`` for each wave.
BW_HD int decode_lds_row(int K) { return K + 8; }                                  // bfloat16 elements
BW_HD size_t decode_rows_bytes(int M, int K) { return ((size_t)M * decode_lds_row(K) * 2 + 15) & ~(size_t)15; }
BW_HD size_t decode_ring_offset(int M, int K, int wave, int stages, int stage_bytes) {
  return decode_rows_bytes(M, K) + (size_t)wave * stages * stage_bytes;
}
BW_HD size_t decode_lds_bytes(int M, int K, int waves, int stages, int stage_bytes) {
  return decode_rows_bytes(M, K) + (size_t)waves * stages * stage_bytes;
}
// Can the rows live in LDS beside 64 KB of rings, and does a row fit a wave's registers?
BW_HD bool decode_gemm_admits(int M, int N, int K, int lda) {
  if (M <= 0 || M > 16 || N <= 0 || K <= 0 || (K % 64)) return false;
  if (K > DEC_SEG || (lda % 4) || lda < K) return false;
  if ((size_t)M * decode_lds_row(K) * 2 + 64 * 1024 > DEC_MAX_LDS) return false;
  return true;
}
// bfloat16 element where vector c of row m is stored, and where lane (g, r) reads its 8 elements of a step's half kk
// (rows past M read row 0; their products are thrown away).
BW_HD size_t decode_norm_store_elem(int m, int c, int K) { return (size_t)m * decode_lds_row(K) + 4 * c; }
BW_HD size_t decode_operand_elem(int r, int M, int g, int step, int kk, int K) {
  return (size_t)(r < M ? r : 0) * decode_lds_row(K) + 8 * g + 64 * step + 32 * kk;
}
// Byte offset inside a stage of a wave's ring (16 rows of W, 128 bytes each, chunks permuted as above).
BW_HD int decode_ring_operand_offset(int r, int g, int kk) { return mid_operand_offset(r, g, kk); }
