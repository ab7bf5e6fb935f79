// bfloat16 matrix product on the matrix cores: y[m][n] = sum_k x[m][k] * W[n][k],
// x bfloat16 [M][K], W bfloat16 row-major [N][K], 32-bit accumulation.
//
// Arithmetic, the same for every M (one row or thousands): K is cut into segments of 2048
// (a property of the weight, never of the batch).  Within a segment each 16x16 block of
// outputs is one accumulator that runs v_mfma_f32_16x16x32_bf16 over k ascending in steps
// of 32 from zero; within an instruction lane group g holds k = kk+8g..kk+8g+7.  Segment
// results are added in 32-bit left to right: y = ((p0 + p1) + p2) + ..., and where the product
// is added into a residual the chain starts there: y = ((res + p0) + p1) + ...  An output's bits
// therefore depend only on its own row of x and row of W (and its own residual).
//
// Several kernels run this arithmetic; which one is a matter of the shape alone (rows, columns, K), never of the
// values, and they agree bit for bit (the tests compare them).  What bounds them all is how many bytes of loads
// a compute unit keeps in flight and fetches through its L1, so each shape gets the kernel that fetches least:
//   * up to 64 rows (decode steps, short prompt portions):
//       - many columns: the "mid" kernel, a workgroup per 64 columns (32 of SwiGLU, or 32 where there are few
//         columns and more than 16 rows), the rows of x shared by its four strips; optionally RMSNorm of up to 16
//         rows fused in front (the rows normalised into LDS by the workgroup) and rotation + cache write behind
//         (a head a workgroup, or with fewer than 256 heads 16 rotary pairs of one);
//         a residual add of 17 to 64 rows over several segments gives every segment workgroups of its own, which
//         meet in device scratch and are added in segment order by the last to arrive;
//       - up to 16 rows and few columns, or several segments: the "stream" kernel, a wave per strip and segment;
//       - both stream weights and x through rings in LDS filled by buffer loads with LDS as their destination,
//         8 rows of 128 bytes an instruction (whole cache lines; half lines cost nearly as much as whole ones),
//         no registers in between, so the rings are deep; the 16-byte chunks of a row are permuted so that operand
//         reads hit distinct banks; a wave waits for "all but the loads of the stages after this one", which
//         works because loads complete in the order they are issued and nothing else is loaded meanwhile;
//       - anything else (K no multiple of 64, SwiGLU with few columns): the "skinny" kernel, a wave per strip
//         and segment streaming through a ring of registers;
//   * more rows (prompt portions): 128 x 128 x 64 tiles, eight waves, fed through a four-stage LDS ring by the
//     same kind of loads ("tile128"; several segments are joined in registers, or for the residual add added
//     into the output as they end), and for products with at least 128 tiles of 256 x 256 the "big" kernel,
//     which computes twice as much per byte it fetches (a ring of five 32 KB slots, operand reads pipelined
//     under the matrix instructions; one segment, or for a residual add with scratch a workgroup per tile and
//     segment, the segments' sums joined in order by a second kernel); 128 x 256 tiles ("tile256": eight waves of
//     64 x 64, room in the registers for the sums of the segments before) where they make fewer rounds of the compute
//     units than the 128 x 128 ones by enough, which is where K has several segments and the big kernel does not
//     run; the "wide" kernel (128 x 128 tiles staged through registers by four waves) takes what those do not: K no
//     multiple of 64.
//
// Epilogues: store 32-bit, store bfloat16, add into a 32-bit residual (each output owned
// by one lane: no atomics), SwiGLU of two products (gate rows n, up rows N+n of a
// stacked weight) stored as bfloat16: h = g * (1/(1+exp(-g))) * u in 32-bit, or rotary encoding of the
// stacked q|k|v product and the write of k and v to their page slots (heads of 64; up to 64 rows: head sizes
// in multiples of 64).
#include <mutex>

#include "common.h"
#include "api.h"
#include "layout.h"        // the epilogues' numbers, GEMM_SEG, MidShape and the LDS layout of the rows normalised in the kernel

// What the rotary epilogue of the stacked q|k|v product needs: the statements of
// rope_kvwrite_bf16_kernel on the 32-bit products while they are still in registers.
struct QkvRopeArgs {
  const int32_t* positions;    // [rows]; negative = padding row
  const int32_t* row_seq;      // [rows] -> row of the block table
  const int32_t* block_table;
  const float* cos_table;      // [max_pos, 32]
  const float* sin_table;
  bf16_t* k_cache;
  bf16_t* v_cache;
  int heads, kv_heads, page_size, table_stride, write_cache;
  int page_shift;              // page_size is a power of two: positions are split by shift and mask, not by division
  int head_dim = 64;           // (the kernels for up to 64 rows take multiples of 64; the tiled ones 64)
};

// ------------------------------------------------------------------------------ phases of one launch
//
// A decode step is a row of small kernels, each of which has to wait for the one before it, and the end of one
// kernel and the start of the next cost as much as many of them take to stream their weights.  The kernels for up
// to 16 rows can therefore also run as phases of ONE launch: the workgroups of phase 0 come first in block order, then
// those of phase 1, and so on.  Workgroups are handed to the compute units in block order, so when a workgroup runs
// every workgroup of the phases before it is running or done; it asks for its weights at once (they depend on
// nothing), then waits until the phase before it has counted all of its workgroups in (a flag that the last of them
// sets; the wait is bounded: a wave that gives up sets a bit of an error word and goes on, nothing hangs), and only
// then reads what that phase wrote.  What one phase writes and a later one reads travels with stores and loads
// of device scope: the dies' L2s are not coherent with each other, a plain load could hit a stale line.  The
// arithmetic of a phase is the statements of its kernel: the same bits.
struct ChainCtx {
  int bx, by, bz, gx, gy, gz;      // the workgroup's place in its phase's grid, and that grid
  int waves;                       // waves of a workgroup of this phase
  const int* wait_flag;            // null: this phase waits for nothing
  int* err;                        // a word that gets bit err_bit when a wait gives up
  int err_bit, spin_limit;
};

__device__ __forceinline__ ChainCtx launch_ctx() {
  return ChainCtx{(int)blockIdx.x, (int)blockIdx.y, (int)blockIdx.z, (int)gridDim.x, (int)gridDim.y, (int)gridDim.z,
                  (int)(blockDim.x >> 6), nullptr, nullptr, 0, 0};
}

// The workgroup waits for the phase before its own (every wave of the workgroup calls this).
template <bool CH>
__device__ __forceinline__ void chain_wait(const ChainCtx& cc) {
  if constexpr (CH) {
    if (cc.wait_flag == nullptr) return;
    if (threadIdx.x == 0) {
      int spins = 0;
      while (__hip_atomic_load(cc.wait_flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == 0) {
        if (++spins > cc.spin_limit) {
          atomicOr(cc.err, 1 << cc.err_bit);
          break;
        }
        __builtin_amdgcn_s_sleep(1);
      }
    }
    __syncthreads();
    asm volatile("" ::: "memory");
  }
}

// Loads and stores of what another phase of the same launch wrote or will read (DEV), else plain ones.
template <bool DEV>
__device__ __forceinline__ float ld_f32(const float* p) {
  if constexpr (DEV) return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  else return *p;
}
template <bool DEV>
__device__ __forceinline__ void st_f32(float* p, float v) {
  if constexpr (DEV) __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  else *p = v;
}
template <bool DEV>
__device__ __forceinline__ void st_bf16(bf16_t* p, bf16_t v) {
  if constexpr (DEV) __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  else *p = v;
}

template <int EPI, bool DEV = false>
__device__ __forceinline__ void epilogue_store(void* __restrict__ out, size_t o, float v, float u) {
  if constexpr (EPI == EPI_F32) st_f32<DEV>((float*)out + o, v);
  else if constexpr (EPI == EPI_BF16) st_bf16<DEV>((bf16_t*)out + o, f32_to_bf16(v));
  else if constexpr (EPI == EPI_ADD_F32) st_f32<DEV>((float*)out + o, ld_f32<DEV>((const float*)out + o) + v);
  else if constexpr (EPI == EPI_SWIGLU_BF16) st_bf16<DEV>((bf16_t*)out + o, f32_to_bf16(silu_times(v, u)));
}

// (host) The phases asked for while a chain is open wait in a list and leave as one launch (further down).
struct MidCall;
struct RowsCall;
static bool chain_is_open();
static int chain_flush(hipStream_t s);
static int chain_record_mid(int kind, const MidCall& c, int wgs, int lds_bytes, hipStream_t s);
static int chain_record_rows(int kind, const RowsCall& c, int wgs, int waves, int lds_bytes, hipStream_t s);

// Every other launch of this file: what waits in an open chain goes first.
#define BW_LAUNCH(kernel, grid, block, lds, stream, ...)                \
  do {                                                                  \
    if (chain_is_open()) (void)chain_flush(stream);                     \
    hipLaunchKernelGGL(kernel, grid, block, lds, stream, __VA_ARGS__);  \
  } while (0)

#include "gemm_bf16_skinny.h"
#include "gemm_bf16_tiles.h"
#include "gemm_bf16_rows.h"
#include "gemm_bf16_phases.h"

// ------------------------------------------------------------------------------ launch

// How a residual add of 17 to 64 rows runs in the kernel above: 64 or 32 columns a workgroup (as many workgroups
// as there are compute units, if the product has them), a workgroup per tile and segment of K if there are several
// (they meet in device scratch the caller brings).  tiles 0: it does not run there.
// out = (((out + p[0]) + p[1]) + ...) + p[S-1], element by element: the segments of a residual add that
// gemm_bf16_big_kernel left in scratch ([S][M][N]), joined in segment order.
__global__ __launch_bounds__(256) void add_segments_kernel(float* __restrict__ out, const float* __restrict__ parts, int S,
                                                           int M, int N, int ldo) {
  const size_t quads = (size_t)M * (N >> 2);
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= quads) return;
  const int m = (int)(i / (N >> 2)), n = 4 * (int)(i % (N >> 2));
  float* o = out + (size_t)m * ldo + n;
  f32x4 y = *reinterpret_cast<const f32x4*>(o);
  for (int sg = 0; sg < S; ++sg) y = y + *reinterpret_cast<const f32x4*>(parts + ((size_t)sg * M + m) * N + n);
  *reinterpret_cast<f32x4*>(o) = y;
}

static void add_rows_shape(int M, int N, int K, int& tiles, bool& narrow) {
  const int S = (K + GEMM_SEG - 1) / GEMM_SEG;
  tiles = 0;
  narrow = false;
  if (M <= 16 || M > 64 || K % 64) return;
  narrow = ((N + 63) / 64) * S < 256;
  tiles = narrow ? (N + 31) / 32 : (N + 63) / 64;
  if (tiles * S < 32) tiles = 0;
}

// How a residual add of more than 64 rows is laid out.  One workgroup of the tile kernels fits a compute unit, so
// a product goes in rounds of 256 workgroups, and a workgroup that has all of K to itself takes K / 64 steps
// whatever else is idle: an output of 2048 columns and 128 rows is 16 tiles (76 us for K = 8192).
//   whole       128 x 128 tiles with all of K, each finished segment added into the output: needs no scratch.
//   row blocks  the kernel for up to 64 rows once per block of 64 rows, with its workgroup per 32 or 64 columns and
//               segment of K (its scratch if K has several segments): up to 128 rows and three segments, where a
//               launch more costs less than the join below (K = 2048: 16 and 19 us at 65 and 128 rows, for 24).
//   tile split  a 128 x 128 workgroup per tile and segment, the segments' sums whole in scratch and joined in order
//               afterwards (128 rows of K = 8192: 25 us).
//   big split   the same with 256 x 256 tiles, which fetch half as many bytes a flop: for 512 rows or more.
//   tile256     128 x 256 tiles with all of K, the segments joined in registers: needs no scratch.
//   blocks at once  one segment of K only: the kernel for up to 64 rows with all blocks of 64 rows in one launch (its
//               grid's third dimension), while the workgroups fit the chip at once (512): the output projection of
//               2048 columns takes 8.4 us at 128 rows and 13.3 at 512, where 128 x 128 tiles took 16.4 and 21.6.  The
//               q|k|v product with rotation and cache write goes the same way (launch_qkv_rope_mid).
// All five give the same bits.  The choice is by a count of steps: rounds times the steps of a workgroup (a step of
// a 256 x 256 tile counts twice); the join moves 8 bytes an element and segment (about 500,000 elements in the
// time of a step) and is a launch more (8 steps); a split has to win by a tenth.  tiles64: what the 64-row
// kernel's scratch is sized by.
enum AddRoute { ADD_WHOLE, ADD_ROW_BLOCKS, ADD_TILE_SPLIT, ADD_BIG_SPLIT, ADD_TILE256, ADD_TILE256_SPLIT };

// "Blocks at once" for a residual add of more than 64 rows: how many blocks of 64 rows, tiles of 64 or (narrow) 32
// columns; tiles 0: it does not run that way (more than 512 workgroups, or too few to matter).  Several segments of K
// meet in scratch: 4096 floats a workgroup, a counter a (block, tile).
#define ADD_BLOCKS_MAX_WGS 512
static void add_blocks_shape(int M, int N, int K, int& tiles, bool& narrow, int& zb) {
  const int S = (K + GEMM_SEG - 1) / GEMM_SEG;
  tiles = 0;
  narrow = false;
  zb = (M + 63) / 64;
  if (M <= 64 || K % 64 || N <= 0) return;
  const int wide = (N + 63) / 64;
  narrow = wide * zb * S < 192;
  const int t = narrow ? (N + 31) / 32 : wide;
  if (t * zb * S >= 32 && t * zb * S <= ADD_BLOCKS_MAX_WGS) tiles = t;
}

static AddRoute add_route(int M, int N, int K, int ldo, int& tiles64) {
  const int S = (K + GEMM_SEG - 1) / GEMM_SEG;
  tiles64 = 0;
  if (M <= 64 || K % 64) return ADD_WHOLE;
  bool narrow;
  add_rows_shape(64, N, K, tiles64, narrow);
  if (tiles64 && M <= 128 && S <= 3) return ADD_ROW_BLOCKS;
  tiles64 = 0;
  if (S < 2 || N % 4 || ldo % 4) return ADD_WHOLE;
  const long long t128 = (long long)((M + 127) / 128) * ((N + 127) / 128);
  const long long tbig = (long long)((M + BIG_BM - 1) / BIG_BM) * ((N + 255) / 256);
  const long long join = (long long)S * M * N / 500000 + 8;
  const long long whole = ((t128 + 255) / 256) * (K / 64);
  const long long tile_split = ((t128 * S + 255) / 256) * (GEMM_SEG / 64) + join;
  const long long big_split = M >= 2 * BIG_BM ? ((tbig * S + 255) / 256) * 2 * (GEMM_SEG / 64) + join : whole;
  // 128 x 256 tiles: a step of theirs takes 1.0 us (1.6 to 1.75 of the 128 x 128 tile's).  With all of K, the
  // segments joined in registers: no scratch, no join.  A workgroup per tile and segment: where that is one round of
  // the chip and 128 x 128 tiles would be two (1,024 rows of K = 8192 into 2048 columns).
  const long long t256 = (long long)((M + 127) / 128) * ((N + 255) / 256);
  const long long whole256 = ((t256 + 255) / 256) * (K / 64) * 8 / 5;
  const long long t256_split = ((t256 * S + 255) / 256) * (GEMM_SEG / 64) * 7 / 4 + join;
  const long long split3 = tile_split <= big_split ? tile_split : big_split;
  const long long split = t256_split < split3 ? t256_split : split3;
  if (whole256 < whole && whole256 <= split) return ADD_TILE256;
  if (10 * split >= 9 * whole) return ADD_WHOLE;
  if (t256_split < split3) return ADD_TILE256_SPLIT;
  return tile_split <= big_split ? ADD_TILE_SPLIT : ADD_BIG_SPLIT;
}

template <int EPI>
static int launch_gemm_bf16(const bf16_t* x, const bf16_t* w, void* out, int M, int N, int K, int ldx, int ldo,
                            hipStream_t s, const QkvRopeArgs& rp = QkvRopeArgs{}, const MidSplitArgs& sp = MidSplitArgs{},
                            size_t scratch_floats = 0, int num_counters = 0) {
  const int S = (K + GEMM_SEG - 1) / GEMM_SEG;
  constexpr int NB = (EPI == EPI_SWIGLU_BF16) ? 2 : 1;
  if (M <= 64) {
    if constexpr (EPI == EPI_QKV_ROPE) return -2;       // the rotary epilogue belongs to the wide kernel
    else {
      // one segment and enough columns: the rows of x are shared through LDS
      constexpr int MID_COLS = (EPI == EPI_SWIGLU_BF16) ? 32 : 64;
      const int wgs = (N + MID_COLS - 1) / MID_COLS;
      // (the descriptors of W cover a tile's rows each, so only the rows of x have to fit 31 bits of offset)
      const bool fits = (size_t)M * ldx * 2 < ((size_t)1 << 31);
      // (a residual add of several segments starts its chain at the residual: the kernels further down do that)
      if ((S == 1 || EPI != EPI_ADD_F32) && K % 64 == 0 && wgs >= 64 && fits) {
        if (M <= 16) return launch_mid<EPI, 1, false>(x, w, out, M, N, K, ldx, ldo, wgs, s);
        if (M <= 32) return launch_mid<EPI, 2, false>(x, w, out, M, N, K, ldx, ldo, wgs, s);
        // 33 to 64 rows and so few columns that twice the workgroups still fit the chip at once: two blocks of 32 rows,
        // 32 columns a workgroup, which then pulls half the rows of x and half the weights (4096 columns of K = 2048
        // at 64 rows: 9.5 us against 14.1; 2048 columns, further down: 8.4 against 10.7)
        if constexpr (EPI == EPI_ADD_F32 || EPI == EPI_F32 || EPI == EPI_BF16) {
          if (2 * ((N + 31) / 32) <= 256)
            return launch_mid<EPI, 2, false, true>(x, w, out, M, N, K, ldx, ldo, (N + 31) / 32, s, MidNormArgs{}, QkvRopeArgs{}, 1,
                                                   MidSplitArgs{}, 2);
        }
        return launch_mid<EPI, 4, false>(x, w, out, M, N, K, ldx, ldo, wgs, s);
      }
      // a residual add of more than 16 rows and fewer columns (the other kernel for it fetches W once per block of
      // 16 rows): narrower tiles, and several segments if the caller brought scratch for them to meet in
      if constexpr (EPI == EPI_ADD_F32) {
        int tiles;
        bool narrow;
        add_rows_shape(M, N, K, tiles, narrow);
        if (tiles && fits && (S == 1 || (sp.scratch != nullptr && sp.counters != nullptr))) {
          if (S > 1 && (scratch_floats < (size_t)tiles * S * 4096 || num_counters < tiles)) return -6;
          const MidNormArgs na{};
          const QkvRopeArgs no{};
          if (narrow) {
            if (M <= 32) return launch_mid<EPI, 2, false, true>(x, w, out, M, N, K, ldx, ldo, tiles, s, na, no, S, sp);
            // one segment and so few tiles that twice as many still fit the chip at once: two blocks of 32 rows, each
            // workgroup then pulls half the rows of x beside its weights
            if (S == 1 && 2 * tiles <= 256)
              return launch_mid<EPI, 2, false, true>(x, w, out, M, N, K, ldx, ldo, tiles, s, na, no, S, sp, 2);
            return launch_mid<EPI, 4, false, true>(x, w, out, M, N, K, ldx, ldo, tiles, s, na, no, S, sp);
          }
          if (M <= 32) return launch_mid<EPI, 2, false>(x, w, out, M, N, K, ldx, ldo, tiles, s, na, no, S, sp);
          return launch_mid<EPI, 4, false>(x, w, out, M, N, K, ldx, ldo, tiles, s, na, no, S, sp);
        }
      }
    }
    if constexpr (EPI != EPI_SWIGLU_BF16 && EPI != EPI_QKV_ROPE) {
      // up to 16 rows: a wave per strip and segment, streaming through its own ring in LDS
      if (M <= 16 && K % 64 == 0 && S <= 40 && (size_t)M * ldx * 2 < ((size_t)1 << 31)) {
        // one segment and few columns: everything asked for at once
        if ((N + 15) / 16 < 256 && K <= 64 * BURST_STEPS) return launch_burst<EPI>(x, w, out, M, N, K, ldx, ldo, s);
        // (two segments and 256 strips, the 8B shape's output projection: half strips, 512 workgroups of two waves of which
        // two share a compute unit, were slower: 10.7 us against 9.6)
        if ((N + 15) / 16 < 256) return launch_stream<EPI, 8>(x, w, out, M, N, K, ldx, ldo, S, s);
        return launch_stream<EPI, 16>(x, w, out, M, N, K, ldx, ldo, S, s);
      }
    }
    const int row_blocks = (M + 15) / 16, strips = (N + 15) / 16;
    // Few columns and more than 16 rows: a workgroup per block of 16 rows (the strips of W are then
    // fetched once per block of rows, from cache after the first, by four times the waves).  Many
    // columns: one wave takes all rows of its strip.
    const bool split_rows = row_blocks > 1 && strips < 256;
    const int wm = split_rows ? 1 : row_blocks;
    const int waves = S < 4 ? S : 4;      // one wave per SIMD: the operand ring may use up to 512 registers
    // few columns: half strips, so that there are at least as many workgroups as compute units
    const bool half = strips < 256 && row_blocks == 1;
    dim3 grid(half ? (N + 7) / 8 : strips, split_rows ? row_blocks : 1), block(64 * waves);
    const size_t lds = S > 1 ? (size_t)S * NB * wm * 4 * 64 * sizeof(float) : 0;
    if (lds > 64 * 1024) return -2;
    if ((size_t)M * ldx * 2 >= ((size_t)1 << 31) || (size_t)16 * K * 2 >= ((size_t)1 << 31)) return -2;   // offsets within x, within a strip of W
#define BW_SKINNY(WMV, DV, CWV)                                                                                    \
  if (K % 32)                                                                                                      \
    BW_LAUNCH((gemm_bf16_skinny_kernel<WMV, EPI, DV, true, CWV>), grid, block, lds, s, x, w, out, M, N, K, ldx, ldo, S); \
  else                                                                                                             \
    BW_LAUNCH((gemm_bf16_skinny_kernel<WMV, EPI, DV, false, CWV>), grid, block, lds, s, x, w, out, M, N, K, ldx, ldo, S);
    switch (wm) {
      case 1:
        if (half) { BW_SKINNY(1, 16, 8) }
        else { BW_SKINNY(1, 16, 16) }
        break;
      case 2: BW_SKINNY(2, (NB == 2 ? 8 : 16), 16) break;
      case 3: BW_SKINNY(3, 8, 16) break;
      default: BW_SKINNY(4, 8, 16) break;
    }
#undef BW_SKINNY
  } else {
    if constexpr (EPI == EPI_ADD_F32) {
      // Few enough workgroups to be on the chip at once (the output projection of a short prompt is 16 tiles of 128 x 128
      // for 128 rows and 2048 columns, whatever is idle): the kernel for up to 64 rows, a workgroup per block of 64 rows,
      // 64 or 32 columns and segment of K, all blocks in one launch.
      if ((size_t)M * ldx * 2 < ((size_t)1 << 31)) {
        // (one segment, and blocks of 32 rows by 32 columns still fit the chip at once: as for 33 to 64 rows above)
        if (S == 1 && K % 64 == 0 && ((N + 31) / 32) * ((M + 31) / 32) <= 256 && ((N + 31) / 32) * ((M + 31) / 32) >= 32)
          return launch_mid<EPI, 2, false, true>(x, w, out, M, N, K, ldx, ldo, (N + 31) / 32, s, MidNormArgs{}, QkvRopeArgs{}, 1,
                                                 MidSplitArgs{}, (M + 31) / 32);
        int tiles, zb;
        bool narrow;
        add_blocks_shape(M, N, K, tiles, narrow, zb);
        const bool scratch_ok = S == 1 || (sp.scratch != nullptr && sp.counters != nullptr &&
                                           scratch_floats >= (size_t)tiles * zb * S * 4096 && num_counters >= tiles * zb);
        if (tiles && scratch_ok) {
          const MidNormArgs na{};
          const QkvRopeArgs no{};
          if (narrow) return launch_mid<EPI, 4, false, true>(x, w, out, M, N, K, ldx, ldo, tiles, s, na, no, S, sp, zb);
          return launch_mid<EPI, 4, false>(x, w, out, M, N, K, ldx, ldo, tiles, s, na, no, S, sp, zb);
        }
      }
      int tiles;
      const AddRoute route = add_route(M, N, K, ldo, tiles);
      if (route == ADD_ROW_BLOCKS && (size_t)M * ldx * 2 < ((size_t)1 << 31) &&
          (S == 1 || (sp.scratch != nullptr && sp.counters != nullptr && scratch_floats >= (size_t)tiles * S * 4096 &&
                      num_counters >= tiles))) {
        for (int m0 = 0; m0 < M; m0 += 64) {
          const int rc = launch_gemm_bf16<EPI>(x + (size_t)m0 * ldx, w, (float*)out + (size_t)m0 * ldo, M - m0 < 64 ? M - m0 : 64, N, K,
                                               ldx, ldo, s, rp, sp, scratch_floats, num_counters);
          if (rc) return rc;
        }
        return 0;
      }
      if (route == ADD_TILE256) return launch_tile256<EPI>(x, w, out, M, N, K, ldx, ldo, s);
      if (route == ADD_BIG_SPLIT && sp.scratch != nullptr && ((uintptr_t)out & 15) == 0) {
        if (scratch_floats < (size_t)S * M * N) return -6;
        const int bm = (M + BIG_BM - 1) / BIG_BM, bn = (N + 255) / 256;
        static bool allowed = false;                 // more than 64 KB of dynamic LDS has to be asked for once
        if (!allowed) {
          (void)hipFuncSetAttribute((const void*)gemm_bf16_big_kernel<EPI_F32>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                    BIG_SLOTS * BIG_SLOT);
          allowed = true;
        }
        BW_LAUNCH((gemm_bf16_big_kernel<EPI_F32>), dim3(bm * bn, S), dim3(512), BIG_SLOTS * BIG_SLOT, s, x, w,
                           (void*)sp.scratch, M, N, K, ldx, N, bm, bn, rp, (size_t)M * N);
        const size_t quads = (size_t)M * (N >> 2);
        BW_LAUNCH(add_segments_kernel, dim3((unsigned)((quads + 255) / 256)), dim3(256), 0, s, (float*)out, sp.scratch, S,
                           M, N, ldo);
        return BW_LAUNCH_CHECK();
      }
      if (route == ADD_TILE256_SPLIT && sp.scratch != nullptr && ((uintptr_t)out & 15) == 0) {
        if (scratch_floats < (size_t)S * M * N) return -6;
        const int rc = launch_tile256<EPI_F32>(x, w, (void*)sp.scratch, M, N, K, ldx, N, s, QkvRopeArgs{}, S, (size_t)M * N);
        if (rc) return rc;
        const size_t quads = (size_t)M * (N >> 2);
        BW_LAUNCH(add_segments_kernel, dim3((unsigned)((quads + 255) / 256)), dim3(256), 0, s, (float*)out, sp.scratch, S,
                           M, N, ldo);
        return BW_LAUNCH_CHECK();
      }
      if (route == ADD_TILE_SPLIT && sp.scratch != nullptr && ((uintptr_t)out & 15) == 0) {
        if (scratch_floats < (size_t)S * M * N) return -6;
        const int mt = (M + 127) / 128, nt = (N + 127) / 128;
        static bool allowed = false;
        if (!allowed) {
          (void)hipFuncSetAttribute((const void*)gemm_bf16_tile128_kernel<EPI_F32>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                    T128_STAGES * T128_STAGE);
          allowed = true;
        }
        BW_LAUNCH((gemm_bf16_tile128_kernel<EPI_F32>), dim3(mt * nt, S), dim3(512), T128_STAGES * T128_STAGE, s, x, w,
                           (void*)sp.scratch, M, N, K, ldx, N, mt, nt, rp, (size_t)M * N);
        const size_t quads = (size_t)M * (N >> 2);
        BW_LAUNCH(add_segments_kernel, dim3((unsigned)((quads + 255) / 256)), dim3(256), 0, s, (float*)out, sp.scratch, S,
                           M, N, ldo);
        return BW_LAUNCH_CHECK();
      }
    }
    if constexpr (EPI == EPI_F32 || EPI == EPI_BF16) {
      // few enough workgroups of the 64-row kernel to be on the chip at once: all blocks of 64 rows in one launch (a
      // product of 6144 columns at 128 rows 13 us against 20 on 128 x 128 tiles; the SwiGLU product gains nothing)
      const int wgs = (N + 63) / 64, zb = (M + 63) / 64;
      if (K % 64 == 0 && wgs >= 64 && wgs * zb <= ADD_BLOCKS_MAX_WGS && (size_t)M * ldx * 2 < ((size_t)1 << 31))
        return launch_mid<EPI, 4, false>(x, w, out, M, N, K, ldx, ldo, wgs, s, MidNormArgs{}, QkvRopeArgs{}, 1, MidSplitArgs{}, zb);
    }
    if constexpr (EPI != EPI_ADD_F32) {
      // enough 256-row tiles to go round the compute units (a second round at least half full)
      constexpr int BIG_COLS = (EPI == EPI_SWIGLU_BF16) ? 128 : 256;
      const int bm = (M + BIG_BM - 1) / BIG_BM, bn = (N + BIG_COLS - 1) / BIG_COLS;
      // (fewer of these tiles than compute units while the 128-row tiles below would fill the chip in one round: a step
      // of those takes half as long, so they win: gate|up of 512 rows 62 us here, half the chip idle)
      bool half_tiles_win = false;
      if constexpr (EPI == EPI_F32 || EPI == EPI_BF16 || EPI == EPI_SWIGLU_BF16) {
        const int t256 = ((M + 127) / 128) * bn;
        half_tiles_win = (t256 + 255) / 256 < 2 * ((bm * bn + 255) / 256);
      }
      if (S == 1 && K % 64 == 0 && M >= 2 * BIG_BM && bm * bn >= 128 && !half_tiles_win) {
        static bool allowed = false;                 // more than 64 KB of dynamic LDS has to be asked for once
        if (!allowed) {
          (void)hipFuncSetAttribute((const void*)gemm_bf16_big_kernel<EPI>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                    BIG_SLOTS * BIG_SLOT);
          allowed = true;
        }
        BW_LAUNCH((gemm_bf16_big_kernel<EPI>), dim3(bm * bn), dim3(512), BIG_SLOTS * BIG_SLOT, s, x, w, out, M, N, K, ldx,
                           ldo, bm, bn, rp, (size_t)0);
        return BW_LAUNCH_CHECK();
      }
    }
    if constexpr (EPI == EPI_F32 || EPI == EPI_BF16 || EPI == EPI_SWIGLU_BF16 || EPI == EPI_QKV_ROPE) {
      // 128 x 256 tiles where they go round the compute units (the 256 x 256 kernel above took what it takes: one
      // segment of K and enough of its tiles); the q|k|v product of 600 to 1,200 rows among them (four heads of 64 a
      // tile, a head a wave as in the 128 x 128 tiles: 1,024 rows 45.8 us there)
      constexpr int COLS256 = (EPI == EPI_SWIGLU_BF16) ? 128 : 256;
      const int mt = (M + 127) / 128, nt = (N + COLS256 - 1) / COLS256;
      // (in rounds of 256 workgroups; a step of these takes 1.0 us where a 128 x 128 tile's takes 0.58)
      const int rounds256 = (mt * nt + 255) / 256, rounds128 = (mt * ((N + COLS256 / 2 - 1) / (COLS256 / 2)) + 255) / 256;
      if (K % 64 == 0 && 7 * rounds256 <= 4 * rounds128) return launch_tile256<EPI>(x, w, out, M, N, K, ldx, ldo, s, rp);
    }
    constexpr int COLS = (EPI == EPI_SWIGLU_BF16) ? 64 : 128;
    const int m_tiles = (M + WIDE_BM - 1) / WIDE_BM, n_tiles = (N + COLS - 1) / COLS;
    dim3 grid(m_tiles * n_tiles), block(256);
    {
      // K in whole steps of 64: the tiles go straight into an LDS ring
      if (K % 64 == 0) {
        static bool allowed = false;                   // more than 64 KB of dynamic LDS has to be asked for once
        if (!allowed) {
          (void)hipFuncSetAttribute((const void*)gemm_bf16_tile128_kernel<EPI>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                    T128_STAGES * T128_STAGE);
          allowed = true;
        }
        BW_LAUNCH((gemm_bf16_tile128_kernel<EPI>), grid, dim3(512), T128_STAGES * T128_STAGE, s, x, w, out, M, N, K, ldx,
                           ldo, m_tiles, n_tiles, rp, (size_t)0);
        return BW_LAUNCH_CHECK();
      }
    }
    if (S > 1)
      BW_LAUNCH((gemm_bf16_wide_kernel<EPI, true, false>), grid, block, 0, s, x, w, out, M, N, K, ldx, ldo, m_tiles, n_tiles, rp);
    else if (K % (2 * WIDE_BK) == 0)
      BW_LAUNCH((gemm_bf16_wide_kernel<EPI, false, true>), grid, block, 0, s, x, w, out, M, N, K, ldx, ldo, m_tiles, n_tiles, rp);
    else
      BW_LAUNCH((gemm_bf16_wide_kernel<EPI, false, false>), grid, block, 0, s, x, w, out, M, N, K, ldx, ldo, m_tiles, n_tiles, rp);
  }
  return BW_LAUNCH_CHECK();
}

// What a residual add wants beside its operands to give every segment of K workgroups of its own: floats of
// scratch and counters (int32, zero before the first launch; every launch leaves them zero).  Both 0: it would not.
extern "C" int bw_gemm_add_scratch(int M, int N, int K, long long* scratch_floats, int* counters) {
  int tiles = 0;
  bool narrow = false;
  const int S = K > 0 ? (K + GEMM_SEG - 1) / GEMM_SEG : 0;
  if (M > 64 && N > 0 && S > 1) {                           // a few blocks of 64 rows at once: a cell a workgroup
    int zb;
    add_blocks_shape(M, N, K, tiles, narrow, zb);
    if (tiles) {
      *scratch_floats = (long long)ADD_BLOCKS_MAX_WGS * 4096;   // (the same for every shape: one buffer serves all)
      *counters = ADD_BLOCKS_MAX_WGS;
      return 0;
    }
  }
  const AddRoute route = M > 64 && N > 0 ? add_route(M, N, K, 4, tiles) : ADD_WHOLE;
  if (route == ADD_TILE_SPLIT || route == ADD_BIG_SPLIT || route == ADD_TILE256_SPLIT) {      // a prompt portion: the segments' sums, whole
    *scratch_floats = (long long)S * M * N;
    *counters = 1;                                          // (none is used)
    return 0;
  }
  if (M > 0 && M <= 64 && N > 0 && S > 1) add_rows_shape(M, N, K, tiles, narrow);
  else if (S == 1) tiles = 0;                               // (blocks of 64 rows of one segment share nothing)
  *scratch_floats = (long long)tiles * S * 4096;
  *counters = tiles;
  return 0;
}

// out += x W^T with the scratch that bw_gemm_add_scratch asks for: the bits of bw_gemm_bf16's residual add.
extern "C" int bw_gemm_add_bf16(const void* x, const void* w, void* out, int M, int N, int K, int ldx, int ldo,
                                float* scratch, long long scratch_floats, int32_t* counters, int num_counters,
                                void* stream) {
  if (M <= 0 || N <= 0) return 0;
  if (K <= 0 || (K % 8) || (ldx % 8) || ldx < K || ldo < N) return -2;
  if ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(w)) & 15) return -3;
  return launch_gemm_bf16<EPI_ADD_F32>((const bf16_t*)x, (const bf16_t*)w, out, M, N, K, ldx, ldo, (hipStream_t)stream,
                                       QkvRopeArgs{}, MidSplitArgs{scratch, counters}, (size_t)scratch_floats, num_counters);
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

// The stacked q|k|v product with rotation and cache write in its epilogue (heads of 64 elements, K of one
// segment; more than 64 rows, or up to 64 with at least 64 heads and K in steps of 64): q rotated to q_out [M, heads*64],
// k rotated and v to their page slots.  The bits of gemm_bf16 (32-bit store) + rope_kvwrite.
extern "C" int bw_gemm_qkv_rope_bf16(const void* x, int ldx, const void* w_qkv, void* q_out, const int32_t* positions,
                                     const int32_t* row_seq, const int32_t* block_table, int table_stride,
                                     const float* cos_table, const float* sin_table, void* k_cache, void* v_cache,
                                     int M, int heads, int kv_heads, int head_dim, int K, int page_size,
                                     int write_cache, void* stream) {
  if (M <= 0) return 0;
  if (head_dim % 64) return -4;
  if (K <= 0 || (K % 8) || (ldx % 8) || ldx < K || page_size <= 0) return -2;
  if ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(w_qkv)) & 15) return -3;
  if (page_size <= 0 || (page_size & (page_size - 1))) return -5;
  QkvRopeArgs rp{positions, row_seq, block_table, cos_table, sin_table, (bf16_t*)k_cache, (bf16_t*)v_cache,
                 heads, kv_heads, page_size, table_stride, write_cache, __builtin_ctz((unsigned)page_size), head_dim};
  // up to 64 rows, or a few blocks of 64 rows at once: a workgroup per 32 or 16 rotary pairs of a head
  const int mid = launch_qkv_rope_mid((const bf16_t*)x, ldx, (const bf16_t*)w_qkv, q_out, M, K, rp, (hipStream_t)stream);
  if (mid != -7) return mid;
  if (M <= 64) return -2;
  if (head_dim != 64) return -4;                                   // the tiled kernels' epilogue: heads of 64 ...
  if (K > GEMM_SEG) return -2;                                     // ... and one segment of K
  const int N = (heads + 2 * kv_heads) * 64;
  return launch_gemm_bf16<EPI_QKV_ROPE>((const bf16_t*)x, (const bf16_t*)w_qkv, q_out, M, N, K, ldx, heads * 64,
                                        (hipStream_t)stream, rp);
}

// ------------------------------------------------------------------------------ a residual add that allocates nothing

// out += x W^T like bw_gemm_add_bf16, for callers that can neither allocate device memory nor bring a
// workspace (code under graph capture, tight serving loops, harnesses that forbid hipMalloc): the
// segments' sums and the tiles' counters live in one array in the library's own device image.  Every GPU
// that loads the library holds a copy of the array at an address of its own until the process ends; the
// name of the array is no device address in host code, so the address is asked for once per device and
// kept.  Calls on one GPU share the array: calls that overlap there (two streams, two threads) race.
#define BW_STATIC_SCRATCH_FLOATS (2 * 1024 * 1024)          // 8 MB of sums
#define BW_STATIC_SCRATCH_COUNTERS 1024                      // 4 KB of counters behind them
#define BW_STATIC_MAX_DEVICES 64
static __device__ __align__(256) float scratch[BW_STATIC_SCRATCH_FLOATS + BW_STATIC_SCRATCH_COUNTERS];

__global__ __launch_bounds__(256) void zero_words_kernel(int32_t* __restrict__ p, int n) {
  const int i = (int)(blockIdx.x * 256 + threadIdx.x);
  if (i < n) p[i] = 0;
}

static float* static_scratch_of_device[BW_STATIC_MAX_DEVICES];
static std::mutex static_scratch_mutex;

// The current device's copy of the array (asked for at the first call on that device).
static int static_scratch_address(float** out) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return (int)e;
  if (dev < 0 || dev >= BW_STATIC_MAX_DEVICES) return -2;
  std::lock_guard<std::mutex> hold(static_scratch_mutex);
  if (static_scratch_of_device[dev] == nullptr) {
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess) return (int)e;
    if (p == nullptr) return -2;
    static_scratch_of_device[dev] = (float*)p;
  }
  *out = static_scratch_of_device[dev];
  return 0;
}

extern "C" int bw_gemm_add_bf16_static_max(long long* scratch_floats, int* counters) {
  *scratch_floats = BW_STATIC_SCRATCH_FLOATS;
  *counters = BW_STATIC_SCRATCH_COUNTERS;
  return 0;
}

extern "C" int bw_gemm_add_bf16_static(const void* x, const void* w, void* out, int M, int N, int K, int ldx, int ldo,
                                       void* stream) {
  if (M <= 0 || N <= 0) return 0;
  if (K <= 0 || (K % 8) || (ldx % 8) || ldx < K || ldo < N) return -2;
  if ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(w)) & 15) return -3;
  long long need_floats = 0;
  int need_counters = 0;
  bw_gemm_add_scratch(M, N, K, &need_floats, &need_counters);
  if (need_floats > BW_STATIC_SCRATCH_FLOATS || need_counters > BW_STATIC_SCRATCH_COUNTERS) return -7;
  if (need_floats == 0)      // this shape's kernel joins its segments in registers: nothing to share
    return launch_gemm_bf16<EPI_ADD_F32>((const bf16_t*)x, (const bf16_t*)w, out, M, N, K, ldx, ldo, (hipStream_t)stream);
  float* base = nullptr;
  const int rc = static_scratch_address(&base);
  if (rc != 0) return rc;
  int32_t* count = reinterpret_cast<int32_t*>(base + BW_STATIC_SCRATCH_FLOATS);
  // The counters must be zero when the kernel starts.  Every launch leaves them so, but the array outlives a
  // launch that was aborted half way; a small kernel clears them (a memset node in a captured graph is no
  // safe thing on this hardware's runtime).  The sums need no clearing: every cell is written before it is read.
  BW_LAUNCH(zero_words_kernel, dim3((need_counters + 255) / 256), dim3(256), 0, (hipStream_t)stream, count,
                     need_counters);
  return launch_gemm_bf16<EPI_ADD_F32>((const bf16_t*)x, (const bf16_t*)w, out, M, N, K, ldx, ldo, (hipStream_t)stream,
                                       QkvRopeArgs{}, MidSplitArgs{base, count}, (size_t)need_floats, need_counters);
}
