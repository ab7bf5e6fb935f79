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
// stage.  Plain, residual and SwiGLU epilogues; segments joined left to right in registers (a residual add's chain
// starts at the residual, which is read when the first segment ends).  K a multiple of 64.
#define T256_STAGE (48 * 1024)
#define T256_STAGES 3

template <int EPI>
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(2, 2))) void gemm_bf16_tile256_kernel(
    const bf16_t* __restrict__ x, const bf16_t* __restrict__ w, void* __restrict__ out, int M, int N, int K, int ldx,
    int ldo, int m_tiles, int n_tiles) {
  static_assert(EPI != EPI_QKV_ROPE, "plain, residual and SwiGLU epilogues");
  constexpr bool GLU = EPI == EPI_SWIGLU_BF16;
  constexpr int COLS = GLU ? 128 : 256;
  extern __shared__ __attribute__((aligned(16))) unsigned char t256_lds[];   // [3 stages][x 16 KB | W 32 KB]
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
      (void*)(x + (size_t)m0 * ldx), 0, (int)((((size_t)a_rows - 1) * ldx + K) * 2), 0x00020000);
  const bool up = GLU && wave >= 4;
  const __amdgpu_buffer_rsrc_t rs_b = __builtin_amdgcn_make_buffer_rsrc(
      (void*)(w + ((size_t)(up ? N : 0) + n0) * K), 0, (int)((size_t)b_rows * K * 2), 0x00020000);
  const int b_row0 = GLU ? 32 * (wave & 3) : 32 * wave;
  const int lrow = lane >> 3, lslot = lane & 7;
  int voff_a[2], voff_b[4];
#pragma unroll
  for (int t = 0; t < 4; ++t) {
    const int r16 = (8 * t + lrow) & 15;                    // the row within its block of 16
    const int chunk = lslot ^ (r16 >> 1);
    if (t < 2) voff_a[t] = ((16 * wave + 8 * t + lrow) * ldx + 8 * chunk) * 2;
    voff_b[t] = ((b_row0 + 8 * t + lrow) * K + 8 * chunk) * 2;
  }
  typedef __attribute__((address_space(3))) void* lds_ptr;
  const int steps = K / 64;
  auto issue = [&](int step) {
    unsigned char* dst = t256_lds + (step % T256_STAGES) * T256_STAGE;
    const bool real = step < steps;                                     // scalar; past K: outside the descriptors
#pragma unroll
    for (int t = 0; t < 2; ++t)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_a, (lds_ptr)(dst + (2 * wave + t) * 1024), 16, real ? voff_a[t] : 0x7ffffff0,
                                               step * 128, 0, 0);
#pragma unroll
    for (int t = 0; t < 4; ++t)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_b, (lds_ptr)(dst + 16 * 1024 + (4 * wave + t) * 1024), 16,
                                               real ? voff_b[t] : 0x7ffffff0, step * 128, 0, 0);
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
                        EPI == EPI_ADD_F32 && K > GEMM_SEG, QkvRopeArgs{});
}

template <int EPI>
static int launch_tile256(const bf16_t* x, const bf16_t* w, void* out, int M, int N, int K, int ldx, int ldo, hipStream_t s) {
  constexpr int COLS256 = (EPI == EPI_SWIGLU_BF16) ? 128 : 256;
  const int mt = (M + 127) / 128, nt = (N + COLS256 - 1) / COLS256;
  static bool allowed = false;                   // more than 64 KB of dynamic LDS has to be asked for once
  if (!allowed) {
    (void)hipFuncSetAttribute((const void*)gemm_bf16_tile256_kernel<EPI>, hipFuncAttributeMaxDynamicSharedMemorySize,
                              T256_STAGES * T256_STAGE);
    allowed = true;
  }
  BW_LAUNCH((gemm_bf16_tile256_kernel<EPI>), dim3(mt * nt), dim3(512), T256_STAGES * T256_STAGE, s, x, w, out, M, N, K, ldx,
                     ldo, mt, nt);
  return BW_LAUNCH_CHECK();
}

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

// ------------------------------------------------------------------------------ several phases, one launch

#define CHAIN_MAX_PHASES 6
#define CHAIN_SYNC_WORDS 4096          // 32-bit words the caller brings, zero before the first launch: phase p counts its
#define CHAIN_FLAGS_AT 2048            // workgroups in at word 64 p and raises its flag at word 2048 + 64 p
#define CHAIN_LDS_BYTES (160 * 1024 - 256)

struct ChainPhase {
  int kind, first, gx, waves;          // which kernel's statements, the phase's first block, its workgroups and their waves
  MidCall mid;
  RowsCall rows;
};
struct ChainArgs {
  int n, spin_limit;
  int* sync;
  int* err;
  ChainPhase ph[CHAIN_MAX_PHASES];
};

// Workgroups in block order, phase after phase.  A workgroup runs its phase's statements (waves the phase has no use
// for end at once), then counts itself in: every wave waits until its own device-scope stores are acknowledged, a
// barrier, and the first thread adds one to the phase's counter.  The last one to arrive puts the counter back to
// zero, takes down the flag its own phase waited for (every workgroup of the phase is past that wait) and raises the
// flag the next phase waits for: after the launch every word is zero again.
// (The statements are for the device pass only: they name types that the host pass does not know, and unlike those of
// the other kernels they do not all hang on a template parameter.  CH is true.)
template <bool CH>
__global__ __launch_bounds__(512) void gemm_bf16_chain_kernel(const ChainArgs c) {
#if defined(__HIP_DEVICE_COMPILE__)
  int p = 0;
#pragma unroll
  for (int i = 1; i < CHAIN_MAX_PHASES; ++i)
    if (i < c.n && (int)blockIdx.x >= c.ph[i].first) p = i;
  const ChainPhase& P = c.ph[p];
  if (wave_index() >= P.waves) return;
  const ChainCtx cc{(int)blockIdx.x - P.first, 0, 0, P.gx, 1, 1, P.waves, p > 0 ? c.sync + CHAIN_FLAGS_AT + 64 * (p - 1) : nullptr,
                    c.err, p, c.spin_limit};
  const MidCall& m = P.mid;
  const RowsCall& r = P.rows;
  switch (P.kind) {
    case CK_QKV_NARROW:
      mid_body<EPI_QKV_ROPE, 1, true, true, true, CH>(nullptr, m.w, m.out, m.M, m.N, m.K, 0, m.ldo, m.na, m.rp, MidSplitArgs{}, cc);
      break;
    case CK_QKV_WIDE:
      mid_body<EPI_QKV_ROPE, 1, true, false, true, CH>(nullptr, m.w, m.out, m.M, m.N, m.K, 0, m.ldo, m.na, m.rp, MidSplitArgs{}, cc);
      break;
    case CK_GLU:
      mid_body<EPI_SWIGLU_BF16, 1, true, false, true, CH>(nullptr, m.w, m.out, m.M, m.N, m.K, 0, m.ldo, m.na, m.rp, MidSplitArgs{}, cc);
      break;
    case CK_F32:
      mid_body<EPI_F32, 1, true, false, true, CH>(nullptr, m.w, m.out, m.M, m.N, m.K, 0, m.ldo, m.na, m.rp, MidSplitArgs{}, cc);
      break;
    case CK_BURST_ADD: burst_body<EPI_ADD_F32, CH>(r.x, r.w, r.out, r.M, r.N, r.K, r.ldx, r.ldo, cc); break;
    case CK_STREAM_ADD_8_8: stream_body<EPI_ADD_F32, 8, 8, CH>(r.x, r.w, r.out, r.M, r.N, r.K, r.ldx, r.ldo, r.S, cc); break;
    case CK_STREAM_ADD_8_16: stream_body<EPI_ADD_F32, 8, 16, CH>(r.x, r.w, r.out, r.M, r.N, r.K, r.ldx, r.ldo, r.S, cc); break;
    case CK_STREAM_ADD_16_8: stream_body<EPI_ADD_F32, 16, 8, CH>(r.x, r.w, r.out, r.M, r.N, r.K, r.ldx, r.ldo, r.S, cc); break;
    case CK_STREAM_ADD_16_16: stream_body<EPI_ADD_F32, 16, 16, CH>(r.x, r.w, r.out, r.M, r.N, r.K, r.ldx, r.ldo, r.S, cc); break;
  }
  __builtin_amdgcn_s_waitcnt(vmcnt_only(0));
  __syncthreads();
  if (threadIdx.x == 0) {
    const int blocks = (p + 1 < c.n ? c.ph[p + 1].first : (int)gridDim.x) - P.first;
    int* counter = c.sync + 64 * p;
    if (__hip_atomic_fetch_add(counter, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == blocks - 1) {
      __hip_atomic_store(counter, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      if (p > 0) __hip_atomic_store(c.sync + CHAIN_FLAGS_AT + 64 * (p - 1), 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      if (p + 1 < c.n) __hip_atomic_store(c.sync + CHAIN_FLAGS_AT + 64 * p, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
  }
#endif
}

// (host) The chain that is open in this thread, if any: what bw_chain_begin was given, and the phases that wait.
struct ChainState {
  bool open = false;
  int* sync = nullptr;
  int* err = nullptr;
  int spin_limit = 0;
  int n = 0, blocks = 0, lds = 0;
  hipStream_t stream = nullptr;
  ChainPhase ph[CHAIN_MAX_PHASES];
};
static thread_local ChainState g_chain;

static bool chain_is_open() { return g_chain.open; }

static int chain_flush(hipStream_t s) {
  ChainState& g = g_chain;
  if (g.n == 0) return 0;
  ChainArgs a;
  a.n = g.n;
  a.spin_limit = g.spin_limit;
  a.sync = g.sync;
  a.err = g.err;
  for (int i = 0; i < g.n; ++i) a.ph[i] = g.ph[i];
  for (int i = g.n; i < CHAIN_MAX_PHASES; ++i) a.ph[i] = ChainPhase{};
  static bool allowed = false;                       // more than 64 KB of dynamic LDS has to be asked for once
  if (!allowed) {
    (void)hipFuncSetAttribute((const void*)gemm_bf16_chain_kernel<true>, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    allowed = true;
  }
  const int blocks = g.blocks, lds = g.lds;
  hipStream_t stream = g.stream;
  g.n = g.blocks = g.lds = 0;
  (void)s;                                           // (the phases were asked for on g.stream; a caller on another stream has flushed)
  hipLaunchKernelGGL(gemm_bf16_chain_kernel<true>, dim3(blocks), dim3(512), lds, stream, a);
  return BW_LAUNCH_CHECK();
}

static int chain_append(const ChainPhase& ph, int wgs, int lds_bytes, hipStream_t s) {
  ChainState& g = g_chain;
  if (lds_bytes > CHAIN_LDS_BYTES || wgs <= 0) return -2;
  if (g.n > 0 && (g.stream != s || g.n == CHAIN_MAX_PHASES)) {
    const int rc = chain_flush(g.stream);
    if (rc) return rc;
  }
  g.stream = s;
  g.ph[g.n] = ph;
  g.ph[g.n].first = g.blocks;
  g.ph[g.n].gx = wgs;
  g.blocks += wgs;
  if (lds_bytes > g.lds) g.lds = lds_bytes;
  ++g.n;
  return 0;
}

static int chain_record_mid(int kind, const MidCall& c, int wgs, int lds_bytes, hipStream_t s) {
  ChainPhase ph{};
  ph.kind = kind;
  ph.waves = 8;
  ph.mid = c;
  return chain_append(ph, wgs, lds_bytes, s);
}

static int chain_record_rows(int kind, const RowsCall& c, int wgs, int waves, int lds_bytes, hipStream_t s) {
  if ((size_t)c.M * c.ldo * 4 >= ((size_t)1 << 31)) return -2;
  ChainPhase ph{};
  ph.kind = kind;
  ph.waves = waves;
  ph.rows = c;
  return chain_append(ph, wgs, lds_bytes, s);
}

// From bw_chain_begin to bw_chain_end (in the calling thread) the products of up to 16 rows that can run as phases
// (RMSNorm + product with SwiGLU, with a 32-bit store or with rotation and cache write; residual adds of few columns)
// are not launched when they are asked for but wait, and leave as one launch when anything else is launched through this
// library, at bw_chain_flush or at the end.  sync: CHAIN_SYNC_WORDS 32-bit words, zero before the first chain (every
// launch leaves them zero; after an error word that is not zero the caller clears them).  err: a word that gets a bit
// for every phase one of whose waits gave up after spin_limit looks.  Launches that do not come through this library
// (another library's kernels on the same stream) must not be made while phases wait: they would overtake them.
extern "C" int bw_chain_sync_words() { return CHAIN_SYNC_WORDS; }

extern "C" int bw_chain_begin(void* sync, int sync_words, void* err, int spin_limit) {
  if (g_chain.open || sync == nullptr || err == nullptr || sync_words < CHAIN_SYNC_WORDS || spin_limit < 0) return -2;
  g_chain = ChainState{};
  g_chain.open = true;
  g_chain.sync = (int*)sync;
  g_chain.err = (int*)err;
  g_chain.spin_limit = spin_limit;
  return 0;
}

extern "C" int bw_chain_flush(void* stream) { return g_chain.open ? chain_flush((hipStream_t)stream) : 0; }

// (for the launches of this library's other source files)
int bw_chain_flush_open(void* stream) { return bw_chain_flush(stream); }

extern "C" int bw_chain_end(void* stream) {
  if (!g_chain.open) return -2;
  const int rc = chain_flush((hipStream_t)stream);
  g_chain.open = false;
  return rc;
}

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
enum AddRoute { ADD_WHOLE, ADD_ROW_BLOCKS, ADD_TILE_SPLIT, ADD_BIG_SPLIT, ADD_TILE256 };

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
  const long long split = tile_split <= big_split ? tile_split : big_split;
  // 128 x 256 tiles with all of K, the segments joined in registers: no scratch, no join; a step of theirs takes
  // 1.0 us (1.6 of the 128 x 128 tile's)
  const long long t256 = (long long)((M + 127) / 128) * ((N + 255) / 256);
  const long long whole256 = ((t256 + 255) / 256) * (K / 64) * 8 / 5;
  if (whole256 < whole && whole256 <= split) return ADD_TILE256;
  if (10 * split >= 9 * whole) return ADD_WHOLE;
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
    if constexpr (EPI == EPI_F32 || EPI == EPI_BF16 || EPI == EPI_SWIGLU_BF16) {
      // 128 x 256 tiles where they go round the compute units (the 256 x 256 kernel above took what it takes: one
      // segment of K and enough of its tiles)
      constexpr int COLS256 = (EPI == EPI_SWIGLU_BF16) ? 128 : 256;
      const int mt = (M + 127) / 128, nt = (N + COLS256 - 1) / COLS256;
      // (in rounds of 256 workgroups; a step of these takes 1.0 us where a 128 x 128 tile's takes 0.58)
      const int rounds256 = (mt * nt + 255) / 256, rounds128 = (mt * ((N + COLS256 / 2 - 1) / (COLS256 / 2)) + 255) / 256;
      if (K % 64 == 0 && 7 * rounds256 <= 4 * rounds128) return launch_tile256<EPI>(x, w, out, M, N, K, ldx, ldo, s);
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
  if (route == ADD_TILE_SPLIT || route == ADD_BIG_SPLIT) {      // a prompt portion: the segments' sums, whole
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
