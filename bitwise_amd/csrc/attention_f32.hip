// True 32-bit causal attention over the paged cache, in the reference's operation order
// (src/kernels.cpp:312-368): for the query at position p of head h,
//   pass 1: s_j = dot_canonical(q, K_j) * scale for j = lo..p, mx = max s_j;
//   pass 2: for j = lo..p in key order: e = exp(s_j - mx); sum += e; acc[d] = fma(e, V_j[d], acc[d]);
//   out[d] = acc[d] * (1/sum).
// dot_canonical is the 16-chain split with the fixed tree (src/kernels.cpp:57-64, :86-101).
// lo is 0, or p-window+1 for a windowed cache.  A workgroup of 256 threads per (row, head): in pass 1 each
// thread takes keys j = lo+t, lo+t+256, ... and leaves their scores in LDS, where they become e_j once the
// maximum is known (contexts whose scores do not fit LDS recompute the scores of a chunk of keys in pass 2: the
// same deterministic function, so the same bits); in pass 2 the keys' value rows come into LDS a chunk at a time and
// thread d walks the chunk in key order for its own d.  The same code runs for a row of a prompt portion and
// for a decoded token, so the bits cannot differ.
#include "common.h"
#include "api.h"

struct AttnF32Args {
  const float* q;            // [rows, q_stride], head h at h*hd
  const int32_t* positions;  // [rows]
  const int32_t* row_seq;    // [rows]
  const int32_t* block_table;
  const float* k_cache;      // [pages][kv_heads][page_size][hd]
  const float* v_cache;      // same layout
  float* out;                // [rows, out_stride]
  int rows, heads, kv_heads, head_dim, page_size, table_stride, q_stride, out_stride, window;
  float scale;
  int page_shift;            // log2 of the page size, or -1 if it is no power of two
  const int32_t* tiles;      // [tiles][4] = row0, tokens, seq, 0 (consecutive rows of one sequence); null: a row a workgroup
};

// A key's row in registers.
template <int HD>
struct KeyRow {
  f32x4 v[HD / 4];
};

template <int HD>
__device__ __forceinline__ void load_row(KeyRow<HD>& r, const float* __restrict__ k) {
#pragma unroll
  for (int i = 0; i < HD / 4; ++i) r.v[i] = *reinterpret_cast<const f32x4*>(k + 4 * i);
}

template <int HD>
__device__ __forceinline__ float dot_canonical(const float* __restrict__ q_lds, const KeyRow<HD>& k) {
  float lane[16];
#pragma unroll
  for (int i = 0; i < 16; ++i) lane[i] = 0.0f;
#pragma unroll
  for (int c = 0; c < HD / 16; ++c)
#pragma unroll
    for (int i = 0; i < 16; ++i) lane[i] = fmaf(q_lds[c * 16 + i], k.v[c * 4 + (i >> 2)][i & 3], lane[i]);
  float s8[8], s4[4];
#pragma unroll
  for (int i = 0; i < 8; ++i) s8[i] = lane[i] + lane[i + 8];
#pragma unroll
  for (int i = 0; i < 4; ++i) s4[i] = s8[i] + s8[i + 4];
  const float a = s4[0] + s4[2];
  const float b = s4[1] + s4[3];
  return a + b;
}

#define ATT32_THREADS 256
#define ATT32_TABLE 2048            // entries of a block table's row that the workgroup keeps in LDS

// Keys of a chunk of pass 2: as many as 32 KB of value rows hold, at most one a thread.
template <int HD>
struct Att32Shape {
  static constexpr int T = ATT32_THREADS;
  static constexpr int KC = (8192 / HD) < T ? (8192 / HD) : T;
  static constexpr int SEGS = HD / 4;                              // 16-byte pieces of a key's row
  static constexpr int VJ = (KC * SEGS + T - 1) / T;               // pieces of a chunk's value rows a thread
  static constexpr int LDS_BYTES = 2 * KC * HD * (int)sizeof(float);
  static constexpr int BLK = 16, NBLK = KC / BLK;                  // the walk of a whole chunk: blocks of keys
};

// The walk of KC keys (a whole chunk) for element d: blocks of 16 keys, the next block's e_j and values read from
// LDS while this block's steps run (the walking wave has its SIMD to itself when tokens are decoded: what hides
// its read latency is its own chain).  Keys past the last whole block, and chunks that are not whole, take the
// plain loop.
template <int HD>
__device__ __forceinline__ void walk_chunk(const float* __restrict__ ed, const float* __restrict__ vd, float& sum, float& acc) {
  using S = Att32Shape<HD>;
  constexpr int BLK = S::BLK, NBLK = S::NBLK;
  float ev[2][BLK], vv[2][BLK];
#pragma unroll
  for (int i = 0; i < BLK; ++i) {
    ev[0][i] = ed[i];
    vv[0][i] = vd[i * HD];
  }
#pragma unroll
  for (int blk = 0; blk < NBLK; ++blk) {
    if (blk + 1 < NBLK) {
#pragma unroll
      for (int i = 0; i < BLK; ++i) {
        ev[(blk + 1) & 1][i] = ed[BLK * (blk + 1) + i];
        vv[(blk + 1) & 1][i] = vd[(BLK * (blk + 1) + i) * HD];
      }
    }
#pragma unroll
    for (int i = 0; i < BLK; ++i) {
      sum += ev[blk & 1][i];
      acc = fmaf(ev[blk & 1][i], vv[blk & 1][i], acc);
    }
  }
#pragma unroll
  for (int jj = BLK * NBLK; jj < S::KC; ++jj) {
    sum += ed[jj];
    acc = fmaf(ed[jj], vd[jj * HD], acc);
  }
}

// KEEP: the scores of pass 1 stay in LDS (``capacity`` of them: as many keys as a row of the block table, or the
// window, can hold), turn into e_j there once the maximum is known, and pass 2 fetches values only: the keys are
// read once and every dot product is computed once.  The e_j are the same function of the same numbers, so the bits
// are those of the two-pass form, which remains for contexts whose scores do not fit.
template <int HD, bool KEEP>
__global__ __launch_bounds__(ATT32_THREADS) void attention_f32_kernel(AttnF32Args a) {
  using S = Att32Shape<HD>;
  constexpr int T = S::T, KC = S::KC, SEGS = S::SEGS, VJ = S::VJ;
  extern __shared__ __attribute__((aligned(16))) float v_lds[];    // [2][KC][HD]: value rows of a chunk of keys; KEEP: then the scores
  float* scores = v_lds + 2 * KC * HD;
  __shared__ float q_lds[HD];
  __shared__ float e_lds[2][KC];
  __shared__ float red[T / 64];
  __shared__ int table_lds[ATT32_TABLE];
  const int row = a.tiles != nullptr ? a.tiles[4 * blockIdx.x] : blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
  const int pos = a.positions[row];
  if (pos < 0) return;
  const int kvh = h / (a.heads / a.kv_heads);
  const int32_t* table = a.block_table + (size_t)(a.tiles != nullptr ? a.tiles[4 * blockIdx.x + 2] : a.row_seq[row]) * a.table_stride;
  const float* qh = a.q + (size_t)row * a.q_stride + (size_t)h * HD;
  for (int i = tid; i < HD; i += T) q_lds[i] = qh[i];
  // the pages of the keys: from LDS where the row's table fits (a lookup in memory before every key's loads
  // would double the time a key takes)
  const int pages = (a.page_shift >= 0 ? pos >> a.page_shift : pos / a.page_size) + 1;
  const bool table_fits = pages <= ATT32_TABLE;
  if (table_fits)
    for (int i = tid; i < pages; i += T) table_lds[i] = table[i];
  __syncthreads();
  const int lo = (a.window > 0 && pos - a.window + 1 > 0) ? pos - a.window + 1 : 0;
  const size_t head_off = (size_t)kvh * a.page_size * HD;
  const size_t page_stride = (size_t)a.kv_heads * a.page_size * HD;
  // element offset of key j (clamped to the last key: loads past it stay inside the sequence and go unused)
  auto offset_of = [&](int j) -> size_t {
    j = j < pos ? j : pos;
    const int page = a.page_shift >= 0 ? j >> a.page_shift : j / a.page_size;
    const int slot = a.page_shift >= 0 ? j & (a.page_size - 1) : j % a.page_size;
    const int id = table_fits ? table_lds[page] : table[page];
    return (size_t)id * page_stride + head_off + (size_t)slot * HD;
  };

  // pass 1: the maximum (exact whatever the order), a key a thread at a time, the next key's row on its way
  // while this one's score is computed (two sets of registers in turn)
  float mx = -INFINITY;
  {
    KeyRow<HD> ka, kb;
    int j = lo + tid;
    load_row<HD>(ka, a.k_cache + offset_of(j));
    for (; j <= pos; j += 2 * T) {
      load_row<HD>(kb, a.k_cache + offset_of(j + T));
      const float s0 = dot_canonical<HD>(q_lds, ka) * a.scale;
      if constexpr (KEEP) scores[j - lo] = s0;
      mx = fmaxf(mx, s0);
      load_row<HD>(ka, a.k_cache + offset_of(j + 2 * T));
      if (j + T <= pos) {
        const float s1 = dot_canonical<HD>(q_lds, kb) * a.scale;
        if constexpr (KEEP) scores[j + T - lo] = s1;
        mx = fmaxf(mx, s1);
      }
    }
  }
  mx = wave_max(mx);
  if ((tid & 63) == 0) red[tid >> 6] = mx;
  __syncthreads();
  mx = red[0];
#pragma unroll
  for (int w = 1; w < T / 64; ++w) mx = fmaxf(mx, red[w]);

  // pass 2, KC keys at a time: the last KC threads compute e_j of a key each (the same deterministic function of
  // the key as in pass 1) and all threads bring the keys' value rows into LDS; thread d < HD then walks the
  // chunk in key order for element d.  The next chunk is fetched before the walk and parked after it, into the
  // other buffers: one barrier a chunk, and the loads fly during the walk.
  f32x4 vreg[VJ];
  auto fetch = [&](int j0) {
#pragma unroll
    for (int i = 0; i < VJ; ++i) {
      const int c = tid + T * i;
      const int cc = c < KC * SEGS ? c : KC * SEGS - 1;
      vreg[i] = *reinterpret_cast<const f32x4*>(a.v_cache + offset_of(j0 + cc / SEGS) + 4 * (cc % SEGS));
    }
  };
  auto stash = [&](int buf) {
#pragma unroll
    for (int i = 0; i < VJ; ++i) {
      const int c = tid + T * i;                           // piece c = key c / SEGS, elements 4 * (c % SEGS)..: float 4c of the buffer
      if (c < KC * SEGS) *reinterpret_cast<f32x4*>(v_lds + buf * KC * HD + 4 * c) = vreg[i];
    }
  };
  const int et = tid - (T - KC);                           // this thread's key within a chunk, if not negative
  KeyRow<HD> krow;
  auto park = [&](int j0, int buf) {                       // ``krow`` holds key j0 + et; afterwards key j0 + KC + et
    if (KEEP || et < 0) return;
    const int j = j0 + et;
    const float e = bw_expf(dot_canonical<HD>(q_lds, krow) * a.scale - mx);
    load_row<HD>(krow, a.k_cache + offset_of(j + KC));
    e_lds[buf][et] = j <= pos ? e : 0.0f;
  };
  float acc = 0.0f, sum = 0.0f;
  auto walk = [&](int j0, int buf) {                       // thread d < HD: keys j0 .. of the chunk in ``buf``, in key order
    if (tid >= HD) return;
    const int cnt = (pos - j0 + 1) < KC ? (pos - j0 + 1) : KC;
    const float* vd = v_lds + buf * KC * HD + tid;
    const float* ed = KEEP ? scores + (j0 - lo) : e_lds[buf];
    if (cnt == KC) {
      walk_chunk<HD>(ed, vd, sum, acc);
    } else {
#pragma unroll 8
      for (int jj = 0; jj < cnt; ++jj) {
        const float ej = ed[jj];
        sum += ej;
        acc = fmaf(ej, vd[jj * HD], acc);
      }
    }
  };
  if constexpr (KEEP) {
    // Values only.  Three chunks of them are on their way at any time (three sets of registers in turn; a chunk in
    // flight is what keeps a compute unit's share of the memory system busy across a trip to memory), the first
    // three asked for before the scores turn into e_j.  Chunks past the last key fetch the last key again.
    f32x4 r0[VJ], r1[VJ], r2[VJ];
    auto fetch_into = [&](f32x4 (&reg)[VJ], int j0) {
#pragma unroll
      for (int i = 0; i < VJ; ++i) {
        const int c = tid + T * i;
        const int cc = c < KC * SEGS ? c : KC * SEGS - 1;
        reg[i] = *reinterpret_cast<const f32x4*>(a.v_cache + offset_of(j0 + cc / SEGS) + 4 * (cc % SEGS));
      }
    };
    auto stash_from = [&](int buf, const f32x4 (&reg)[VJ]) {
#pragma unroll
      for (int i = 0; i < VJ; ++i) {
        const int c = tid + T * i;
        if (c < KC * SEGS) *reinterpret_cast<f32x4*>(v_lds + buf * KC * HD + 4 * c) = reg[i];
      }
    };
    fetch_into(r0, lo);
    fetch_into(r1, lo + KC);
    fetch_into(r2, lo + 2 * KC);
    // every thread turns the scores it wrote itself into e_j; the barrier behind the first chunk's values publishes them
    for (int j = lo + tid; j <= pos; j += T) scores[j - lo] = bw_expf(scores[j - lo] - mx);
    stash_from(0, r0);
    __syncthreads();
    int buf = 0;
    for (int j0 = lo; j0 <= pos; j0 += 3 * KC) {           // (pos is the same for the whole workgroup: so are the exits)
      fetch_into(r0, j0 + 3 * KC);
      walk(j0, buf);
      stash_from(buf ^ 1, r1);
      __syncthreads();
      buf ^= 1;
      if (j0 + KC > pos) break;
      fetch_into(r1, j0 + 4 * KC);
      walk(j0 + KC, buf);
      stash_from(buf ^ 1, r2);
      __syncthreads();
      buf ^= 1;
      if (j0 + 2 * KC > pos) break;
      fetch_into(r2, j0 + 5 * KC);
      walk(j0 + 2 * KC, buf);
      stash_from(buf ^ 1, r0);
      __syncthreads();
      buf ^= 1;
    }
  } else {
    if (et >= 0) load_row<HD>(krow, a.k_cache + offset_of(lo + et));
    fetch(lo);
    park(lo, 0);
    stash(0);
    __syncthreads();
    int buf = 0;
    for (int j0 = lo; j0 <= pos; j0 += KC) {
      const bool more = j0 + KC <= pos;
      if (more) {
        fetch(j0 + KC);
        park(j0 + KC, buf ^ 1);
      }
      walk(j0, buf);
      if (more) stash(buf ^ 1);
      __syncthreads();
      buf ^= 1;
    }
  }
  if (tid < HD) a.out[(size_t)row * a.out_stride + (size_t)h * HD + tid] = acc * (1.0f / sum);
}

// Prompt portions: a workgroup per tile of up to 16 consecutive rows of one sequence and head, so that a chunk of
// 64 keys (and, in pass 2, their values) comes into LDS once for all of the tile's queries.  Thread (qi, kl)
// holds query qi's row in registers and computes its scores against keys kl, kl+16, kl+32, kl+48 of the chunk
// (dot_canonical, the same function of query and key as in the kernel above: the same bits); in pass 2 the e_j
// are parked in LDS and thread (qi, dl) walks the chunk in key order for elements dl, dl+16, ... of query qi,
// skipping the keys its query does not see.  Per query this is the statement sequence of the kernel above.
#define ATT32_QT 16
#define ATT32_CH 64

template <int HD>
__device__ __forceinline__ float dot_canonical_lds(const float (&q)[HD], const float* __restrict__ k) {
  float lane[16];
#pragma unroll
  for (int i = 0; i < 16; ++i) lane[i] = 0.0f;
#pragma unroll
  for (int c = 0; c < HD / 16; ++c)
#pragma unroll
    for (int i = 0; i < 16; ++i) lane[i] = fmaf(q[c * 16 + i], k[c * 16 + i], lane[i]);
  float s8[8], s4[4];
#pragma unroll
  for (int i = 0; i < 8; ++i) s8[i] = lane[i] + lane[i + 8];
#pragma unroll
  for (int i = 0; i < 4; ++i) s4[i] = s8[i] + s8[i + 4];
  const float x = s4[0] + s4[2];
  const float y = s4[1] + s4[3];
  return x + y;
}

template <int HD>
struct Att32Tile {
  static constexpr int T = ATT32_THREADS, CH = ATT32_CH, QT = ATT32_QT;
  static constexpr int KSTR = HD + 1;                               // floats from key to key in LDS (odd: no bank conflicts)
  static constexpr int PJ = CH * (HD / 4) / T;                      // 16-byte pieces of a chunk's rows a thread
  static constexpr int ND = HD / 16;                                // output elements a thread
  static constexpr int LDS_BYTES = (CH * KSTR + CH * HD + QT * CH) * (int)sizeof(float);
};

template <int HD>
__global__ __launch_bounds__(ATT32_THREADS) void attention_f32_tile_kernel(AttnF32Args a) {
  using S = Att32Tile<HD>;
  constexpr int T = S::T, CH = S::CH, KSTR = S::KSTR, PJ = S::PJ, ND = S::ND, SEGS = HD / 4;
  extern __shared__ __attribute__((aligned(16))) float tile_lds[];
  float* k_lds = tile_lds;                    // [CH][KSTR]
  float* v_lds = tile_lds + CH * KSTR;        // [CH][HD]
  float* e_lds = v_lds + CH * HD;             // [QT][CH]
  const int tid = threadIdx.x, qi = tid >> 4, kl = tid & 15, h = blockIdx.y;
  const int row0 = a.tiles[4 * blockIdx.x], ntok = a.tiles[4 * blockIdx.x + 1], seq = a.tiles[4 * blockIdx.x + 2];
  if (ntok <= 0) return;
  const int32_t* table = a.block_table + (size_t)seq * a.table_stride;
  const bool active = qi < ntok;
  const int my_row = row0 + (active ? qi : 0);
  const int pos_q = active ? a.positions[my_row] : -1;              // a padding row: nothing to do either
  const int lo_q = (a.window > 0 && pos_q - a.window + 1 > 0) ? pos_q - a.window + 1 : 0;
  // the tile's keys: from the first key any query sees to the last one (rows are in position order)
  const int pos_first = a.positions[row0], pos_last = a.positions[row0 + ntok - 1];
  if (pos_last < 0) return;
  const int lo_min = (a.window > 0 && pos_first - a.window + 1 > 0) ? pos_first - a.window + 1 : 0;
  const int kvh = h / (a.heads / a.kv_heads);
  const size_t head_off = (size_t)kvh * a.page_size * HD;
  const size_t page_stride = (size_t)a.kv_heads * a.page_size * HD;
  auto offset_of = [&](int j) -> size_t {                           // clamped to the tile's last key
    j = j < pos_last ? j : pos_last;
    const int page = a.page_shift >= 0 ? j >> a.page_shift : j / a.page_size;
    const int slot = a.page_shift >= 0 ? j & (a.page_size - 1) : j % a.page_size;
    return (size_t)table[page] * page_stride + head_off + (size_t)slot * HD;
  };
  float q[HD];
  {
    const float* qh = a.q + (size_t)my_row * a.q_stride + (size_t)h * HD;
#pragma unroll
    for (int i = 0; i < HD / 4; ++i) {
      const f32x4 t = *reinterpret_cast<const f32x4*>(qh + 4 * i);
      q[4 * i] = t[0]; q[4 * i + 1] = t[1]; q[4 * i + 2] = t[2]; q[4 * i + 3] = t[3];
    }
  }
  f32x4 kreg[PJ], vreg[PJ];
  auto fetch = [&](int c0, bool values) {
#pragma unroll
    for (int i = 0; i < PJ; ++i) {
      const int c = tid + T * i;
      const size_t off = offset_of(c0 + c / SEGS) + 4 * (c % SEGS);
      kreg[i] = *reinterpret_cast<const f32x4*>(a.k_cache + off);
      if (values) vreg[i] = *reinterpret_cast<const f32x4*>(a.v_cache + off);
    }
  };
  auto stash = [&](bool values) {
#pragma unroll
    for (int i = 0; i < PJ; ++i) {
      const int c = tid + T * i, key = c / SEGS, d = 4 * (c % SEGS);
      float* kd = k_lds + key * KSTR + d;
      kd[0] = kreg[i][0]; kd[1] = kreg[i][1]; kd[2] = kreg[i][2]; kd[3] = kreg[i][3];
      if (values) *reinterpret_cast<f32x4*>(v_lds + key * HD + d) = vreg[i];
    }
  };

  // pass 1: every query's maximum
  float mx = -INFINITY;
  fetch(lo_min, false);
  for (int c0 = lo_min; c0 <= pos_last; c0 += CH) {
    __syncthreads();                                                // everyone is done with the chunk before
    stash(false);
    __syncthreads();
    if (c0 + CH <= pos_last) fetch(c0 + CH, false);
#pragma unroll
    for (int u = 0; u < CH / 16; ++u) {
      const int key = c0 + kl + 16 * u;
      if (key >= lo_q && key <= pos_q) mx = fmaxf(mx, dot_canonical_lds<HD>(q, k_lds + (kl + 16 * u) * KSTR) * a.scale);
    }
  }
  mx = fmaxf(mx, __shfl_xor(mx, 8, 16));
  mx = fmaxf(mx, __shfl_xor(mx, 4, 16));
  mx = fmaxf(mx, __shfl_xor(mx, 2, 16));
  mx = fmaxf(mx, __shfl_xor(mx, 1, 16));

  // pass 2
  float acc[ND], sum = 0.0f;
#pragma unroll
  for (int u = 0; u < ND; ++u) acc[u] = 0.0f;
  fetch(lo_min, true);
  for (int c0 = lo_min; c0 <= pos_last; c0 += CH) {
    __syncthreads();
    stash(true);
    __syncthreads();
    if (c0 + CH <= pos_last) fetch(c0 + CH, true);
#pragma unroll
    for (int u = 0; u < CH / 16; ++u) {
      const int key = c0 + kl + 16 * u;
      float e = 0.0f;
      if (key >= lo_q && key <= pos_q) e = bw_expf(dot_canonical_lds<HD>(q, k_lds + (kl + 16 * u) * KSTR) * a.scale - mx);
      e_lds[qi * CH + kl + 16 * u] = e;
    }
    __syncthreads();
    if (pos_q >= 0) {
      // this query's keys of the chunk: jlo..jhi (none if jlo > jhi)
      const int jlo = lo_q > c0 ? lo_q - c0 : 0;
      const int jhi = pos_q - c0 < CH - 1 ? pos_q - c0 : CH - 1;
      const float* eq = e_lds + qi * CH;
      const float* vq = v_lds + kl;
#pragma unroll 4
      for (int jj = jlo; jj <= jhi; ++jj) {
        const float ej = eq[jj];
        sum += ej;
#pragma unroll
        for (int u = 0; u < ND; ++u) acc[u] = fmaf(ej, vq[jj * HD + 16 * u], acc[u]);
      }
    }
  }
  if (pos_q >= 0) {
    const float inv = 1.0f / sum;
    float* o = a.out + (size_t)my_row * a.out_stride + (size_t)h * HD + kl;
#pragma unroll
    for (int u = 0; u < ND; ++u) o[16 * u] = acc[u] * inv;
  }
}

template <int HD>
static void launch_attention_f32_tiles(const AttnF32Args& a, dim3 grid, hipStream_t s) {
  static bool allowed = false;
  if (!allowed) {
    (void)hipFuncSetAttribute((const void*)attention_f32_tile_kernel<HD>, hipFuncAttributeMaxDynamicSharedMemorySize,
                              Att32Tile<HD>::LDS_BYTES);
    allowed = true;
  }
  hipLaunchKernelGGL(attention_f32_tile_kernel<HD>, grid, dim3(ATT32_THREADS), Att32Tile<HD>::LDS_BYTES, s, a);
}

#define ATT32_KEEP_LDS (144 * 1024)     // dynamic LDS of the kernel that keeps its scores: the values' chunks and the scores

template <int HD>
static void launch_attention_f32(const AttnF32Args& a, dim3 grid, hipStream_t s) {
  static bool allowed = false;                         // 64 KB of dynamic LDS and more has to be asked for once
  if (!allowed) {
    (void)hipFuncSetAttribute((const void*)attention_f32_kernel<HD, false>, hipFuncAttributeMaxDynamicSharedMemorySize,
                              Att32Shape<HD>::LDS_BYTES);
    (void)hipFuncSetAttribute((const void*)attention_f32_kernel<HD, true>, hipFuncAttributeMaxDynamicSharedMemorySize,
                              ATT32_KEEP_LDS);
    allowed = true;
  }
  // the most keys a query of this launch can see: what a row of the block table covers, or the window
  long long capacity = (long long)a.table_stride * a.page_size;
  if (a.window > 0 && a.window < capacity) capacity = a.window;
  const long long keep_bytes = Att32Shape<HD>::LDS_BYTES + ((capacity + 3) & ~3ll) * (long long)sizeof(float);
  if (keep_bytes <= ATT32_KEEP_LDS)
    hipLaunchKernelGGL((attention_f32_kernel<HD, true>), grid, dim3(ATT32_THREADS), (size_t)keep_bytes, s, a);
  else
    hipLaunchKernelGGL((attention_f32_kernel<HD, false>), grid, dim3(ATT32_THREADS), Att32Shape<HD>::LDS_BYTES, s, a);
}

static int attention_f32_dispatch(const AttnF32Args& a, int items, int tiled, hipStream_t s) {
  if (a.kv_heads <= 0 || a.heads % a.kv_heads || a.heads > 65535) return -2;
  dim3 grid(items, a.heads);
#define BW_CASE(HD) case HD: if (tiled) launch_attention_f32_tiles<HD>(a, grid, s); else launch_attention_f32<HD>(a, grid, s); break;
#define BW_ROWS(HD) case HD: if (tiled) return -4; launch_attention_f32<HD>(a, grid, s); break;
  switch (a.head_dim) {
    BW_CASE(16) BW_CASE(32) BW_CASE(48) BW_CASE(64) BW_CASE(80) BW_CASE(96) BW_CASE(112) BW_CASE(128)
    BW_ROWS(160) BW_ROWS(192) BW_ROWS(224) BW_ROWS(256)
    default: return -4;  // head size not compiled in
  }
#undef BW_CASE
#undef BW_ROWS
  return BW_LAUNCH_CHECK();
}

extern "C" int bw_attention_f32(const float* q, int q_stride, const int32_t* positions, const int32_t* row_seq,
                                const int32_t* block_table, int table_stride, const float* k_cache,
                                const float* v_cache, float* out, int out_stride, int rows, int heads,
                                int kv_heads, int head_dim, int page_size, int window, float scale, void* stream) {
  if (rows <= 0) return 0;
  AttnF32Args a{q, positions, row_seq, block_table, k_cache, v_cache, out, rows, heads, kv_heads, head_dim,
                page_size, table_stride, q_stride, out_stride, window, scale,
                (page_size & (page_size - 1)) == 0 ? __builtin_ctz((unsigned)page_size) : -1, nullptr};
  return attention_f32_dispatch(a, rows, 0, (hipStream_t)stream);
}

// The same over a list of tiles ([tiles][4] = row0, tokens, sequence, 0; a tile's rows are consecutive rows of one
// sequence in position order).  tiled = 1: a workgroup per tile of up to 16 rows (head sizes up to 128; -4
// otherwise); tiled = 0: a workgroup per tile's first row (tiles of one row).  Both give the bits of bw_attention_f32.
extern "C" int bw_attention_f32_tiles(const float* q, int q_stride, const int32_t* positions, const int32_t* block_table,
                                      int table_stride, const int32_t* tiles, int num_tiles, int tiled,
                                      const float* k_cache, const float* v_cache, float* out, int out_stride, int heads,
                                      int kv_heads, int head_dim, int page_size, int window, float scale, void* stream) {
  if (num_tiles <= 0) return 0;
  if (tiles == nullptr) return -2;
  AttnF32Args a{q, positions, nullptr, block_table, k_cache, v_cache, out, 0, heads, kv_heads, head_dim,
                page_size, table_stride, q_stride, out_stride, window, scale,
                (page_size & (page_size - 1)) == 0 ? __builtin_ctz((unsigned)page_size) : -1, tiles};
  return attention_f32_dispatch(a, num_tiles, tiled, (hipStream_t)stream);
}
