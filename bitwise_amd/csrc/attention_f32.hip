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

// A workgroup barrier for data that meets in LDS: this wave's LDS writes are done, then the barrier.  (The
// language's own barrier also waits for every load from memory that is still on its way, which would end the
// fetching ahead of the values across the chunks' barriers.)
__device__ __forceinline__ void lds_barrier() {
  asm volatile("" ::: "memory");
  __builtin_amdgcn_s_waitcnt(0xc07f);                    // lgkmcnt(0)
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
}
#define ATT32_TABLE 2048            // entries of a block table's row that the workgroup keeps in LDS

// Keys of a chunk of pass 2: as many as 32 KB of value rows hold, at most one a thread.
template <int HD>
struct Att32Shape {
  static constexpr int T = ATT32_THREADS;
  static constexpr int KC = ((8192 / HD) < T ? (8192 / HD) : T) & ~3;   // (a multiple of 4: the values of four keys lie side by side in LDS)
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
    // (KEEP: the launcher has seen to it that pages are a power of two and the table's row fits: no branch, no division)
    const int page = (KEEP || a.page_shift >= 0) ? j >> a.page_shift : j / a.page_size;
    const int slot = (KEEP || a.page_shift >= 0) ? j & (a.page_size - 1) : j % a.page_size;
    // (KEEP: the launcher has seen to it that the row fits.  A lookup in memory here, even one that is never
    // taken, makes the compiler wait for every load that is on its way before the next one is issued.)
    int id;
    if constexpr (KEEP) id = table_lds[page];
    else id = table_fits ? table_lds[page] : table[page];
    return (size_t)id * page_stride + head_off + (size_t)slot * HD;
  };

  // pass 1: the scores and their maximum (exact whatever the order).  Sixteen lanes take a key: lane t holds the
  // elements t, t + 16, ... of the query and loads those of the key (the sixteen lanes' loads are 64 bytes side by
  // side), so chain t of the canonical dot is its own, and the tree is the butterflies of a row of sixteen lanes
  // (l ^ 8, ^ 4, ^ 2, ^ 1: lane[i] + lane[i + 8], then + 4, then (s4[0] + s4[2]) + (s4[1] + s4[3]); an addition
  // gives the same bits whichever side a lane's own value stands on).  Four keys a group are on their way while
  // one is worked on.
  float mx = -INFINITY;
  {
    constexpr int NC = HD / 16, G = T / 16, DEPTH = 4;
    const int grp = tid >> 4, t = tid & 15;
    float qr[NC], kr[DEPTH][NC];
#pragma unroll
    for (int c = 0; c < NC; ++c) qr[c] = q_lds[16 * c + t];
    auto fetch_key = [&](float (&dst)[NC], int j) {
      const float* kp = a.k_cache + offset_of(j) + t;
#pragma unroll
      for (int c = 0; c < NC; ++c) dst[c] = kp[16 * c];
    };
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) fetch_key(kr[d], lo + grp + d * G);
    for (int base = lo; base <= pos; base += DEPTH * G) {          // (the same trips for every thread)
#pragma unroll
      for (int d = 0; d < DEPTH; ++d) {
        const int j = base + grp + d * G;
        float chain = 0.0f;
#pragma unroll
        for (int c = 0; c < NC; ++c) chain = fmaf(qr[c], kr[d][c], chain);
        fetch_key(kr[d], j + DEPTH * G);                           // (past the last key: the last key again, unused)
        const float sc = row16_sum(chain) * a.scale;
        if (j <= pos) {
          if constexpr (KEEP) {
            if (t == 0) scores[j - lo] = sc;
          }
          mx = fmaxf(mx, sc);
        }
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
    // Where the walk leaves two waves or more without an element (head sizes up to 128), those waves alone fetch
    // and stash, and the walking waves only walk: a chunk then costs the longer of the two, not their sum.
    constexpr int WW = (HD + 63) / 64, LW = T / 64 - WW;     // waves that walk, waves that do not
    constexpr bool APART = LW >= 2;
    constexpr int LT = APART ? 64 * LW : T;                  // threads that fetch and stash
    constexpr int VL = (KC * SEGS + LT - 1) / LT;            // pieces of a chunk's value rows for each of them
    const int lt = APART ? tid - 64 * WW : tid;              // (negative: this thread walks only)
    const bool loads = lt >= 0;
    f32x4 r0[VL], r1[VL], r2[VL];
    auto fetch_into = [&](f32x4 (&reg)[VL], int j0) {
      size_t off[VL];                                        // (all the pages looked up before the first load goes out)
#pragma unroll
      for (int i = 0; i < VL; ++i) {
        const int c = lt + LT * i;
        const int cc = c < KC * SEGS ? c : KC * SEGS - 1;
        off[i] = offset_of(j0 + cc / SEGS) + 4 * (cc % SEGS);
      }
#pragma unroll
      for (int i = 0; i < VL; ++i) reg[i] = *reinterpret_cast<const f32x4*>(a.v_cache + off[i]);
    };
    // The values of four keys lie side by side in LDS, [key / 4][place of d][key % 4], so that the walking thread
    // reads four keys' values of its element with one instruction; d's place is (d % 4) * HD / 4 + d / 4, which
    // spreads the stores of a wave (four keys, sixteen pieces each) over the banks.
    auto stash_from = [&](int buf, const f32x4 (&reg)[VL]) {
#pragma unroll
      for (int i = 0; i < VL; ++i) {
        const int c = lt + LT * i;                           // piece c = key c / SEGS, elements 4 * (c % SEGS)..
        if (c < KC * SEGS) {
          const int kk = c / SEGS, seg = c % SEGS;
          float* dst = v_lds + buf * KC * HD + (kk >> 2) * HD * 4 + seg * 4 + (kk & 3);
#pragma unroll
          for (int e = 0; e < 4; ++e) dst[e * SEGS * 4] = reg[i][e];
        }
      }
    };
    const int my_place = (tid & 3) * SEGS + (tid >> 2);      // (of element ``tid``, for the threads that walk)
    auto walk4 = [&](int j0, int buf) {                      // thread d < HD: the chunk's keys in key order, four a read
      if (tid >= HD) return;
      const int cnt = (pos - j0 + 1) < KC ? (pos - j0 + 1) : KC;
      const float* vb = v_lds + buf * KC * HD + my_place * 4;
      const float* eb = scores + (j0 - lo);
      if (cnt == KC) {
        // a whole chunk: KC / 4 reads of four e_j and of four values, written out so that the reads of the next
        // four quads are on their way while these four are chained (no condition, no register handed on)
        constexpr int NQ = KC / 4, BQ = 4;
        f32x4 ev[2][BQ], vv[2][BQ];
#pragma unroll
        for (int u = 0; u < BQ; ++u) {
          ev[0][u] = *reinterpret_cast<const f32x4*>(eb + 4 * u);
          vv[0][u] = *reinterpret_cast<const f32x4*>(vb + u * HD * 4);
        }
#pragma unroll
        for (int q0 = 0; q0 < NQ; q0 += BQ) {
          const int cur = (q0 / BQ) & 1;
          if (q0 + BQ < NQ) {
#pragma unroll
            for (int u = 0; u < BQ; ++u)
              if (q0 + BQ + u < NQ) {
                ev[cur ^ 1][u] = *reinterpret_cast<const f32x4*>(eb + 4 * (q0 + BQ + u));
                vv[cur ^ 1][u] = *reinterpret_cast<const f32x4*>(vb + (q0 + BQ + u) * HD * 4);
              }
          }
#pragma unroll
          for (int u = 0; u < BQ; ++u)
            if (q0 + u < NQ) {
#pragma unroll
              for (int i = 0; i < 4; ++i) {
                sum += ev[cur][u][i];
                acc = fmaf(ev[cur][u][i], vv[cur][u][i], acc);
              }
            }
        }
      } else {
#pragma unroll 4
        for (int jj = 0; jj < cnt; ++jj) {                   // the sequence's last keys
          const float ej = eb[jj];
          sum += ej;
          acc = fmaf(ej, vb[(jj >> 2) * HD * 4 + (jj & 3)], acc);
        }
      }
    };
    // one chunk's turn: the chunk three ahead is asked for into ``next``, the chunk in ``buf`` is walked, the
    // chunk one ahead goes from ``ready`` into the other buffer; the barrier publishes it
    auto turn = [&](f32x4 (&next)[VL], const f32x4 (&ready)[VL], int j0, int buf) {
      if constexpr (APART) {
        if (loads) {
          fetch_into(next, j0 + 3 * KC);
          stash_from(buf ^ 1, ready);
        } else {
          walk4(j0, buf);
        }
      } else {
        fetch_into(next, j0 + 3 * KC);
        walk4(j0, buf);
        stash_from(buf ^ 1, ready);
      }
      lds_barrier();
    };
    if (loads) {
      fetch_into(r0, lo);
      fetch_into(r1, lo + KC);
      fetch_into(r2, lo + 2 * KC);
    }
    // the scores turn into e_j (the barrier behind the maximum has published them; the one behind the first chunk's
    // values publishes the e_j)
    for (int j = lo + tid; j <= pos; j += T) scores[j - lo] = bw_expf(scores[j - lo] - mx);
    if (loads) stash_from(0, r0);
    lds_barrier();
    int buf = 0;
    for (int j0 = lo; j0 <= pos; j0 += 3 * KC) {           // (pos is the same for the whole workgroup: so are the exits)
      turn(r0, r1, j0, buf);
      if (j0 + KC > pos) break;
      turn(r1, r2, j0 + KC, buf ^ 1);
      if (j0 + 2 * KC > pos) break;
      turn(r2, r0, j0 + 2 * KC, buf);
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
  mx = row16_max(mx);

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

// ------------------------------------------------------------------------------ prompt portions on the matrix cores

// A wave per tile of up to 32 consecutive rows of one sequence and head.  v_mfma_f32_32x32x1_2b_f32 is, for every
// one of its 2 x 32 x 32 outputs, one fused multiply-add d = fma(a, b, d) with a single rounding: a chain of them
// is the scalar chain, bit for bit.  So both products of the attention run there, in the reference's order:
//   * scores, transposed (rows: 32 keys, columns: the tile's queries): chain c of dot_canonical (elements
//     16 j + c, j ascending) is HD / 16 instructions; the instruction's two blocks run chains c and c + 8, whose
//     sums the tree adds first (s8[c] = lane[c] + lane[c + 8]): the same registers of the two blocks.  The rest
//     of the tree, the scale and the maximum are vector instructions on 16 scores a lane.
//   * pass 2, keys in order: e = exp(s - max) where the query sees the key, else 0 (a key it does not see adds
//     +0 to a sum that is never -0, and fma(0, v, acc) = acc for the finite v of a written cache slot: the bits of
//     skipping it); sum += e along the keys, which a query's two lanes (l and l + 32 hold alternate groups of
//     four keys) hand back and forth; acc[q][d] = fma(e[q][k], v[k][d], acc[q][d]) is one instruction a key
//     (two for more than 64 elements), its A operand broadcast from the half of the wave that holds the key.
// The scores are computed twice (pass 1 keeps only the maximum), as in the kernels above.
typedef __attribute__((ext_vector_type(32))) float f32x32;

template <int HD>
struct Att32Mfma {
  static constexpr int NJ = HD / 16;            // steps of a chain of the dot
  static constexpr int NB = (HD + 63) / 64;     // accumulators of the second product, 64 output elements each
};

// 16 scores a lane: keys kb + 8 (r / 4) + 4 (lane / 32) + r % 4 against query lane % 32, before the scale.
// An instruction occupies the matrix core for 64 clocks, so one chain at a time keeps it busy; two accumulators
// alternate, the vector adds of one chain's tree running under the next chain's instructions, and the order is
// pinned (left to itself the scheduler starts all eight chains at once: eight accumulators of 32 registers).
// ``first`` is the chain's first key operand, kr[0][c], handed in by the caller (see the pins below).
template <int HD>
__device__ __forceinline__ f32x32 mfma_chain(const float (&kr)[HD / 16][8], const float (&qv)[HD / 16][8], int c, float first) {
  f32x32 acc = {};                               // (a constant zero: the first instruction's addend)
  acc = __builtin_amdgcn_mfma_f32_32x32x1f32(first, qv[0][c], acc, 0, 0, 0);
#pragma unroll
  for (int j = 1; j < HD / 16; ++j) acc = __builtin_amdgcn_mfma_f32_32x32x1f32(kr[j][c], qv[j][c], acc, 0, 0, 0);
  return acc;
}

// Pins 16 values and the next chain's first operand at this point of the program: statements like this one keep
// their order, so the sums above are computed (and the accumulators they read are free) before the chain below
// starts.  Left to itself the compiler starts all eight chains at once, eight accumulators of 32 registers, and
// spills what else the kernel holds.
#define BW_PIN16(v, k)                                                                                             \
  asm volatile("" : "+v"(v[0]), "+v"(v[1]), "+v"(v[2]), "+v"(v[3]), "+v"(v[4]), "+v"(v[5]), "+v"(v[6]), "+v"(v[7]),  \
               "+v"(v[8]), "+v"(v[9]), "+v"(v[10]), "+v"(v[11]), "+v"(v[12]), "+v"(v[13]), "+v"(v[14]), "+v"(v[15]), "+v"(k))

template <int HD>
__device__ __forceinline__ void mfma_scores(const float (&kr)[HD / 16][8], const float (&qv)[HD / 16][8], float (&s)[16]) {
  // lane[c] + lane[c + 8] of dot_canonical is block 0 + block 1 of chain c: the same registers of the two halves.
  // Two accumulators alternate: while one chain runs on the matrix core, the vector adds fold the chain before it.
  float x[16], t[16], k0;
  f32x32 p = mfma_chain<HD>(kr, qv, 0, kr[0][0]);
  f32x32 q = mfma_chain<HD>(kr, qv, 4, kr[0][4]);
#pragma unroll
  for (int i = 0; i < 16; ++i) x[i] = p[i] + p[16 + i];                           // s8[0]
  k0 = kr[0][2];
  BW_PIN16(x, k0);
  p = mfma_chain<HD>(kr, qv, 2, k0);
#pragma unroll
  for (int i = 0; i < 16; ++i) x[i] = x[i] + (q[i] + q[16 + i]);                  // s4[0] = s8[0] + s8[4]
  k0 = kr[0][6];
  BW_PIN16(x, k0);
  q = mfma_chain<HD>(kr, qv, 6, k0);
#pragma unroll
  for (int i = 0; i < 16; ++i) t[i] = p[i] + p[16 + i];                           // s8[2]
  k0 = kr[0][1];
  BW_PIN16(t, k0);
  p = mfma_chain<HD>(kr, qv, 1, k0);
#pragma unroll
  for (int i = 0; i < 16; ++i) x[i] = x[i] + (t[i] + (q[i] + q[16 + i]));         // s4[0] + s4[2]
  k0 = kr[0][5];
  BW_PIN16(x, k0);
  q = mfma_chain<HD>(kr, qv, 5, k0);
#pragma unroll
  for (int i = 0; i < 16; ++i) s[i] = p[i] + p[16 + i];                           // s8[1]
  k0 = kr[0][3];
  BW_PIN16(s, k0);
  p = mfma_chain<HD>(kr, qv, 3, k0);
#pragma unroll
  for (int i = 0; i < 16; ++i) s[i] = s[i] + (q[i] + q[16 + i]);                  // s4[1] = s8[1] + s8[5]
  k0 = kr[0][7];
  BW_PIN16(s, k0);
  q = mfma_chain<HD>(kr, qv, 7, k0);
#pragma unroll
  for (int i = 0; i < 16; ++i) t[i] = p[i] + p[16 + i];                           // s8[3]
  k0 = 0.0f;
  BW_PIN16(t, k0);
#pragma unroll
  for (int i = 0; i < 16; ++i) s[i] = x[i] + (s[i] + (t[i] + (q[i] + q[16 + i])));   // (s4[0] + s4[2]) + (s4[1] + s4[3])
  BW_PIN16(s, k0);
}

// Who takes which tile: a workgroup is eight waves of one head, and the hardware deals a workgroup's waves out to
// the compute unit's four SIMDs in turn, so waves w and w + 4 share a matrix core.  Wave w takes tile 4 k + w from
// the front of the list and wave w + 4 tile n - 1 - (4 k + w) from its back: the tiles of a long prompt come in
// position order, the work of a tile grows with its position, and so every matrix core gets a short tile and a
// long one, the same sum everywhere.  Workgroups of a head run on one die (the hardware deals workgroups out to the
// eight dies in turn), whose L2 then holds the keys and values of its heads only.
template <int HD>
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(2, 2))) void attention_f32_mfma_kernel(AttnF32Args a, int num_tiles, int groups) {
  constexpr int NJ = Att32Mfma<HD>::NJ, NB = Att32Mfma<HD>::NB;
  const int wave = wave_index(), lane = threadIdx.x & 63, col = lane & 31, h2 = lane >> 5;
  int h, k;
  {
    const int L = blockIdx.x;
    if (a.heads % 8 == 0) {
      const int die = L & 7, idx = L >> 3;                          // the idx-th workgroup of that die
      h = (idx / groups) * 8 + die;
      k = idx % groups;
    } else {
      h = L / groups;
      k = L % groups;
    }
  }
  const int front = 4 * k + (wave & 3), half_n = (num_tiles + 1) >> 1;
  const int tile = wave < 4 ? front : num_tiles - 1 - front;
  if (front >= half_n || (wave >= 4 && tile < half_n)) return;       // (the middle tile of an odd count is a front tile)
  const int row0 = a.tiles[4 * tile], ntok = a.tiles[4 * tile + 1], seq = a.tiles[4 * tile + 2];
  if (ntok <= 0) return;
  const int32_t* table = a.block_table + (size_t)seq * a.table_stride;
  const bool active = col < ntok;
  const int my_row = row0 + (active ? col : ntok - 1);
  const int pos_q = active ? a.positions[my_row] : -1;
  const int lo_q = (a.window > 0 && pos_q - a.window + 1 > 0) ? pos_q - a.window + 1 : 0;
  const int pos_first = a.positions[row0], pos_last = a.positions[row0 + ntok - 1];
  if (pos_last < 0) return;
  const int lo_min = (a.window > 0 && pos_first - a.window + 1 > 0) ? pos_first - a.window + 1 : 0;
  const int lo_last = (a.window > 0 && pos_last - a.window + 1 > 0) ? pos_last - a.window + 1 : 0;   // the last row's first key
  const int kvh = h / (a.heads / a.kv_heads);
  const float* kc = a.k_cache + (size_t)kvh * a.page_size * HD;     // this head's rows of page 0
  const float* vc = a.v_cache + (size_t)kvh * a.page_size * HD;
  const size_t page_stride = (size_t)a.kv_heads * a.page_size * HD;
  // where key kb + col lies: its page and its row within the page's rows of this head (keys past the tile's last are
  // that last key again: a written slot, whose products nobody sees)
  auto locate = [&](int kb, int& page, int& slot) {
    int j = kb + col;
    j = j < pos_last ? j : pos_last;
    page = table[a.page_shift >= 0 ? j >> a.page_shift : j / a.page_size];
    slot = a.page_shift >= 0 ? j & (a.page_size - 1) : j % a.page_size;
  };
  // this lane's half of its query's row: elements 16 j + 8 h2 + c
  float qv[NJ][8];
  {
    const float* qh = a.q + (size_t)my_row * a.q_stride + (size_t)h * HD + 8 * h2;
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
      const f32x4 t0 = *reinterpret_cast<const f32x4*>(qh + 16 * j), t1 = *reinterpret_cast<const f32x4*>(qh + 16 * j + 4);
      qv[j][0] = t0[0]; qv[j][1] = t0[1]; qv[j][2] = t0[2]; qv[j][3] = t0[3];
      qv[j][4] = t1[0]; qv[j][5] = t1[1]; qv[j][6] = t1[2]; qv[j][7] = t1[3];
    }
  }
  // the same half of the row of the lane's key
  auto load_keys_at = [&](const float* kp, float (&kr)[NJ][8]) {
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
      const f32x4 t0 = *reinterpret_cast<const f32x4*>(kp + 16 * j), t1 = *reinterpret_cast<const f32x4*>(kp + 16 * j + 4);
      kr[j][0] = t0[0]; kr[j][1] = t0[1]; kr[j][2] = t0[2]; kr[j][3] = t0[3];
      kr[j][4] = t1[0]; kr[j][5] = t1[1]; kr[j][6] = t1[2]; kr[j][7] = t1[3];
    }
  };
  auto load_keys = [&](int page, int slot, float (&kr)[NJ][8]) {
    load_keys_at(kc + (size_t)page * page_stride + (size_t)slot * HD + 8 * h2, kr);
  };
  const int key_of_reg = 4 * h2;                                    // register r: key kb + 8 (r / 4) + 4 h2 + r % 4
  // A whole block of 32 keys that starts at a multiple of 16, in pages of 16 slots or more, is two runs of 16 rows
  // that lie one behind the other in memory: two addresses a block, found by the scalar unit, instead of one a key
  // (address arithmetic is instructions of this wave too, and a wave's instructions do not overlap its own matrix
  // instructions).  Other blocks (a window's unaligned start, the tile's last block) take the general way.
  const bool runs16 = a.page_shift >= 4;
  auto run_start = [&](const float* cache, int j) -> const float* {  // the row of key j (a multiple of 16): scalar
    return cache + (size_t)table[j >> a.page_shift] * page_stride + (size_t)(j & (a.page_size - 1)) * HD;
  };
  auto load_keys_runs = [&](int kb, float (&kr)[NJ][8]) {
    const float* r0 = run_start(kc, kb);
    const float* r1 = run_start(kc, kb + 16);
    load_keys_at((col < 16 ? r0 : r1) + (col & 15) * HD + 8 * h2, kr);
  };

  // keys kb .. kb + 31 into kr; page and slot are set for the general way's value loads
  auto fetch_keys = [&](int kb, int& page, int& slot, float (&kr)[NJ][8]) {
    if (runs16 && (kb & 15) == 0 && kb + 31 <= pos_last) load_keys_runs(kb, kr);
    else {
      locate(kb, page, slot);
      load_keys(page, slot, kr);
    }
  };

  // pass 1: every query's maximum.  Two blocks of keys a turn of the loop, each in registers of its own, asked for a
  // whole block ahead of its use.
  float mx = -INFINITY;
  {
    float ka[NJ][8], kb2[NJ][8];
    int page, slot;
    fetch_keys(lo_min, page, slot, ka);
    if (lo_min + 32 <= pos_last) fetch_keys(lo_min + 32, page, slot, kb2);
#define ATT_PASS1(KB, KR)                                                                  \
    {                                                                                      \
      float s[16];                                                                         \
      mfma_scores<HD>(KR, qv, s);                                                          \
      if ((KB) + 64 <= pos_last) fetch_keys((KB) + 64, page, slot, KR);                    \
      __builtin_amdgcn_sched_barrier(0);                                                   \
      if ((KB) + 31 <= pos_first && (KB) >= lo_last) {       /* every query of the tile sees every key of the block */ \
        _Pragma("unroll") for (int r = 0; r < 16; ++r) mx = fmaxf(mx, s[r] * a.scale);     \
      } else {                                                                             \
        _Pragma("unroll") for (int r = 0; r < 16; ++r) {                                   \
          const int key = (KB) + 8 * (r >> 2) + key_of_reg + (r & 3);                      \
          const float t = fmaxf(mx, s[r] * a.scale);                                       \
          mx = (key >= lo_q && key <= pos_q) ? t : mx;                                     \
        }                                                                                  \
      }                                                                                    \
    }
    for (int kb = lo_min; kb <= pos_last; kb += 64) {
      ATT_PASS1(kb, ka)
      if (kb + 32 <= pos_last) ATT_PASS1(kb + 32, kb2)
    }
#undef ATT_PASS1
  }
  {
    float lower, upper;
    lane_halves<32>(mx, lower, upper);
    mx = fmaxf(lower, upper);
  }

  // pass 2: the keys of the next block are asked for when this block's scores are done, its values then too (for
  // heads of up to 64 elements, whose registers allow a second set), so both have a block's time to arrive.
  constexpr bool VAHEAD = false;
  f32x32 acc[NB];
#pragma unroll
  for (int nb = 0; nb < NB; ++nb) acc[nb] = f32x32{};
  float sum = 0.0f;
  {
    float kr[NJ][8];
    float va[32][NB], vb[VAHEAD ? 32 : 1][NB];
    int page, slot;
    page = 0;
    slot = 0;
    fetch_keys(lo_min, page, slot, kr);
    // a block's 32 value rows, element 64 nb + lane of each (zero past the head's size).  Where key k lies is what
    // lane k found for the keys' rows.  Every lane loads (clamped), and the zero is a select: nothing near a matrix
    // instruction runs under a partial execution mask.
#define ATT_VALUES(KB, VV)                                                                                              \
    if (runs16 && ((KB) & 15) == 0 && (KB) + 31 <= pos_last) {                                                          \
      const float* r0 = run_start(vc, (KB));                                                                            \
      const float* r1 = run_start(vc, (KB) + 16);                                                                       \
      _Pragma("unroll") for (int k = 0; k < 32; ++k) {                                                                  \
        const float* vp = (k < 16 ? r0 : r1) + (k & 15) * HD;                                                           \
        _Pragma("unroll") for (int nb = 0; nb < NB; ++nb) {                                                             \
          const int d = 64 * nb + lane;                                                                                 \
          const float t = vp[d < HD ? d : HD - 1];                                                                      \
          VV[k][nb] = d < HD ? t : 0.0f;                                                                                \
        }                                                                                                               \
      }                                                                                                                 \
    } else {                                                                                                            \
      _Pragma("unroll") for (int k = 0; k < 32; ++k) {                                                                  \
        const float* vp = vc + (size_t)__builtin_amdgcn_readlane(page, k) * page_stride +                               \
                          (size_t)__builtin_amdgcn_readlane(slot, k) * HD;                                              \
        _Pragma("unroll") for (int nb = 0; nb < NB; ++nb) {                                                             \
          const int d = 64 * nb + lane;                                                                                 \
          const float t = vp[d < HD ? d : HD - 1];                                                                      \
          VV[k][nb] = d < HD ? t : 0.0f;                                                                                \
        }                                                                                                               \
      }                                                                                                                 \
    }
    // Eight keys at a time (registers 4 g2 .. 4 g2 + 3: keys 8 g2 .. + 3 in the lower half of the wave, 8 g2 + 4 .. + 7
    // in the upper): their exponentials, sum += e in key order (the two halves hand the sum back and forth: after
    // the swap r[0] is the lower half's value in every lane, r[1] the upper half's), and
    // acc[q][d] = fma(e[q][k], v[k][d], acc[q][d]), k ascending; the vector work of the next eight keys runs under
    // these matrix instructions.
#define ATT_PASS2(KB, VCUR, VNEXT)                                                                                      \
    {                                                                                                                   \
      float e[16];                                                                                                      \
      if (!VAHEAD) { ATT_VALUES(KB, VCUR) }                                                                             \
      __builtin_amdgcn_sched_barrier(0);                                                                                \
      mfma_scores<HD>(kr, qv, e);                                                                                       \
      if ((KB) + 32 <= pos_last) {                                                                                      \
        fetch_keys((KB) + 32, page, slot, kr);                                                                          \
        if (VAHEAD) { ATT_VALUES((KB) + 32, VNEXT) }                                                                    \
      }                                                                                                                 \
      __builtin_amdgcn_sched_barrier(0);                                                                                \
      /* the exponentials' arguments; a key the query does not see: an argument whose exponential is 0 */               \
      if (!((KB) + 31 <= pos_first && (KB) >= lo_last)) {                                                               \
        _Pragma("unroll") for (int r = 0; r < 16; ++r) {                                                                \
          const int key = (KB) + 8 * (r >> 2) + key_of_reg + (r & 3);                                                   \
          e[r] = (key >= lo_q && key <= pos_q) ? e[r] * a.scale - mx : -200.0f;                                         \
        }                                                                                                               \
      } else {                                                                                                          \
        _Pragma("unroll") for (int r = 0; r < 16; ++r) e[r] = e[r] * a.scale - mx;                                      \
      }                                                                                                                 \
      __builtin_amdgcn_sched_barrier(0);                                                                                \
      _Pragma("unroll") for (int g2 = 0; g2 < 4; ++g2) {                                                                \
        _Pragma("unroll") for (int i = 0; i < 4; ++i) e[4 * g2 + i] = bw_expf(e[4 * g2 + i]);                    \
        float t = sum;                                                                                                  \
        _Pragma("unroll") for (int i = 0; i < 4; ++i) t += e[4 * g2 + i];   /* meaningful in the lower half */          \
        t = __uint_as_float(__builtin_amdgcn_permlane32_swap(__float_as_uint(t), __float_as_uint(t), false, false)[0]); \
        _Pragma("unroll") for (int i = 0; i < 4; ++i) t += e[4 * g2 + i];   /* meaningful in the upper half */          \
        sum = __uint_as_float(__builtin_amdgcn_permlane32_swap(__float_as_uint(t), __float_as_uint(t), false, false)[1]); \
        _Pragma("unroll") for (int i = 0; i < 4; ++i)                                                                   \
          _Pragma("unroll") for (int nb = 0; nb < NB; ++nb)                                                             \
            acc[nb] = __builtin_amdgcn_mfma_f32_32x32x1f32(e[4 * g2 + i], VCUR[8 * g2 + i][nb], acc[nb], 1, 0, 0);      \
        _Pragma("unroll") for (int i = 0; i < 4; ++i)                                                                   \
          _Pragma("unroll") for (int nb = 0; nb < NB; ++nb)                                                             \
            acc[nb] = __builtin_amdgcn_mfma_f32_32x32x1f32(e[4 * g2 + i], VCUR[8 * g2 + 4 + i][nb], acc[nb], 1, 1, 0);  \
      }                                                                                                                 \
      __builtin_amdgcn_sched_barrier(0);                                                                                \
    }
    if constexpr (VAHEAD) {
      ATT_VALUES(lo_min, va)
      for (int kb = lo_min; kb <= pos_last; kb += 64) {
        ATT_PASS2(kb, va, vb)
        if (kb + 32 <= pos_last) ATT_PASS2(kb + 32, vb, va)
      }
    } else {
      for (int kb = lo_min; kb <= pos_last; kb += 32) ATT_PASS2(kb, va, va)
    }
#undef ATT_PASS2
#undef ATT_VALUES
  }
  // out[q][d] = acc[q][d] * (1 / sum[q]): register r of block b is query 8 (r / 4) + 4 h2 + r % 4, element 64 nb + 32 b + col
  const float inv = 1.0f / sum;
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    const int q = 8 * (r >> 2) + key_of_reg + (r & 3);
    const float inv_q = __shfl(inv, q, 64);
    if (q >= ntok) continue;
    float* o = a.out + (size_t)(row0 + q) * a.out_stride + (size_t)h * HD;
#pragma unroll
    for (int nb = 0; nb < NB; ++nb)
#pragma unroll
      for (int b = 0; b < 2; ++b) {
        const int d = 64 * nb + 32 * b + col;
        if (d < HD) o[d] = acc[nb][16 * b + r] * inv_q;
      }
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
  if (keep_bytes <= ATT32_KEEP_LDS && a.table_stride <= ATT32_TABLE && a.page_shift >= 0)   // (and the table's row fits the kernel's copy of it)
    hipLaunchKernelGGL((attention_f32_kernel<HD, true>), grid, dim3(ATT32_THREADS), (size_t)keep_bytes, s, a);
  else
    hipLaunchKernelGGL((attention_f32_kernel<HD, false>), grid, dim3(ATT32_THREADS), Att32Shape<HD>::LDS_BYTES, s, a);
}

static int attention_f32_dispatch(const AttnF32Args& a, int items, int tiled, hipStream_t s) {
  if (a.kv_heads <= 0 || a.heads % a.kv_heads || a.heads > 65535) return -2;
  dim3 grid(items, a.heads);
#define BW_CASE(HD) case HD:                                                                                          \
    if (tiled == 2) {                                                                                                \
      const int groups = (((items + 1) >> 1) + 3) >> 2;                                                                  \
      hipLaunchKernelGGL(attention_f32_mfma_kernel<HD>, dim3(groups * a.heads), dim3(512), 0, s, a, items, groups);      \
    } else if (tiled) launch_attention_f32_tiles<HD>(a, grid, s);                                                        \
    else launch_attention_f32<HD>(a, grid, s);                                                                           \
    break;
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
// sequence in position order).  tiled = 1: a workgroup per tile of up to 16 rows; tiled = 2: a wave per tile of up to
// 32 rows, both products on the matrix cores (head sizes up to 128; -4 otherwise); tiled = 0: a workgroup per tile's
// first row (tiles of one row).  All give the bits of bw_attention_f32.
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
