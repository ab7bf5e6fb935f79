// bfloat16 causal attention over the paged cache on the matrix cores.
//
// Arithmetic (one definition for prompt portions and decoded tokens alike): the keys of a
// sequence are cut at absolute positions into partitions of 64.  For a query (one column of
// a 16-column tile) and a partition t the partial result is
//   s_j = (q . k_j) * scale           32-bit, from v_mfma_f32_16x16x32_bf16 over d ascending
//   m_t = max_j s_j                   over the partition's keys the query may see
//   p_j = bf16(exp(s_j - m_t)),  l_t = sum_j p_j (fixed order),  O_t = sum_j p_j * v_j (MFMA, keys ascending)
// and the partials are folded strictly left to right over t:
//   m' = max(m, m_t); a = exp(m - m'); b = exp(m_t - m'); l = fma(l, a, l_t*b); O = fma(O, a, O_t*b)
// (the first partition a query sees initialises the state; a partition it cannot see is
// skipped).  out = O * (1/l).  The fold kernel walks the partitions inside one wave; the
// split kernel computes one partition per wave and the combine kernel performs the same fold
// from memory, so both routes give the same bits, and a query's result depends on nothing
// but its own row, its position and the cache contents at positions it may see.
//
// Layout: S^T = K Q^T is computed (keys are MFMA rows, queries are columns), so the
// probabilities come out of the accumulator in exactly the lane layout that the second
// product O^T = V^T P^T needs for its B operand; no LDS is used.  K pages are
// [kv_head][slot][hd]; V pages are transposed, [kv_head][hd][slot], so that an A-operand
// lane reads 4 consecutive keys of one d with one 8-byte load.
#include "common.h"
#include "api.h"

#define ATT_PART 64

struct AttnBf16Args {
  const bf16_t* q;            // [rows, q_stride]
  const int32_t* positions;   // [rows]; negative = padding row
  const int32_t* block_table; // [seqs, table_stride]
  const int32_t* tiles;       // [tiles][4] = row0, tokens, seq, 0
  const bf16_t* k_cache;
  const bf16_t* v_cache;
  bf16_t* out;                // [rows, out_stride]
  float* part_o;              // split mode: [items][max_parts][hd/4][4][hpt]
  float* part_ml;             // split mode: [items][max_parts][2][hpt]
  int heads, kv_heads, page_size, table_stride, q_stride, out_stride, window, hpt, nsub, max_parts;
  float scale;
};

template <int HD>
struct TileCtx {
  static constexpr int NT = HD / 16;          // 16-wide d tiles
  static constexpr int KS = (HD + 31) / 32;   // 32-deep k steps of the score product
  int lane, r, g;
  int row_c, head_c, pos_c, lo_c;             // this lane's column (query): row, head, position, first visible key
  int kvh, kmax, kmin;                        // tile-wide: kv head, last and first key any column sees
  const int32_t* table;
  u32x4 qf[KS];
};

template <int HD>
__device__ __forceinline__ bool tile_setup(const AttnBf16Args& a, int tile, int head_item, TileCtx<HD>& t) {
  t.lane = threadIdx.x & 63;
  t.r = t.lane & 15;
  t.g = t.lane >> 4;
  const int group = a.heads / a.kv_heads;
  t.kvh = head_item / a.nsub;
  const int sub = head_item % a.nsub;
  const int row0 = a.tiles[tile * 4 + 0], ntok = a.tiles[tile * 4 + 1], seq = a.tiles[tile * 4 + 2];
  t.table = a.block_table + (size_t)seq * a.table_stride;
  const int tok = t.r / a.hpt, hh = t.r % a.hpt;
  const bool col_ok = tok < ntok && (sub * a.hpt + hh) < group && t.r < (16 / a.hpt) * a.hpt;
  t.row_c = row0 + (col_ok ? tok : 0);
  t.head_c = t.kvh * group + sub * a.hpt + (col_ok ? hh : 0);
  t.pos_c = col_ok ? a.positions[t.row_c] : -1;
  t.lo_c = (a.window > 0 && t.pos_c - a.window + 1 > 0) ? t.pos_c - a.window + 1 : 0;
  int kmax = t.pos_c, kmin = t.pos_c >= 0 ? t.lo_c : 0x7fffffff;
#pragma unroll
  for (int off = 8; off >= 1; off >>= 1) {
    kmax = max(kmax, __shfl_xor(kmax, off, BW_WAVE));
    kmin = min(kmin, __shfl_xor(kmin, off, BW_WAVE));
  }
  t.kmax = kmax;
  t.kmin = kmin;
  if (kmax < 0) return false;
#pragma unroll
  for (int ks = 0; ks < TileCtx<HD>::KS; ++ks) {
    const int d0 = 32 * ks + 8 * t.g;
    u32x4 v = {0u, 0u, 0u, 0u};
    if (t.pos_c >= 0 && d0 < HD)
      v = *reinterpret_cast<const u32x4*>(a.q + (size_t)t.row_c * a.q_stride + (size_t)t.head_c * HD + d0);
    t.qf[ks] = v;
  }
  return true;
}

// One partition's partial for the tile: per column m_p, l_p (replicated over the 4 lane
// groups) and O_p[dt][i] = element d = 16dt + 4g + i of the column.
template <int HD>
__device__ __forceinline__ void partition_partial(const AttnBf16Args& a, const TileCtx<HD>& t, int part,
                                                  float& m_p, float& l_p, f32x4 (&o_p)[HD / 16]) {
  constexpr int NT = HD / 16, KS = (HD + 31) / 32;
  const int key0 = part * ATT_PART;
  const size_t kpage = (size_t)a.kv_heads * a.page_size * HD;
  f32x4 st[4];
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    st[u] = (f32x4){0.f, 0.f, 0.f, 0.f};
    const int key_r = key0 + 16 * u + t.r;           // the key this lane feeds as an A row
    const bool k_ok = key_r <= t.kmax && key_r >= t.kmin;
    const bf16_t* kp = nullptr;
    if (k_ok)
      kp = a.k_cache + (size_t)t.table[key_r / a.page_size] * kpage +
           ((size_t)t.kvh * a.page_size + key_r % a.page_size) * HD;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const int d0 = 32 * ks + 8 * t.g;
      u32x4 kf = {0u, 0u, 0u, 0u};
      if (k_ok && d0 < HD) kf = *reinterpret_cast<const u32x4*>(kp + d0);
      st[u] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(kf), as_bf16x8(t.qf[ks]), st[u], 0, 0, 0);
    }
  }
  // scale, mask, column maximum
  float mx = -INFINITY;
  bool vis[4][4];
#pragma unroll
  for (int u = 0; u < 4; ++u)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int key = key0 + 16 * u + 4 * t.g + i;
      vis[u][i] = key <= t.pos_c && key >= t.lo_c;
      const float s = st[u][i] * a.scale;
      st[u][i] = s;
      if (vis[u][i]) mx = fmaxf(mx, s);
    }
  mx = fmaxf(mx, __shfl_xor(mx, 16, BW_WAVE));
  mx = fmaxf(mx, __shfl_xor(mx, 32, BW_WAVE));
  m_p = mx;
  // probabilities, rounded to bfloat16 once; their sum in fixed order
  float lsum = 0.0f;
  u32x4 pf[2];
#pragma unroll
  for (int w = 0; w < 2; ++w) {
    float p[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const int u = 2 * w + (e >> 2), i = e & 3;
      const float pe = vis[u][i] ? fast_exp(st[u][i] - mx) : 0.0f;
      const bf16_t pb = f32_to_bf16(pe);
      p[e] = bf16_to_f32(pb);
      lsum += p[e];
    }
    pf[w] = (u32x4){pack_bf16x2(p[0], p[1]), pack_bf16x2(p[2], p[3]), pack_bf16x2(p[4], p[5]), pack_bf16x2(p[6], p[7])};
  }
  lsum += __shfl_xor(lsum, 16, BW_WAVE);
  lsum += __shfl_xor(lsum, 32, BW_WAVE);
  l_p = lsum;
  // O_p^T = V^T P^T, keys ascending in steps of 32
  const size_t vpage = (size_t)a.kv_heads * HD * a.page_size;
#pragma unroll
  for (int dt = 0; dt < NT; ++dt) {
    o_p[dt] = (f32x4){0.f, 0.f, 0.f, 0.f};
    const int d = 16 * dt + t.r;
#pragma unroll
    for (int w = 0; w < 2; ++w) {
      u32x4 vf;
#pragma unroll
      for (int hseg = 0; hseg < 2; ++hseg) {
        const int kA = key0 + 32 * w + 16 * hseg + 4 * t.g;   // 4 consecutive keys
        u32x2 v2 = {0u, 0u};
        if (kA <= t.kmax && kA + 3 >= t.kmin) {
          const bf16_t* vp = a.v_cache + (size_t)t.table[kA / a.page_size] * vpage +
                             ((size_t)t.kvh * HD + d) * a.page_size + kA % a.page_size;
          v2 = *reinterpret_cast<const u32x2*>(vp);
          // keys beyond the last written one (or before the window) hold stale data: zero them
          const int over = kA + 3 - t.kmax;                  // keys kA+4-over .. kA+3 are unwritten
          if (over >= 1) v2[1] &= (over >= 2) ? 0u : 0x0000ffffu;
          if (over >= 3) v2[0] &= (over >= 4) ? 0u : 0x0000ffffu;
          const int under = t.kmin - kA;                     // keys kA .. kA+under-1 are gone
          if (under >= 1) v2[0] &= (under >= 2) ? 0u : 0xffff0000u;
          if (under >= 3) v2[1] &= (under >= 4) ? 0u : 0xffff0000u;
        }
        vf[2 * hseg] = v2[0];
        vf[2 * hseg + 1] = v2[1];
      }
      o_p[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(vf), as_bf16x8(pf[w]), o_p[dt], 0, 0, 0);
    }
  }
}

template <int NT>
__device__ __forceinline__ void fold(float& m, float& l, f32x4 (&o)[NT], float m_p, float l_p, const f32x4 (&o_p)[NT]) {
  if (m_p == -INFINITY) return;       // the query sees no key of this partition
  if (m == -INFINITY) {               // first partition it sees
    m = m_p;
    l = l_p;
#pragma unroll
    for (int dt = 0; dt < NT; ++dt) o[dt] = o_p[dt];
    return;
  }
  const float mn = fmaxf(m, m_p);
  const float fa = fast_exp(m - mn), fb = fast_exp(m_p - mn);
  l = fmaf(l, fa, l_p * fb);
#pragma unroll
  for (int dt = 0; dt < NT; ++dt)
#pragma unroll
    for (int i = 0; i < 4; ++i) o[dt][i] = fmaf(o[dt][i], fa, o_p[dt][i] * fb);
  m = mn;
}

template <int HD>
__device__ __forceinline__ void finish(const AttnBf16Args& a, const TileCtx<HD>& t, float l, const f32x4 (&o)[HD / 16]) {
  if (t.pos_c < 0) return;
  const float inv = 1.0f / l;
  bf16_t* dst = a.out + (size_t)t.row_c * a.out_stride + (size_t)t.head_c * HD;
#pragma unroll
  for (int dt = 0; dt < HD / 16; ++dt) {
    u32x2 pk = {pack_bf16x2(o[dt][0] * inv, o[dt][1] * inv), pack_bf16x2(o[dt][2] * inv, o[dt][3] * inv)};
    *reinterpret_cast<u32x2*>(dst + 16 * dt + 4 * t.g) = pk;
  }
}

// Route 1: one wave folds all partitions of its tile.
template <int HD>
__global__ __launch_bounds__(64) void attention_fold_kernel(AttnBf16Args a) {
  constexpr int NT = HD / 16;
  TileCtx<HD> t;
  if (!tile_setup<HD>(a, blockIdx.x, blockIdx.y, t)) return;
  float m = -INFINITY, l = 0.0f;
  f32x4 o[NT];
#pragma unroll
  for (int dt = 0; dt < NT; ++dt) o[dt] = (f32x4){0.f, 0.f, 0.f, 0.f};
  for (int part = t.kmin / ATT_PART; part <= t.kmax / ATT_PART; ++part) {
    float m_p, l_p;
    f32x4 o_p[NT];
    partition_partial<HD>(a, t, part, m_p, l_p, o_p);
    fold<NT>(m, l, o, m_p, l_p, o_p);
  }
  finish<HD>(a, t, l, o);
}

// Route 2a: one wave per (tile, partition) stores the partial.  Tiles of this route hold one
// token, so the live columns are the first hpt (one per head of the group); only those are
// stored: O as [register][lane group][column], m and l as [column].
template <int HD>
__global__ __launch_bounds__(64) void attention_split_kernel(AttnBf16Args a) {
  constexpr int NT = HD / 16;
  TileCtx<HD> t;
  if (!tile_setup<HD>(a, blockIdx.x, blockIdx.y, t)) return;
  const int part = blockIdx.z;
  if (part < t.kmin / ATT_PART || part > t.kmax / ATT_PART) return;
  float m_p, l_p;
  f32x4 o_p[NT];
  partition_partial<HD>(a, t, part, m_p, l_p, o_p);
  if (t.r >= a.hpt) return;
  const size_t item = ((size_t)blockIdx.x * gridDim.y + blockIdx.y) * a.max_parts + part;
  if (t.g == 0) {
    a.part_ml[(item * 2 + 0) * a.hpt + t.r] = m_p;
    a.part_ml[(item * 2 + 1) * a.hpt + t.r] = l_p;
  }
  float* po = a.part_o + item * (size_t)(HD * a.hpt);
#pragma unroll
  for (int dt = 0; dt < NT; ++dt)
#pragma unroll
    for (int i = 0; i < 4; ++i) po[((dt * 4 + i) * 4 + t.g) * a.hpt + t.r] = o_p[dt][i];
}

// Route 2b: the same left fold, reading the stored partials in partition order.
template <int HD>
__global__ __launch_bounds__(64) void attention_combine_kernel(AttnBf16Args a) {
  constexpr int NT = HD / 16;
  TileCtx<HD> t;
  if (!tile_setup<HD>(a, blockIdx.x, blockIdx.y, t)) return;
  float m = -INFINITY, l = 0.0f;
  f32x4 o[NT];
#pragma unroll
  for (int dt = 0; dt < NT; ++dt) o[dt] = (f32x4){0.f, 0.f, 0.f, 0.f};
  if (t.r < a.hpt) {
    for (int part = t.kmin / ATT_PART; part <= t.kmax / ATT_PART; ++part) {
      const size_t item = ((size_t)blockIdx.x * gridDim.y + blockIdx.y) * a.max_parts + part;
      const float m_p = a.part_ml[(item * 2 + 0) * a.hpt + t.r];
      const float l_p = a.part_ml[(item * 2 + 1) * a.hpt + t.r];
      const float* po = a.part_o + item * (size_t)(HD * a.hpt);
      f32x4 o_p[NT];
#pragma unroll
      for (int dt = 0; dt < NT; ++dt)
#pragma unroll
        for (int i = 0; i < 4; ++i) o_p[dt][i] = po[((dt * 4 + i) * 4 + t.g) * a.hpt + t.r];
      fold<NT>(m, l, o, m_p, l_p, o_p);
    }
  }
  finish<HD>(a, t, l, o);
}

extern "C" int bw_attention_bf16(const void* q, int q_stride, const int32_t* positions, const int32_t* block_table,
                                 int table_stride, const int32_t* tiles, int num_tiles, const void* k_cache,
                                 const void* v_cache, void* out, int out_stride, int heads, int kv_heads,
                                 int head_dim, int page_size, int window, float scale, int split, int max_parts,
                                 float* part_o, float* part_ml, void* stream) {
  if (num_tiles <= 0) return 0;
  if (kv_heads <= 0 || heads % kv_heads) return -2;
  if (page_size < 4 || (page_size & (page_size - 1)) || page_size > ATT_PART) return -5;  // 4-key loads stay inside a page
  if ((q_stride % 8) || (out_stride % 4)) return -3;
  const int group = heads / kv_heads;
  AttnBf16Args a;
  a.q = (const bf16_t*)q; a.positions = positions; a.block_table = block_table; a.tiles = tiles;
  a.k_cache = (const bf16_t*)k_cache; a.v_cache = (const bf16_t*)v_cache; a.out = (bf16_t*)out;
  a.part_o = part_o; a.part_ml = part_ml;
  a.heads = heads; a.kv_heads = kv_heads; a.page_size = page_size; a.table_stride = table_stride;
  a.q_stride = q_stride; a.out_stride = out_stride; a.window = window;
  a.hpt = group < 16 ? group : 16;
  a.nsub = (group + a.hpt - 1) / a.hpt;
  a.max_parts = max_parts;
  a.scale = scale;
  if (kv_heads * a.nsub > 65535 || max_parts > 65535) return -2;
  if (split && (max_parts <= 0 || !part_o || !part_ml)) return -2;
  hipStream_t s = (hipStream_t)stream;
  dim3 grid(num_tiles, kv_heads * a.nsub), block(64);
#define BW_CASE(HD)                                                                                   \
  case HD:                                                                                            \
    if (split) {                                                                                      \
      hipLaunchKernelGGL(attention_split_kernel<HD>, dim3(grid.x, grid.y, max_parts), block, 0, s, a); \
      hipLaunchKernelGGL(attention_combine_kernel<HD>, grid, block, 0, s, a);                         \
    } else {                                                                                          \
      hipLaunchKernelGGL(attention_fold_kernel<HD>, grid, block, 0, s, a);                            \
    }                                                                                                 \
    break;
  switch (head_dim) {
    BW_CASE(16) BW_CASE(32) BW_CASE(48) BW_CASE(64) BW_CASE(80) BW_CASE(96) BW_CASE(112) BW_CASE(128)
    BW_CASE(160) BW_CASE(192) BW_CASE(224) BW_CASE(256)
    default: return -4;
  }
#undef BW_CASE
  return BW_LAUNCH_CHECK();
}
