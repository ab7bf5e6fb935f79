// bfloat16 causal attention over the paged cache on the matrix cores.
//
// Arithmetic (one definition for prompt portions and decoded tokens alike): the keys of a
// sequence are cut at absolute positions into partitions of 64.  Everything is in the base-2
// domain with c = scale * log2(e).  For a query (one column of a 16-column tile) and a
// partition t the partial result is
//   d_j = q . k_j                      32-bit, from v_mfma_f32_16x16x32_bf16 over the head's elements ascending
//   m_t = (max_j d_j) * c              over the partition's keys the query may see
//   p_j = bf16(exp2(fma(d_j, c, -m_t))), 0 for a key it may not see
//   l_t = sum_j p_j                    on the matrix core against rows of ones
//   O_t = sum_j p_j * v_j              by MFMA, keys ascending in steps of 32
// and the partials are folded strictly left to right over t, without branches:
//   m' = max(m, m_t); a = exp2(m - m'); b = exp2(m_t - m'); l = fma(l, a, l_t*b); O = fma(O, a, O_t*b)
// from the state m = -inf, l = 0, O = 0.  out = O * (1/l).  The fold kernel and the decode
// kernel call the same device functions for the partial and run the same statements for the
// fold, so both give the same bits, and a query's result depends on nothing but its own row,
// its position and the cache contents at positions it may see.
//
// Layout: S^T = K Q^T is computed (keys are MFMA rows, queries are columns), so the
// probabilities come out of the accumulator in exactly the lane layout that the second
// product O^T = V^T P^T needs for its B operand.  K pages are [kv_head][slot][hd]; V pages are
// transposed, [kv_head][hd][slot], so that an A-operand lane reads 4 consecutive keys of one
// element with one 8-byte load.
//
// Work shapes: the fold kernel (prompt portions) gives a workgroup of up to 8 waves as many
// tiles of one sequence and kv head, a tile a wave; the threads together stage each partition's
// keys and values once in LDS (the next partition's loads fly meanwhile), and every wave whose
// queries see the partition folds it into its own state.  The decode kernel (tiles of one
// token) gives a workgroup one tile and each of its 8 waves one partition at a time, operands
// straight from the pages into registers; the partials meet in LDS and are folded there in
// partition order.
#include "common.h"
#include "api.h"

#define ATT_PART 64
#define FOLD_QT(HD) 1                      // tiles per wave of the fold kernel
#define FOLD_NW(HD) ((HD) <= 192 ? 8 : 4)  // waves per workgroup of the fold kernel

struct AttnBf16Args {
  const bf16_t* q;            // [rows, q_stride]
  const int32_t* positions;   // [rows]; negative = padding row
  const int32_t* block_table; // [seqs, table_stride]
  const int32_t* tiles;       // [tiles][4] = row0, tokens, seq, 0; null: tile t is row t of sequence t
  const bf16_t* k_cache;
  const bf16_t* v_cache;
  bf16_t* out;                // [rows, out_stride]
  int heads, kv_heads, page_size, page_shift, num_pages, table_stride, q_stride, out_stride, window, hpt, nsub, num_tiles;
  float scale_log2;           // softmax scale times log2(e)
};

// What the lanes of a wave share for one group of tiles: sequence, kv head, key range.
struct GroupCtx {
  int lane, r, g, kvh, sub, kmax, kmin;
  const int32_t* table;
};

template <int HD>
struct TileCtx {
  static constexpr int KS = (HD + 31) / 32;   // 32-deep k steps of the score product
  int row_c, head_c, pos_c, lo_c;             // this lane's column (query): row, head, position, first visible key
  int all_hi, all_lo;                         // keys all_lo..all_hi are visible to every column (all_hi < all_lo: to none)
  u32x4 qf[KS];
};

template <int HD, int QT>
__device__ __forceinline__ bool group_setup(const AttnBf16Args& a, int first_tile, int head_item, GroupCtx& gc,
                                            TileCtx<HD> (&tc)[QT]) {
  gc.lane = threadIdx.x & 63;
  gc.r = gc.lane & 15;
  gc.g = gc.lane >> 4;
  const int group = a.heads / a.kv_heads;
  gc.kvh = head_item / a.nsub;
  gc.sub = head_item % a.nsub;
  const int tok = gc.r / a.hpt, hh = gc.r % a.hpt;
  const bool col_in = (gc.sub * a.hpt + hh) < group && gc.r < (16 / a.hpt) * a.hpt;
  int seq = 0;
  int kmax = -1, kmin = 0x7fffffff;
#pragma unroll
  for (int t = 0; t < QT; ++t) {
    const int tile = first_tile + t;
    int row0 = tile, ntok = 1, tseq = tile;
    if (tile >= a.num_tiles) ntok = 0;
    else if (a.tiles != nullptr) {
      row0 = a.tiles[tile * 4 + 0];
      ntok = a.tiles[tile * 4 + 1];
      tseq = a.tiles[tile * 4 + 2];
    }
    if (t == 0) seq = tseq;
    const bool ok = col_in && tok < ntok;
    tc[t].row_c = row0 + (ok ? tok : 0);
    tc[t].head_c = gc.kvh * group + gc.sub * a.hpt + (ok ? hh : 0);
    tc[t].pos_c = ok ? a.positions[tc[t].row_c] : -1;
    tc[t].lo_c = (a.window > 0 && tc[t].pos_c - a.window + 1 > 0) ? tc[t].pos_c - a.window + 1 : 0;
    kmax = max(kmax, tc[t].pos_c);
    if (tc[t].pos_c >= 0) kmin = min(kmin, tc[t].lo_c);
    // columns without a query do not count: what they compute is finite and never stored
    int hi = tc[t].pos_c >= 0 ? tc[t].pos_c : 0x7fffffff, lo = tc[t].pos_c >= 0 ? tc[t].lo_c : -1;
    hi = row16_min(hi);                                    // (moves between registers, no trip through LDS)
    lo = row16_max(lo);
    tc[t].all_hi = __builtin_amdgcn_readfirstlane(hi);   // the same in every lane: say so, branches on them are scalar then
    tc[t].all_lo = __builtin_amdgcn_readfirstlane(lo);
  }
  kmax = row16_max(kmax);
  kmin = row16_min(kmin);
  gc.kmax = __builtin_amdgcn_readfirstlane(kmax);
  gc.kmin = __builtin_amdgcn_readfirstlane(kmin);
  gc.table = a.block_table + (size_t)seq * a.table_stride;
  if (gc.kmax < 0) return false;
#pragma unroll
  for (int t = 0; t < QT; ++t)
#pragma unroll
    for (int ks = 0; ks < TileCtx<HD>::KS; ++ks) {
      const int d0 = 32 * ks + 8 * gc.g;
      u32x4 v = {0u, 0u, 0u, 0u};
      if (tc[t].pos_c >= 0 && d0 < HD)
        v = *reinterpret_cast<const u32x4*>(a.q + (size_t)tc[t].row_c * a.q_stride + (size_t)tc[t].head_c * HD + d0);
      tc[t].qf[ks] = v;
    }
  return true;
}

// ---- operands from the pages straight into registers (the decode kernel)
//
// Every load is unconditional and its address is always inside the cache (table index clamped
// into the row, page clamped into the pool), so that no load waits for a branch and the table
// lookups of a partition can be issued a partition ahead of the loads that need them.  Keys
// need no masking: a key no query sees gets probability 0 whatever its score.  Values do: 0
// times stale data (never written, or given back) could be NaN, so in a partition that is not
// wholly live the stale keys' values are zeroed before the product.
struct PartPages {
  int k[4], v[4];
};

__device__ __forceinline__ void load_pages(const AttnBf16Args& a, const GroupCtx& gc, int part, PartPages& pg) {
  const int key0 = part * ATT_PART;
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    const int pk = (key0 + 16 * u + gc.r) >> a.page_shift, pv = (key0 + 16 * u + 4 * gc.g) >> a.page_shift;
    pg.k[u] = gc.table[pk < a.table_stride ? pk : a.table_stride - 1];
    pg.v[u] = gc.table[pv < a.table_stride ? pv : a.table_stride - 1];
  }
}

__device__ __forceinline__ size_t clamp_page(const AttnBf16Args& a, int page) {
  return (size_t)min((unsigned)page, (unsigned)(a.num_pages - 1));
}

template <int HD>
struct KFrags {
  u32x4 k[4][(HD + 31) / 32];
};
// Keys of one partition as A operands: lane (r, g) feeds key 16u + r, elements 32ks + 8g .. +7.
template <int HD>
__device__ __forceinline__ void load_keys(const AttnBf16Args& a, const GroupCtx& gc, int part, const PartPages& pg,
                                          KFrags<HD>& kf) {
  constexpr int KS = (HD + 31) / 32;
  const size_t kpage = (size_t)a.kv_heads * a.page_size * HD;
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    const int slot = (16 * u + gc.r) & (a.page_size - 1);
    const bf16_t* kp = a.k_cache + clamp_page(a, pg.k[u]) * kpage + ((size_t)gc.kvh * a.page_size + slot) * HD;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const int d0 = 32 * ks + 8 * gc.g;
      if constexpr (HD % 32 != 0) {                 // the last step is half empty: zero against a zero query
        const u32x4 v = *reinterpret_cast<const u32x4*>(kp + (d0 < HD ? d0 : 0));
        kf.k[u][ks] = d0 < HD ? v : (u32x4){0u, 0u, 0u, 0u};
      } else {
        kf.k[u][ks] = *reinterpret_cast<const u32x4*>(kp + d0);
      }
    }
  }
}

// Values of one partition as A operands of O^T = V^T P^T: lane (r, g) feeds d = 16dt + r and, for
// the 32-key step w, keys 32w + 4g .. +3 and 32w + 16 + 4g .. +3 (the order in which the
// probabilities sit in the score accumulators).
template <int HD, int DT0, int NDT>
__device__ __forceinline__ void load_values_range(const AttnBf16Args& a, const GroupCtx& gc, const PartPages& pg,
                                                  u32x4 (&out)[NDT][2]) {
  const size_t vpage = (size_t)a.kv_heads * HD * a.page_size;
#pragma unroll
  for (int w = 0; w < 2; ++w)
#pragma unroll
    for (int hseg = 0; hseg < 2; ++hseg) {
      const int slot = (32 * w + 16 * hseg + 4 * gc.g) & (a.page_size - 1);
      const bf16_t* vp = a.v_cache + clamp_page(a, pg.v[2 * w + hseg]) * vpage + (size_t)gc.kvh * HD * a.page_size + slot;
#pragma unroll
      for (int dt = 0; dt < NDT; ++dt) {
        const u32x2 v2 = *reinterpret_cast<const u32x2*>(vp + (size_t)(16 * (DT0 + dt) + gc.r) * a.page_size);
        out[dt][w][2 * hseg] = v2[0];
        out[dt][w][2 * hseg + 1] = v2[1];
      }
    }
}

// Zero the values of keys outside kmin..kmax (four keys of one d in two words: m0 the first two).
__device__ __forceinline__ void stale_masks(int kA, int kmin, int kmax, uint32_t& m0, uint32_t& m1) {
  m0 = (kA <= kmax && kA + 3 >= kmin) ? 0xffffffffu : 0u;
  m1 = m0;
  const int over = kA + 3 - kmax;                        // keys kA+4-over .. kA+3 are unwritten
  if (over >= 1) m1 &= (over >= 2) ? 0u : 0x0000ffffu;
  if (over >= 3) m0 &= (over >= 4) ? 0u : 0x0000ffffu;
  const int under = kmin - kA;                           // keys kA .. kA+under-1 are gone
  if (under >= 1) m0 &= (under >= 2) ? 0u : 0xffff0000u;
  if (under >= 3) m1 &= (under >= 4) ? 0u : 0xffff0000u;
}

template <int NDT>
__device__ __forceinline__ void mask_values(const GroupCtx& gc, int part, u32x4 (&v)[NDT][2]) {
  const int key0 = part * ATT_PART;
  if (key0 >= gc.kmin && key0 + ATT_PART - 1 <= gc.kmax) return;   // wholly live
#pragma unroll
  for (int w = 0; w < 2; ++w)
#pragma unroll
    for (int hseg = 0; hseg < 2; ++hseg) {
      uint32_t m0, m1;
      stale_masks(key0 + 32 * w + 16 * hseg + 4 * gc.g, gc.kmin, gc.kmax, m0, m1);
#pragma unroll
      for (int dt = 0; dt < NDT; ++dt) {
        v[dt][w][2 * hseg] &= m0;
        v[dt][w][2 * hseg + 1] &= m1;
      }
    }
}

// Head sizes up to 128 load a partition's values at once (and early); larger ones load them
// 16 elements of d at a time where they are used, to stay within the register file.
template <int HD>
struct VFrags {
  static constexpr bool EARLY = HD <= 128;
  u32x4 v[EARLY ? HD / 16 : 1][2];
};

template <int HD>
__device__ __forceinline__ void load_values(const AttnBf16Args& a, const GroupCtx& gc, const PartPages& pg, VFrags<HD>& vf) {
  if constexpr (VFrags<HD>::EARLY) load_values_range<HD, 0, HD / 16>(a, gc, pg, vf.v);
}

template <int HD, int DT>
__device__ __forceinline__ void pv_step(const AttnBf16Args& a, const GroupCtx& gc, int part, const PartPages& pg,
                                        const VFrags<HD>& vf, const u32x4 (&pf)[2], f32x4 (&o_p)[HD / 16]) {
  if constexpr (DT < HD / 16) {
    o_p[DT] = (f32x4){0.f, 0.f, 0.f, 0.f};
    if constexpr (VFrags<HD>::EARLY) {
#pragma unroll
      for (int w = 0; w < 2; ++w)
        o_p[DT] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(vf.v[DT][w]), as_bf16x8(pf[w]), o_p[DT], 0, 0, 0);
    } else {
      u32x4 v[1][2];
      load_values_range<HD, DT, 1>(a, gc, pg, v);
      mask_values<1>(gc, part, v);
#pragma unroll
      for (int w = 0; w < 2; ++w)
        o_p[DT] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(v[0][w]), as_bf16x8(pf[w]), o_p[DT], 0, 0, 0);
    }
    pv_step<HD, DT + 1>(a, gc, part, pg, vf, pf, o_p);
  }
}

// Maximum without the canonicalising moves that fmaxf costs (the operands are never NaN): the
// median of x, y and +inf.  A builtin and not inline assembly on purpose: the operands often come
// straight out of a matrix instruction, and the compiler inserts the wait states that such a
// read needs only for instructions it knows.
__device__ __forceinline__ float max2_raw(float x, float y) { return __builtin_amdgcn_fmed3f(x, y, INFINITY); }
__device__ __forceinline__ float max3_raw(float x, float y, float z) { return max2_raw(max2_raw(x, y), z); }

// Maximum over the lanes l, l^16, l^32, l^48 (the four lane groups that share a column) with the
// register-to-register lane swaps of gfx950; no trip through LDS.
__device__ __forceinline__ float max_over_lane_groups(float v) {
  typedef __attribute__((ext_vector_type(2))) unsigned u2;
  const u2 h = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  v = max2_raw(__uint_as_float(h[0]), __uint_as_float(h[1]));
  const u2 q = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  return max2_raw(__uint_as_float(q[0]), __uint_as_float(q[1]));
}

// Scores of one tile against one partition -> probabilities as the B operand of the second
// product, and the column's maximum.  ``st`` holds the raw dot products.  Everything is in the
// base-2 domain: c = scale * log2(e), m_p = max_j(dot_j) * c, p_j = bf16(exp2(fma(dot_j, c, -m_p))).
template <int HD>
__device__ __forceinline__ void softmax_partition(const AttnBf16Args& a, const GroupCtx& gc, const TileCtx<HD>& t,
                                                  int key0, const f32x4 (&st)[4], float& m_p, u32x4 (&pf)[2]) {
  float mx = -INFINITY;
  if (key0 >= t.all_lo && key0 + ATT_PART - 1 <= t.all_hi) {
    // every key of the partition is visible to every column: the same statements without the masks
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      mx = max3_raw(mx, st[u][0], st[u][1]);
      mx = max3_raw(mx, st[u][2], st[u][3]);
    }
    mx = max_over_lane_groups(mx);
    mx = mx * a.scale_log2;
#pragma unroll
    for (int w = 0; w < 2; ++w)
#pragma unroll
      for (int e = 0; e < 8; e += 2) {
        const int u = 2 * w + (e >> 2), i = e & 3;
        pf[w][e >> 1] = pack_bf16x2(__builtin_amdgcn_exp2f(fmaf(st[u][i], a.scale_log2, -mx)),
                                    __builtin_amdgcn_exp2f(fmaf(st[u][i + 1], a.scale_log2, -mx)));
      }
  } else {
    bool vis[4][4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int key = key0 + 16 * u + 4 * gc.g + i;
        vis[u][i] = key <= t.pos_c && key >= t.lo_c;
      }
      mx = max3_raw(mx, vis[u][0] ? st[u][0] : -INFINITY, vis[u][1] ? st[u][1] : -INFINITY);
      mx = max3_raw(mx, vis[u][2] ? st[u][2] : -INFINITY, vis[u][3] ? st[u][3] : -INFINITY);
    }
    mx = max_over_lane_groups(mx);
    mx = mx * a.scale_log2;
#pragma unroll
    for (int w = 0; w < 2; ++w)
#pragma unroll
      for (int e = 0; e < 8; e += 2) {
        const int u = 2 * w + (e >> 2), i = e & 3;
        const float p0 = vis[u][i] ? __builtin_amdgcn_exp2f(fmaf(st[u][i], a.scale_log2, -mx)) : 0.0f;
        const float p1 = vis[u][i + 1] ? __builtin_amdgcn_exp2f(fmaf(st[u][i + 1], a.scale_log2, -mx)) : 0.0f;
        pf[w][e >> 1] = pack_bf16x2(p0, p1);
      }
  }
  m_p = mx;
}

// l_p = sum of the rounded probabilities of each column, on the matrix core against rows of ones
// (every accumulator row holds the column's sum, so no lane exchange is needed).
__device__ __forceinline__ float probability_sum(const u32x4 (&pf)[2]) {
  const u32x4 ones = {0x3f803f80u, 0x3f803f80u, 0x3f803f80u, 0x3f803f80u};
  f32x4 acc = {0.f, 0.f, 0.f, 0.f};
  acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(ones), as_bf16x8(pf[0]), acc, 0, 0, 0);
  acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(ones), as_bf16x8(pf[1]), acc, 0, 0, 0);
  return acc[0];
}

// One partition's partial for one tile from operands in registers: per column m_p, l_p
// (replicated over the 4 lane groups) and O_p[dt][i] = element d = 16dt + 4g + i of the column.
// ``pg`` holds the partition's pages (head sizes over 128 load their values here).
template <int HD>
__device__ __forceinline__ void partition_partial(const AttnBf16Args& a, const GroupCtx& gc, const TileCtx<HD>& t,
                                                  int part, const PartPages& pg, const KFrags<HD>& kf, VFrags<HD>& vf,
                                                  float& m_p, float& l_p, f32x4 (&o_p)[HD / 16]) {
  constexpr int KS = (HD + 31) / 32;
  f32x4 st[4];
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    st[u] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
      st[u] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(kf.k[u][ks]), as_bf16x8(t.qf[ks]), st[u], 0, 0, 0);
  }
  u32x4 pf[2];
  softmax_partition<HD>(a, gc, t, part * ATT_PART, st, m_p, pf);
  l_p = probability_sum(pf);
  // O_p^T = V^T P^T, keys ascending in steps of 32
  if constexpr (VFrags<HD>::EARLY) mask_values<HD / 16>(gc, part, vf.v);
  pv_step<HD, 0>(a, gc, part, pg, vf, pf, o_p);
}

// The fold step, without branches.  A state that has seen nothing is m = -inf, l = 0, O = 0, and a
// partial of a partition the query sees nothing of is m_p = -inf, l_p = 0, O_p = 0: with the
// factors below the first leaves the partial as it is (0 * 0 + x) and the second leaves the
// state as it is (x * 1 + 0 * 0).  Only when both are -inf the difference would be NaN, so the
// reference point is moved to 0 then.  The decode kernel's fold from LDS runs the same statements.
__device__ __forceinline__ void fold_scalars(float m, float m_p, float& mn, float& fa, float& fb) {
  mn = max2_raw(m, m_p);
  const float ref = mn == -INFINITY ? 0.0f : mn;
  fa = __builtin_amdgcn_exp2f(m - ref);
  fb = __builtin_amdgcn_exp2f(m_p - ref);
}

template <int NT>
__device__ __forceinline__ void fold(float& m, float& l, f32x4 (&o)[NT], float m_p, float l_p, const f32x4 (&o_p)[NT]) {
  float mn, fa, fb;
  fold_scalars(m, m_p, mn, fa, fb);
  l = fmaf(l, fa, l_p * fb);
#pragma unroll
  for (int dt = 0; dt < NT; ++dt) {
    // o = fmaf(o, fa, o_p * fb), the fused multiply-add written out in its three-address form: the compiler picks
    // the two-address one, whose result lands in the product's register, and then moves every element back to
    // where the loop keeps the state.  (The wait state in front: fa may come straight from the exponential unit.)
    const f32x4 t = {o_p[dt][0] * fb, o_p[dt][1] * fb, o_p[dt][2] * fb, o_p[dt][3] * fb};
    asm("s_nop 0\n\tv_fma_f32 %0, %0, %4, %5\n\tv_fma_f32 %1, %1, %4, %6\n\tv_fma_f32 %2, %2, %4, %7\n\tv_fma_f32 %3, %3, %4, %8"
        : "+v"(o[dt][0]), "+v"(o[dt][1]), "+v"(o[dt][2]), "+v"(o[dt][3])
        : "v"(fa), "v"(t[0]), "v"(t[1]), "v"(t[2]), "v"(t[3]));
  }
  m = mn;
}

// Route 1, for prompt portions.  A workgroup of FoldShape::NW waves owns FoldShape::GROUP consecutive tiles
// of one sequence and one kv head (the host pads every sequence's tile list to a multiple of
// that), wave w the tiles w*QT .. w*QT+QT-1.  The workgroup walks the partitions any of its
// queries may see; the threads together copy a partition's keys and values from the pages into
// LDS (the next partition's loads fly while this one is worked on), and every wave whose queries
// see the partition takes its operands from there and folds it into its own state.  Workgroups
// are handed out from the last tiles to the first: in a prompt the last queries see the most
// keys, and the long workgroups should start first.
template <int HD>
struct FoldShape {
  static constexpr int NW = FOLD_NW(HD);
  static constexpr int QT = FOLD_QT(HD);
  static constexpr int GROUP = NW * QT;
  static constexpr int NBUF = HD <= 128 ? 2 : 1;
  static constexpr int WAVES = HD <= 64 ? 4 : (HD <= 128 ? 2 : 1);   // waves per SIMD the register budget is set for
  // LDS layout, measured on the part: 16-byte operand reads of 16 rows by 4 chunks run at full rate when the rows lie
  // an odd multiple of 32 bytes apart (at twice the time 16 bytes off that, four times at a multiple of 128); 8-byte
  // reads want rows an odd multiple of 8 bytes apart; 128-byte rows read at full rate when their 16-byte chunks are
  // permuted by the row (fold_v_chunk)
  static constexpr int KSTR = HD * 2 + (HD % 32 == 0 ? 32 : 0);   // bytes from key to key
  static constexpr int VSTR = ATT_PART * 2;                       // bytes from d to d: no padding, chunks permuted
  static constexpr int KBYTES = ATT_PART * KSTR;
  static constexpr int BYTES = KBYTES + HD * VSTR;  // one partition
  static constexpr int KJ = (ATT_PART * (HD / 8) + 64 * NW - 1) / (64 * NW);   // 16-byte key chunks per thread
  static constexpr int VJ = (HD * (ATT_PART / 4) + 64 * NW - 1) / (64 * NW);   // 8-byte value chunks per thread
};

// Where the 8-byte slot ``slot`` (keys 4 * slot .. 4 * slot + 3) of the values' row d lies in the row's 128 bytes.
// The second product's operand of lane (g, r) for keys 32w .. 32w + 31 is keys 32w + 4g .. + 3 and 32w + 16 + 4g .. + 3
// of row d = 16 dt + r: those two slots lie side by side as 16-byte chunk 4w + g, so that one read brings the operand,
// and the chunk's place in the row is permuted by the row as the keys' chunks are in the product kernels.
__device__ __forceinline__ int fold_v_chunk(int chunk, int d) { return 16 * (chunk ^ ((d >> 1) & 7)); }
__device__ __forceinline__ int fold_v_offset(int slot, int d) {
  return fold_v_chunk(((slot >> 3) << 2) | (slot & 3), d) + 8 * ((slot >> 2) & 1);
}

template <int HD>
struct Staged {
  u32x4 k[FoldShape<HD>::KJ];
  u32x2 v[FoldShape<HD>::VJ];
};

// What the workgroup shares: sequence, kv head, the range of keys any of its queries sees.
struct WorkgroupCtx {
  const int32_t* table;
  int kvh, kmin, kmax;
};

// What a thread's chunks of a partition look like does not change from partition to partition
// (a partition starts at a multiple of the page size): which of the partition's pages, and
// where in the page.
template <int HD>
struct StagePlan {
  int k_key[FoldShape<HD>::KJ], k_off[FoldShape<HD>::KJ];   // key within the partition (64: no chunk); offset in the page
  int v_key[FoldShape<HD>::VJ], v_off[FoldShape<HD>::VJ], v_d[FoldShape<HD>::VJ];
};

template <int HD>
__device__ __forceinline__ void stage_plan(const AttnBf16Args& a, int kvh, StagePlan<HD>& sp) {
  using S = FoldShape<HD>;
  constexpr int SEG = HD / 8, THREADS = 64 * S::NW;
#pragma unroll
  for (int j = 0; j < S::KJ; ++j) {
    const int c = (int)threadIdx.x + THREADS * j;
    const int key = c / SEG, seg = c % SEG;
    sp.k_key[j] = c < ATT_PART * SEG ? key : ATT_PART;
    sp.k_off[j] = (kvh * a.page_size + (key & (a.page_size - 1))) * HD + seg * 8;   // inside the page for any c
  }
  // values: a chunk is 4 consecutive keys of one d; consecutive threads take consecutive chunks of a page
  const int cshift = a.page_shift - 2;
#pragma unroll
  for (int j = 0; j < S::VJ; ++j) {
    const int c = (int)threadIdx.x + THREADS * j;
    const int within = c & ((1 << cshift) - 1), rowi = c >> cshift;
    const int d = rowi % HD, key = ((rowi / HD) << a.page_shift) + 4 * within;
    sp.v_key[j] = key < ATT_PART ? key : ATT_PART;
    sp.v_off[j] = (kvh * HD + d) * a.page_size + (key & (a.page_size - 1));
    sp.v_d[j] = d;
  }
}

template <int HD>
struct StagePages {
  int k[FoldShape<HD>::KJ], v[FoldShape<HD>::VJ];
};

// The pages of a partition's chunks; the index is clamped into the table's row, so this may be
// asked for a partition past the last one.
template <int HD>
__device__ __forceinline__ void stage_pages(const AttnBf16Args& a, const WorkgroupCtx& wc, const StagePlan<HD>& sp,
                                            int part, StagePages<HD>& pg) {
  using S = FoldShape<HD>;
  const int page0 = (part * ATT_PART) >> a.page_shift;
#pragma unroll
  for (int j = 0; j < S::KJ; ++j) {
    const int pidx = page0 + (sp.k_key[j] >> a.page_shift);
    pg.k[j] = wc.table[pidx < a.table_stride ? pidx : a.table_stride - 1];
  }
#pragma unroll
  for (int j = 0; j < S::VJ; ++j) {
    const int pidx = page0 + (sp.v_key[j] >> a.page_shift);
    pg.v[j] = wc.table[pidx < a.table_stride ? pidx : a.table_stride - 1];
  }
}

// Unconditional loads from addresses that are always inside the cache; see the operand loaders above.  Keys and
// values separately: all waves of a workgroup ask for their chunks at the same point of the loop, and a compute
// unit's one path to memory takes a few hundred clocks to accept a whole partition's requests, so the loop asks for
// the next partition piece by piece, between the phases of its arithmetic.
template <int HD>
__device__ __forceinline__ void stage_load_keys(const AttnBf16Args& a, const StagePlan<HD>& sp, const StagePages<HD>& pg,
                                                Staged<HD>& sg) {
  using S = FoldShape<HD>;
  // (a page's bytes fit 32 bits, so page * bytes is one 32 x 32 -> 64-bit multiply-add onto the chunk's base)
  const unsigned page_bytes = (unsigned)(a.kv_heads * a.page_size * HD) * 2u;
  const unsigned last_page = (unsigned)(a.num_pages - 1);
#pragma unroll
  for (int j = 0; j < S::KJ; ++j)
    sg.k[j] = *reinterpret_cast<const u32x4*>(reinterpret_cast<const unsigned char*>(a.k_cache + sp.k_off[j]) +
                                              (unsigned long long)min((unsigned)pg.k[j], last_page) * page_bytes);
}

template <int HD>
__device__ __forceinline__ void stage_load_values(const AttnBf16Args& a, const StagePlan<HD>& sp, const StagePages<HD>& pg,
                                                  Staged<HD>& sg) {
  using S = FoldShape<HD>;
  const unsigned page_bytes = (unsigned)(a.kv_heads * a.page_size * HD) * 2u;   // values: the same number of elements
  const unsigned last_page = (unsigned)(a.num_pages - 1);
#pragma unroll
  for (int j = 0; j < S::VJ; ++j)
    sg.v[j] = *reinterpret_cast<const u32x2*>(reinterpret_cast<const unsigned char*>(a.v_cache + sp.v_off[j]) +
                                              (unsigned long long)min((unsigned)pg.v[j], last_page) * page_bytes);
}

// Staged partition -> LDS; in a partition that is not wholly live the stale keys' values are zeroed.
template <int HD>
__device__ __forceinline__ void stage_store(const WorkgroupCtx& wc, const StagePlan<HD>& sp, int part,
                                            const Staged<HD>& sg, unsigned char* buf) {
  using S = FoldShape<HD>;
  const int key0 = part * ATT_PART;
  const bool inner = key0 >= wc.kmin && key0 + ATT_PART - 1 <= wc.kmax;
#pragma unroll
  for (int j = 0; j < S::KJ; ++j)
    if (sp.k_key[j] < ATT_PART)
      *reinterpret_cast<u32x4*>(buf + sp.k_key[j] * S::KSTR + (sp.k_off[j] % HD) * 2) = sg.k[j];
#pragma unroll
  for (int j = 0; j < S::VJ; ++j) {
    u32x2 v2 = sg.v[j];
    if (!inner) {
      uint32_t m0, m1;
      stale_masks(key0 + sp.v_key[j], wc.kmin, wc.kmax, m0, m1);
      v2 = (u32x2){v2[0] & m0, v2[1] & m1};
    }
    if (sp.v_key[j] < ATT_PART)
      *reinterpret_cast<u32x2*>(buf + S::KBYTES + sp.v_d[j] * S::VSTR + fold_v_offset(sp.v_key[j] >> 2, sp.v_d[j])) = v2;
  }
}

// Which piece of work (0 = the group of the last tiles, the longest of a prompt; consecutive ranks = the heads of
// one group) the workgroup with this index takes.  Workgroups go to the 8 dies of the chip in turn, and on a die
// to its 32 compute units in turn; a prompt's groups often all fit the chip at once, and then what a compute unit
// gets in its first and in its second turn should add up to the same everywhere: the ranks run forward over the
// compute units in even turns and backward in odd ones, so a long piece meets a short one.
__device__ __forceinline__ int fold_work_rank(int index, int count) {
  if (count % 8 != 0) return index;
  const int die = index & 7, j = index >> 3, per_die = count >> 3;
  const int turn = j >> 5, cu = j & 31;
  const int in_turn = min(32, per_die - 32 * turn);
  return (32 * turn + ((turn & 1) ? in_turn - 1 - cu : cu)) * 8 + die;
}

template <int HD>
__global__ __launch_bounds__(64 * FoldShape<HD>::NW) __attribute__((amdgpu_waves_per_eu(FoldShape<HD>::WAVES, FoldShape<HD>::WAVES))) void attention_fold_kernel(AttnBf16Args a, int groups, int items) {
  using S = FoldShape<HD>;
  constexpr int NT = HD / 16, KS = (HD + 31) / 32, QT = S::QT, NW = S::NW;
  extern __shared__ __align__(16) unsigned char lds[];
  __shared__ int ranges[2 * NW];
  const int wave = wave_index();
  const int rank = fold_work_rank((int)blockIdx.x, (int)gridDim.x);
  const int first_tile = (groups - 1 - rank / items) * S::GROUP;
  GroupCtx gc;
  TileCtx<HD> tc[QT];
  const bool live = group_setup<HD, QT>(a, first_tile + wave * QT, rank % items, gc, tc);
  if (gc.lane == 0) {
    ranges[2 * wave] = live ? gc.kmin : 0x7fffffff;
    ranges[2 * wave + 1] = live ? gc.kmax : -1;
  }
  __syncthreads();
  WorkgroupCtx wc;
  wc.kmin = 0x7fffffff;
  wc.kmax = -1;
#pragma unroll
  for (int w = 0; w < NW; ++w) {
    wc.kmin = min(wc.kmin, ranges[2 * w]);
    wc.kmax = max(wc.kmax, ranges[2 * w + 1]);
  }
  wc.kmin = __builtin_amdgcn_readfirstlane(wc.kmin);
  wc.kmax = __builtin_amdgcn_readfirstlane(wc.kmax);
  if (wc.kmax < 0) return;                       // the same for every thread of the workgroup
  wc.kvh = gc.kvh;
  wc.table = a.block_table + (size_t)(a.tiles != nullptr ? a.tiles[first_tile * 4 + 2] : first_tile) * a.table_stride;
  const int my_first = live ? gc.kmin / ATT_PART : 1, my_last = live ? gc.kmax / ATT_PART : 0;
  float m[QT], l[QT];
  f32x4 o[QT][NT];
#pragma unroll
  for (int t = 0; t < QT; ++t) {
    m[t] = -INFINITY;
    l[t] = 0.0f;
#pragma unroll
    for (int dt = 0; dt < NT; ++dt) o[t][dt] = (f32x4){0.f, 0.f, 0.f, 0.f};
  }
  const int first = wc.kmin / ATT_PART, last = wc.kmax / ATT_PART;
  StagePlan<HD> sp;
  stage_plan<HD>(a, wc.kvh, sp);
  StagePages<HD> pg;
  stage_pages<HD>(a, wc, sp, first, pg);
  Staged<HD> sg;
  stage_load_keys<HD>(a, sp, pg, sg);
  stage_load_values<HD>(a, sp, pg, sg);
  stage_pages<HD>(a, wc, sp, first + 1, pg);
  int b = 0;
  for (int part = first; part <= last; ++part) {
    unsigned char* buf = lds + b * S::BYTES;
    if constexpr (S::NBUF == 1) __syncthreads();   // everyone is done with the partition before
    stage_store<HD>(wc, sp, part, sg, buf);
    __syncthreads();
    // The next partition is asked for in three pieces, each in front of a phase of this one's arithmetic (the
    // addresses are inside the cache for any partition number, so nothing here is conditional).
    const bool mine = part >= my_first && part <= my_last;    // the same for the whole wave
    f32x4 st[QT][4];
    float m_p[QT], l_p[QT];
    u32x4 pf[QT][2];
    stage_load_keys<HD>(a, sp, pg, sg);
    if (mine) {
      // scores of all the wave's tiles; a key operand is read once and used for each of them
#pragma unroll
      for (int u = 0; u < 4; ++u) {
#pragma unroll
        for (int t = 0; t < QT; ++t) st[t][u] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
          const int d0 = 32 * ks + 8 * gc.g;
          u32x4 kfrag = {0u, 0u, 0u, 0u};
          if (d0 < HD) kfrag = *reinterpret_cast<const u32x4*>(buf + (16 * u + gc.r) * S::KSTR + d0 * 2);
#pragma unroll
          for (int t = 0; t < QT; ++t)
            st[t][u] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(kfrag), as_bf16x8(tc[t].qf[ks]), st[t][u], 0, 0, 0);
        }
      }
    }
    stage_load_values<HD>(a, sp, pg, sg);
    if (mine) {
#pragma unroll
      for (int t = 0; t < QT; ++t) {
        softmax_partition<HD>(a, gc, tc[t], part * ATT_PART, st[t], m_p[t], pf[t]);
        l_p[t] = probability_sum(pf[t]);
      }
    }
    stage_pages<HD>(a, wc, sp, part + 2, pg);
    if (mine) {
      f32x4 o_p[QT][NT];
      const unsigned char* vb = buf + S::KBYTES;
#pragma unroll
      for (int dt = 0; dt < NT; ++dt) {
#pragma unroll
        for (int t = 0; t < QT; ++t) o_p[t][dt] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int w = 0; w < 2; ++w) {
          const u32x4 vfrag = *reinterpret_cast<const u32x4*>(vb + (16 * dt + gc.r) * S::VSTR + fold_v_chunk(4 * w + gc.g, gc.r));
#pragma unroll
          for (int t = 0; t < QT; ++t)
            o_p[t][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(vfrag), as_bf16x8(pf[t][w]), o_p[t][dt], 0, 0, 0);
        }
      }
#pragma unroll
      for (int t = 0; t < QT; ++t) fold<NT>(m[t], l[t], o[t], m_p[t], l_p[t], o_p[t]);
    }
    if constexpr (S::NBUF == 2) b ^= 1;
  }
  if (!live) return;
#pragma unroll
  for (int t = 0; t < QT; ++t) {
    if (tc[t].pos_c < 0) continue;
    const float inv = 1.0f / l[t];
    bf16_t* dst = a.out + (size_t)tc[t].row_c * a.out_stride + (size_t)tc[t].head_c * HD;
#pragma unroll
    for (int dt = 0; dt < NT; ++dt) {
      u32x2 pk = {pack_bf16x2(o[t][dt][0] * inv, o[t][dt][1] * inv), pack_bf16x2(o[t][dt][2] * inv, o[t][dt][3] * inv)};
      *reinterpret_cast<u32x2*>(dst + 16 * dt + 4 * gc.g) = pk;
    }
  }
}

// Route 2, for tiles of one token (decoded tokens): the workgroup's W waves deal the
// partitions among themselves (wave w takes partitions w, w+W, ..., prefetching the next one's
// keys), park every partition's partial in LDS, and after one barrier the threads fold the
// partials in partition order (thread t owns output elements t, t + threads, ... of the tile's
// live columns).  The statements are those of fold(), so the bits equal route 1; the waves
// only buy memory parallelism.  LDS holds ``pcap`` partitions; longer contexts take passes.
//
// SPLIT, for so few tiles that a workgroup each would leave most compute units idle: gridDim.z
// workgroups share a tile; workgroup z takes the partitions of rounds z, z + gridDim.z, ... (a
// round = W partitions) and writes their partials to ``scratch`` in device memory instead; each
// workgroup then counts itself in, and the one that finds all others counted in folds all
// partials, again in partition order from the first: the same statements on the same values.
// The counter is back at zero when the kernel ends.

// The fold of ``count`` parked partials, in partition order.  Often a single wave has all the output elements, and
// a wave alone issues an instruction every four clocks whatever the instruction: the work is cut so that the serial
// part is a few instructions a partition.  The factors of fold() for a partition depend only on the column's maxima
// up to it, and a running maximum can be had without running: first a thread per (eight partitions, column) takes
// their maximum; then a thread per (partition, column) takes the maximum of the eights before its own, of the
// partitions of its eight before it and of the passes before, and computes the two factors with fold_scalars() from
// the same two values fold() would see; then an output element's chain is a read, a product and a fused
// multiply-add a partition (the sums' chains run in other threads beside them).  The same statements on the same
// values as fold(): the same bits.  Sums and values wait in LDS between passes; the last pass divides and writes.
//
// The workgroup's LDS: three rows a column, padded to whole eights of partitions (a partition's two factors and its
// sum times its factor, each row read four partitions at a time); two rows of 16 running maxima (a pass reads one
// and writes the other) and the 16 sums; the eights' maxima; the output elements' values; then the partials
// [pcap][hpt][m, l, hd values].
struct FoldLds {
  float* fa;                    // [hpt][row]: the factor of what has been folded so far
  float* fb;                    //             the factor of the partition's partial
  float* lb;                    //             the partial's sum times fb
  float* mcol;
  float* lsum;
  float* eights;
  float* state;
  float* parts;
  int row;                      // floats from column to column of the factors
  __device__ __forceinline__ FoldLds(float* base, int pcap, int hpt, int hd) {
    row = (pcap + 7) & ~7;
    fa = base;
    fb = fa + row * hpt;
    lb = fb + row * hpt;
    mcol = lb + row * hpt;
    lsum = mcol + 32;
    eights = lsum + 16;
    state = eights + fold_lds_eights(pcap, hpt);
    parts = state + ((hpt * hd + 1) & ~1);
  }
  __host__ __device__ static int fold_lds_eights(int pcap, int hpt) { return (((pcap + 7) >> 3) * hpt + 1) & ~1; }
  static size_t bytes(int pcap, int hpt, int hd) {
    return ((size_t)3 * ((pcap + 7) & ~7) * hpt + 48 + fold_lds_eights(pcap, hpt) + (size_t)((hpt * hd + 1) & ~1) +
            (size_t)pcap * hpt * (hd + 2)) * sizeof(float);
  }
};

template <int HD, int W>
__device__ __forceinline__ void decode_fold_pass(const AttnBf16Args& a, const GroupCtx& gc, const FoldLds& lds, int count,
                                                 int pass, bool final_pass, int row) {
  constexpr int THREADS = 64 * W, CELL = HD + 2;
  const float* parts = lds.parts;
  const float* m_before = lds.mcol + 16 * (pass & 1);
  float* m_after = lds.mcol + 16 * ((pass & 1) ^ 1);
  const int pairs = count * a.hpt, eights = ((count + 7) >> 3) * a.hpt;
  for (int c = threadIdx.x; c < eights; c += THREADS) {
    const int k0 = (c / a.hpt) * 8, col = c % a.hpt;
    float m = -INFINITY;
#pragma unroll
    for (int u = 0; u < 8; ++u)       // (past the last partition: the last one again)
      m = max2_raw(m, parts[((size_t)min(k0 + u, count - 1) * a.hpt + col) * CELL]);
    lds.eights[c] = m;
  }
  __syncthreads();
  for (int p = threadIdx.x; p < pairs; p += THREADS) {
    const int wv = p / a.hpt, col = p % a.hpt, full = wv >> 3;
    float m = pass == 0 ? -INFINITY : m_before[col];
    // every read is asked for before the first is used, eight at a time; an index past the end reads the last
    // again, which a maximum does not mind
    for (int c = 0; c < full; c += 8) {
      float v[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) v[u] = lds.eights[min(c + u, full - 1) * a.hpt + col];
#pragma unroll
      for (int u = 0; u < 8; ++u) m = max2_raw(m, v[u]);
    }
    const float* cell = parts + ((size_t)wv * a.hpt + col) * CELL;
    const float m_p = cell[0], l_p = cell[1];
    float v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) v[u] = parts[((size_t)min(8 * full + u, count - 1) * a.hpt + col) * CELL];
#pragma unroll
    for (int u = 0; u < 8; ++u) m = max2_raw(m, 8 * full + u < wv ? v[u] : -INFINITY);
    float mn, fa, fb;
    fold_scalars(m, m_p, mn, fa, fb);
    lds.fa[col * lds.row + wv] = fa;
    lds.fb[col * lds.row + wv] = fb;
    lds.lb[col * lds.row + wv] = l_p * fb;
    if (wv == count - 1) m_after[col] = mn;
  }
  __syncthreads();
  const int elems = a.hpt * HD, cstride = a.hpt * CELL, group = a.heads / a.kv_heads, tail = count & ~7;
  // the sums' chains: the last threads, a column each
  if ((int)threadIdx.x >= THREADS - a.hpt) {
    const int col = THREADS - 1 - (int)threadIdx.x;
    const f32x4* fa4 = reinterpret_cast<const f32x4*>(lds.fa + col * lds.row);
    const f32x4* lb4 = reinterpret_cast<const f32x4*>(lds.lb + col * lds.row);
    float lj = pass == 0 ? 0.0f : lds.lsum[col];
    for (int wv = 0; wv < tail; wv += 8) {
      const f32x4 f0 = fa4[wv >> 2], f1 = fa4[(wv >> 2) + 1], b0 = lb4[wv >> 2], b1 = lb4[(wv >> 2) + 1];
#pragma unroll
      for (int u = 0; u < 4; ++u) lj = fmaf(lj, f0[u], b0[u]);
#pragma unroll
      for (int u = 0; u < 4; ++u) lj = fmaf(lj, f1[u], b1[u]);
    }
    for (int wv = tail; wv < count; ++wv) lj = fmaf(lj, lds.fa[col * lds.row + wv], lds.lb[col * lds.row + wv]);
    lds.lsum[col] = lj;
  }
  for (int e = threadIdx.x; e < elems; e += THREADS) {
    const int col = e / HD, d = e % HD;
    const f32x4* fa4 = reinterpret_cast<const f32x4*>(lds.fa + col * lds.row);
    const f32x4* fb4 = reinterpret_cast<const f32x4*>(lds.fb + col * lds.row);
    const float* cell = parts + (size_t)col * CELL + 2 + d;
    float oj = pass == 0 ? 0.0f : lds.state[e];
    // The next eight partitions' operands are on their way while this eight's chain runs.  Past the last partition
    // the factors' padding and the last partial again are read, and not used.
    f32x4 fa_n[2], fb_n[2];
    float op_n[8];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      fa_n[i] = fa4[i];
      fb_n[i] = fb4[i];
    }
#pragma unroll
    for (int u = 0; u < 8; ++u) op_n[u] = cell[min(u, count - 1) * cstride];
#pragma unroll 2
    for (int wv = 0; wv < tail; wv += 8) {
      f32x4 fa_c[2], fb_c[2];
      float op_c[8];
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        fa_c[i] = fa_n[i];
        fb_c[i] = fb_n[i];
      }
#pragma unroll
      for (int u = 0; u < 8; ++u) op_c[u] = op_n[u];
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        fa_n[i] = fa4[((wv + 8) >> 2) + i];
        fb_n[i] = fb4[((wv + 8) >> 2) + i];
      }
#pragma unroll
      for (int u = 0; u < 8; ++u) op_n[u] = cell[min(wv + 8 + u, count - 1) * cstride];
#pragma unroll
      for (int u = 0; u < 8; ++u) oj = fmaf(oj, fa_c[u >> 2][u & 3], op_c[u] * fb_c[u >> 2][u & 3]);
    }
#pragma unroll
    for (int u = 0; u < 7; ++u)
      if (tail + u < count) oj = fmaf(oj, fa_n[u >> 2][u & 3], op_n[u] * fb_n[u >> 2][u & 3]);
    lds.state[e] = oj;
  }
  if (!final_pass) return;
  __syncthreads();
  for (int e = threadIdx.x; e < elems; e += THREADS) {
    const int col = e / HD, d = e % HD;
    if (gc.sub * a.hpt + col >= group) continue;       // columns of a one-token tile: column c is head sub*hpt + c of the kv head's group
    const float inv = 1.0f / lds.lsum[col];
    a.out[(size_t)row * a.out_stride + (size_t)(gc.kvh * group + gc.sub * a.hpt + col) * HD + d] = f32_to_bf16(lds.state[e] * inv);
  }
}

// DEVICE: the cells lie in device memory and another workgroup, maybe on another die with its own
// L2, will read them in this same kernel: device-scope stores (they write through).
template <int HD, bool DEVICE>
__device__ __forceinline__ void store_partial(const AttnBf16Args& a, const GroupCtx& gc, float* cells, float m_p,
                                              float l_p, const f32x4 (&o_p)[HD / 16]) {
  if (gc.r >= a.hpt) return;
  float* cell = cells + (size_t)gc.r * (HD + 2);    // a partition's cells: [hpt][m, l, hd values]
  auto put = [&](int i, float v) {
    if constexpr (DEVICE) __hip_atomic_store(cell + i, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    else cell[i] = v;
  };
  if (gc.g == 0) {
    put(0, m_p);
    put(1, l_p);
  }
#pragma unroll
  for (int dt = 0; dt < HD / 16; ++dt)
#pragma unroll
    for (int i = 0; i < 4; ++i) put(2 + 16 * dt + 4 * gc.g + i, o_p[dt][i]);
}

template <int HD, int W, bool SPLIT>
__global__ __launch_bounds__(64 * W) __attribute__((amdgpu_waves_per_eu(2))) void attention_decode_kernel(AttnBf16Args a, int pcap, float* __restrict__ scratch,
                                                                  int* __restrict__ counters, int max_parts) {
  constexpr int NT = HD / 16;
  constexpr int THREADS = 64 * W;
  constexpr int CELL = HD + 2;                              // m, l, then hd values
  constexpr bool PREFETCH = HD <= 64 && !SPLIT;
  extern __shared__ __attribute__((aligned(16))) float lds_base[];
  const FoldLds lds(lds_base, pcap, a.hpt, HD);
  float* const parts = lds.parts;                  // [pcap][hpt][CELL]
  __shared__ int is_last;
  GroupCtx gc;
  TileCtx<HD> tc[1];
  const int wave = wave_index();
  // Without a window and with the implicit tile list the first partition is partition 0 of sequence blockIdx.x
  // whatever the position says: its pages are asked for beside the position, not after it (the table index is
  // clamped into the row and the pages into the pool, so a sequence shorter than that costs a wasted load).
  const bool early = a.window == 0 && a.tiles == nullptr;
  PartPages pg_first;
  if (early) {
    gc.r = threadIdx.x & 15;
    gc.g = (threadIdx.x & 63) >> 4;
    gc.table = a.block_table + (size_t)blockIdx.x * a.table_stride;
    load_pages(a, gc, (SPLIT ? (int)blockIdx.z * W : 0) + wave, pg_first);
  }
  const bool live = group_setup<HD, 1>(a, blockIdx.x, blockIdx.y, gc, tc);   // uniform over the workgroup
  if (!SPLIT && !live) return;
  const int first = gc.kmin / ATT_PART, last = gc.kmax / ATT_PART;
  const int row = a.tiles != nullptr ? a.tiles[blockIdx.x * 4] : blockIdx.x;
  if constexpr (SPLIT) {
    const int item = blockIdx.x * gridDim.y + blockIdx.y;
    float* mine = scratch + (size_t)item * max_parts * a.hpt * CELL;
    if (live) {
      PartPages pg;
      KFrags<HD> kf;
      VFrags<HD> vf;
      for (int part = first + blockIdx.z * W + wave; part <= last; part += W * gridDim.z) {
        if (early && part == (int)blockIdx.z * W + wave) pg = pg_first;
        else load_pages(a, gc, part, pg);
        load_keys<HD>(a, gc, part, pg, kf);
        load_values<HD>(a, gc, pg, vf);
        float m_p, l_p;
        f32x4 o_p[NT];
        partition_partial<HD>(a, gc, tc[0], part, pg, kf, vf, m_p, l_p, o_p);
        // The partial goes to the scratch through the wave's own cell of LDS, so that whole runs of bytes are
        // written, 8 a lane: device-scope stores write through, and the words of the accumulator layout (a few
        // lanes, 4 bytes each, 16 bytes apart) would each be a write of part of a line.  (A wave's LDS
        // instructions are carried out in order: the reads below see the stores above.)
        float* park = parts + (size_t)wave * a.hpt * CELL;
        store_partial<HD, false>(a, gc, park, m_p, l_p, o_p);
        const unsigned long long* from = reinterpret_cast<const unsigned long long*>(park);
        unsigned long long* to = reinterpret_cast<unsigned long long*>(mine + (size_t)(part - first) * a.hpt * CELL);
        for (int i = gc.lane; i < a.hpt * CELL / 2; i += 64)
          __hip_atomic_store(to + i, from[i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
    }
    // Every wave waits until its own device-scope stores are acknowledged (they write through: once the
    // wave's count of outstanding memory operations is zero they are in memory, no cache has to be written
    // back), then the barrier: when thread 0 counts the workgroup in, all of its partials are visible to the
    // device.  The count's atomic returns a value, so thread 0 has it before the second barrier, and the last
    // workgroup issues its loads (device scope again: they do not read a stale line of this die's L2) only
    // after that barrier.
    __builtin_amdgcn_s_waitcnt(vmcnt_only(0));
    __syncthreads();
    if (threadIdx.x == 0) is_last = atomicAdd(&counters[item], 1) == (int)gridDim.z - 1;
    __syncthreads();
    if (!is_last) return;
    if (threadIdx.x == 0) counters[item] = 0;
    if (!live) return;
    for (int pass0 = first; pass0 <= last; pass0 += pcap) {
      const int count = (last - pass0) < pcap ? last - pass0 + 1 : pcap;
      const float* src = mine + (size_t)(pass0 - first) * a.hpt * CELL;
      // eight loads of 8 bytes in flight a thread (a loop of one load and its store waits a memory round trip for
      // each: 40 us for the 66 KB of a group of four heads of 128 over 32 partitions)
      const int total = count * a.hpt * CELL / 2;
      const unsigned long long* src64 = reinterpret_cast<const unsigned long long*>(src);
      unsigned long long* parts64 = reinterpret_cast<unsigned long long*>(parts);
      for (int base = 0; base < total; base += 8 * THREADS) {
        unsigned long long v[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const int i = base + j * THREADS + (int)threadIdx.x;
          v[j] = __hip_atomic_load(src64 + (i < total ? i : 0), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const int i = base + j * THREADS + (int)threadIdx.x;
          if (i < total) parts64[i] = v[j];
        }
      }
      __syncthreads();
      decode_fold_pass<HD, W>(a, gc, lds, count, (pass0 - first) / pcap, pass0 + pcap > last, row);
      __syncthreads();
    }
  } else {
    for (int pass0 = first; pass0 <= last; pass0 += pcap) {
      const int pass_last = (last - pass0) < pcap ? last : pass0 + pcap - 1;
      KFrags<HD> kf, kf_next;
      VFrags<HD> vf, vf_next;
      PartPages pg, pg_now;
      int part = pass0 + wave;
      if (early && pass0 == 0) pg = pg_first;
      else load_pages(a, gc, part, pg);
      if constexpr (PREFETCH) {
        load_keys<HD>(a, gc, part, pg, kf);
        load_values<HD>(a, gc, pg, vf);
        load_pages(a, gc, part + W, pg);
      }
      for (; part <= pass_last; part += W) {
        if constexpr (PREFETCH) {
          if (part + W <= pass_last) {
            load_keys<HD>(a, gc, part + W, pg, kf_next);
            load_values<HD>(a, gc, pg, vf_next);
            load_pages(a, gc, part + 2 * W, pg);
          }
        } else {
          pg_now = pg;
          load_keys<HD>(a, gc, part, pg_now, kf);
          load_values<HD>(a, gc, pg_now, vf);
          load_pages(a, gc, part + W, pg);
        }
        float m_p, l_p;
        f32x4 o_p[NT];
        partition_partial<HD>(a, gc, tc[0], part, PREFETCH ? pg : pg_now, kf, vf, m_p, l_p, o_p);
        store_partial<HD, false>(a, gc, parts + (size_t)(part - pass0) * a.hpt * CELL, m_p, l_p, o_p);
        if constexpr (PREFETCH) {
          kf = kf_next;
          vf = vf_next;
        }
      }
      __syncthreads();
      decode_fold_pass<HD, W>(a, gc, lds, pass_last - pass0 + 1, (pass0 - first) / pcap, pass_last == last, row);
      __syncthreads();
    }
  }
}

#define DECODE_W 8
#define BW_LDS_BYTES (160 * 1024 - 256)   // a compute unit's LDS less the kernels' few static words
#define DECODE_W_MANY 4          // waves a workgroup where there are two workgroups or more for every compute unit: two of
                                 // these share a compute unit, and a token's first keys do not wait for a whole
                                 // generation of eight-wave workgroups before it (16 requests of 32 heads: 2.61 -> 2.52 ms
                                 // a step at 2,048-token contexts, 1.76 -> 1.69 at 512)
#define DECODE_MANY 257          // that many workgroups: more than there are compute units
#define DECODE_MANY_LONG 1024    // heads of 128 or more in a cache laid out for long contexts (more than 80 partitions a
                                 // request): eight waves' loads in flight are worth more there up to this many (64
                                 // requests of 8 heads of 128 at 8,192 tokens: 16.3 ms a step against 16.5)

// How a decode launch over ``num_tiles`` tiles is split: workgroups per tile (1 = no split) and
// the partitions a tile's scratch must hold.  Depends on nothing that changes from step to step.
static void decode_split_shape(int num_tiles, int items, int table_stride, int page_size, int& nsplit, int& max_parts) {
  max_parts = (table_stride * page_size + ATT_PART - 1) / ATT_PART + 1;
  const int rounds = (max_parts + DECODE_W - 1) / DECODE_W;
  const int wgs = num_tiles * items;
  nsplit = wgs >= 256 ? 1 : 256 / wgs;
  if (nsplit > rounds) nsplit = rounds;
  if (nsplit < 1) nsplit = 1;
}

template <int HD>
static int launch_attention(const AttnBf16Args& a, int decode, float* scratch, size_t scratch_floats, int* counters,
                            int num_counters, hipStream_t s) {
  const int items = a.kv_heads * a.nsub;
  if (decode) {
    constexpr int W = DECODE_W, WM = DECODE_W_MANY;
    const size_t cell = (size_t)a.hpt * (HD + 2) * sizeof(float);
    // LDS: the partials of ``pcap`` partitions (what fits 48 KB, at least one a wave) and what the fold keeps beside them
    auto shape = [&](int waves, int& pcap) {
      pcap = (int)((48 * 1024) / cell);
      pcap = pcap < waves ? waves : (pcap > 256 ? 256 : pcap);
      return FoldLds::bytes(pcap, a.hpt, HD);
    };
    int pcap;
    size_t lds_bytes = shape(W, pcap);
    int nsplit, max_parts;
    decode_split_shape(a.num_tiles, items, a.table_stride, a.page_size, nsplit, max_parts);
    if (scratch == nullptr || counters == nullptr) nsplit = 1;
    bool few_waves = nsplit == 1 && a.num_tiles * items >= ((HD >= 128 && max_parts > 80) ? DECODE_MANY_LONG : DECODE_MANY);
    if (lds_bytes > BW_LDS_BYTES) {                // sixteen heads of 256 a workgroup: only four waves' partials fit
      few_waves = true;
      nsplit = 1;
    }
    if (few_waves) lds_bytes = shape(WM, pcap);
    if (lds_bytes > BW_LDS_BYTES) return -8;
    // more than 64 KB of dynamic LDS has to be asked for once per kernel
    static bool allowed[3] = {false, false, false};
    const int variant = nsplit > 1 ? 0 : (few_waves ? 1 : 2);
    if (lds_bytes > 48 * 1024 && !allowed[variant]) {
      const void* fn = variant == 0 ? (const void*)attention_decode_kernel<HD, W, true>
                     : variant == 1 ? (const void*)attention_decode_kernel<HD, WM, false>
                                    : (const void*)attention_decode_kernel<HD, W, false>;
      if (hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, BW_LDS_BYTES) != hipSuccess) return -8;
      allowed[variant] = true;
    }
    if (nsplit > 1) {
      if (scratch_floats < (size_t)a.num_tiles * items * max_parts * a.hpt * (HD + 2) || num_counters < a.num_tiles * items)
        return -6;
      hipLaunchKernelGGL((attention_decode_kernel<HD, W, true>), dim3(a.num_tiles, items, nsplit), dim3(64 * W), lds_bytes, s,
                         a, pcap, scratch, counters, max_parts);
    } else if (few_waves) {                        // (the partials are folded in partition order whatever the waves: the same bits)
      hipLaunchKernelGGL((attention_decode_kernel<HD, WM, false>), dim3(a.num_tiles, items), dim3(64 * WM), lds_bytes, s, a,
                         pcap, nullptr, nullptr, 0);
    } else {
      hipLaunchKernelGGL((attention_decode_kernel<HD, W, false>), dim3(a.num_tiles, items), dim3(64 * W), lds_bytes, s, a,
                         pcap, nullptr, nullptr, 0);
    }
  } else {
    using S = FoldShape<HD>;
    constexpr int lds_bytes = S::NBUF * S::BYTES;
    static bool allowed = false;                   // more than 64 KB of dynamic LDS has to be asked for once
    if (!allowed && lds_bytes > 48 * 1024) {
      (void)hipFuncSetAttribute((const void*)attention_fold_kernel<HD>, hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes);
      allowed = true;
    }
    const int groups = (a.num_tiles + S::GROUP - 1) / S::GROUP;
    hipLaunchKernelGGL((attention_fold_kernel<HD>), dim3(groups * items), dim3(64 * S::NW), lds_bytes, s, a, groups, items);
  }
  return 0;
}

extern "C" int bw_attention_fold_group_tiles(int head_dim) { return FOLD_NW(head_dim) * FOLD_QT(head_dim); }

// What a split decode launch needs beside its inputs: floats of scratch and counters (int32, zero
// before the first launch; every launch leaves them zero).  Both 0: the launch is not split.
extern "C" int bw_attention_decode_scratch(int num_tiles, int heads, int kv_heads, int head_dim, int table_stride,
                                           int page_size, long long* scratch_floats, int* counters) {
  *scratch_floats = 0;
  *counters = 0;
  if (num_tiles <= 0 || kv_heads <= 0 || heads % kv_heads || page_size <= 0) return -2;
  const int group = heads / kv_heads;
  const int hpt = group < 16 ? group : 16, nsub = (group + hpt - 1) / hpt;
  int nsplit, max_parts;
  decode_split_shape(num_tiles, kv_heads * nsub, table_stride, page_size, nsplit, max_parts);
  if (nsplit > 1) {
    *scratch_floats = (long long)num_tiles * kv_heads * nsub * max_parts * hpt * (head_dim + 2);
    *counters = num_tiles * kv_heads * nsub;
  }
  return 0;
}

extern "C" int bw_attention_bf16(const void* q, int q_stride, const int32_t* positions, const int32_t* block_table,
                                 int table_stride, const int32_t* tiles, int num_tiles, const void* k_cache,
                                 const void* v_cache, int num_pages, void* out, int out_stride, int heads,
                                 int kv_heads, int head_dim, int page_size, int window, float scale, int decode,
                                 float* scratch, long long scratch_floats, int32_t* counters, int num_counters,
                                 void* stream) {
  if (num_tiles <= 0) return 0;
  if (num_pages <= 0) return -2;
  if (kv_heads <= 0 || heads % kv_heads) return -2;
  if (page_size < 4 || (page_size & (page_size - 1)) || page_size > ATT_PART) return -5;  // 4-key loads stay inside a page
  if ((q_stride % 8) || (out_stride % 4)) return -3;
  if (reinterpret_cast<uintptr_t>(scratch) & 7) return -3;      // partials travel in 8-byte words
  const int group = heads / kv_heads;
  AttnBf16Args a;
  a.q = (const bf16_t*)q; a.positions = positions; a.block_table = block_table; a.tiles = tiles;
  a.k_cache = (const bf16_t*)k_cache; a.v_cache = (const bf16_t*)v_cache; a.out = (bf16_t*)out;
  a.heads = heads; a.kv_heads = kv_heads; a.page_size = page_size; a.table_stride = table_stride;
  a.page_shift = __builtin_ctz((unsigned)page_size);
  a.num_pages = num_pages;
  a.q_stride = q_stride; a.out_stride = out_stride; a.window = window;
  a.hpt = group < 16 ? group : 16;
  a.nsub = (group + a.hpt - 1) / a.hpt;
  a.num_tiles = num_tiles;
  if (!(scale > 0.0f)) return -2;                // the maximum is taken before the scaling
  a.scale_log2 = scale * 1.44269504088896340736f;
  if (kv_heads * a.nsub > 65535) return -2;
  if ((long long)kv_heads * page_size * head_dim * 2 >= (1ll << 31)) return -2;    // a page's bytes as a 32-bit factor
  hipStream_t s = (hipStream_t)stream;
  int rc = 0;
#define BW_CASE(HD) case HD: rc = launch_attention<HD>(a, decode, scratch, (size_t)scratch_floats, counters, num_counters, s); break;
  switch (head_dim) {
    BW_CASE(16) BW_CASE(32) BW_CASE(48) BW_CASE(64) BW_CASE(80) BW_CASE(96) BW_CASE(112) BW_CASE(128)
    BW_CASE(160) BW_CASE(192) BW_CASE(224) BW_CASE(256)
    default: return -4;
  }
#undef BW_CASE
  if (rc) return rc;
  return BW_LAUNCH_CHECK();
}
