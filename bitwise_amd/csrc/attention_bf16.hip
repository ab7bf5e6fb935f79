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
// decode kernel gives every partition a wave of its own and performs the same fold from LDS
// in partition order, so both routes give the same bits, and a query's result depends on
// nothing but its own row, its position and the cache contents at positions it may see.
//
// Layout: S^T = K Q^T is computed (keys are MFMA rows, queries are columns), so the
// probabilities come out of the accumulator in exactly the lane layout that the second
// product O^T = V^T P^T needs for its B operand; no LDS is used.  K pages are
// [kv_head][slot][hd]; V pages are transposed, [kv_head][hd][slot], so that an A-operand
// lane reads 4 consecutive keys of one d with one 8-byte load.
//
// Work shapes: in the fold kernel a wave owns up to QT tiles (QT*16 queries of one sequence
// and kv head) and reuses every loaded K and V operand for all of them, prefetching the next
// partition's keys while it works; in the decode kernel a workgroup owns one tile (one token,
// the heads of one kv head) and each of its waves one partition at a time, all loads of a
// partition issued at once.
#include "common.h"
#include "api.h"

#define ATT_PART 64

struct AttnBf16Args {
  const bf16_t* q;            // [rows, q_stride]
  const int32_t* positions;   // [rows]; negative = padding row
  const int32_t* block_table; // [seqs, table_stride]
  const int32_t* tiles;       // [tiles][4] = row0, tokens, seq, 0; null: tile t is row t of sequence t
  const bf16_t* k_cache;
  const bf16_t* v_cache;
  bf16_t* out;                // [rows, out_stride]
  int heads, kv_heads, page_size, table_stride, q_stride, out_stride, window, hpt, nsub, num_tiles;
  float scale;
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
  }
#pragma unroll
  for (int off = 8; off >= 1; off >>= 1) {
    kmax = max(kmax, __shfl_xor(kmax, off, BW_WAVE));
    kmin = min(kmin, __shfl_xor(kmin, off, BW_WAVE));
  }
  gc.kmax = kmax;
  gc.kmin = kmin;
  gc.table = a.block_table + (size_t)seq * a.table_stride;
  if (kmax < 0) return false;
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

template <int HD>
struct KFrags {
  u32x4 k[4][(HD + 31) / 32];
};
// Keys of one partition as A operands: lane (r, g) feeds key 16u + r, elements 32ks + 8g .. +7.
template <int HD>
__device__ __forceinline__ void load_keys(const AttnBf16Args& a, const GroupCtx& gc, int part, KFrags<HD>& kf) {
  constexpr int KS = (HD + 31) / 32;
  const int key0 = part * ATT_PART;
  const size_t kpage = (size_t)a.kv_heads * a.page_size * HD;
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    const int key_r = key0 + 16 * u + gc.r;
    const bool k_ok = key_r <= gc.kmax && key_r >= gc.kmin;
    // the table entry is read whether or not the key is live (index clamped into the row), so
    // that this load does not have to wait for the positions
    const int pidx = key_r / a.page_size;
    const int page = gc.table[pidx < a.table_stride ? pidx : a.table_stride - 1];
    const bf16_t* kp = a.k_cache + (size_t)page * kpage + ((size_t)gc.kvh * a.page_size + key_r % a.page_size) * HD;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const int d0 = 32 * ks + 8 * gc.g;
      u32x4 v = {0u, 0u, 0u, 0u};
      if (k_ok && d0 < HD) v = *reinterpret_cast<const u32x4*>(kp + d0);
      kf.k[u][ks] = v;
    }
  }
}

// Values of one partition as A operands of O^T = V^T P^T: lane (r, g) feeds d = 16dt + r and, for
// the 32-key step w, keys 32w + 4g .. +3 and 32w + 16 + 4g .. +3 (the order in which the
// probabilities sit in the score accumulators).  Keys no query of the group may see hold stale
// data (never written, or given back): they are zeroed, so that 0 * garbage cannot make a NaN.
template <int HD, int DT0, int NDT>
__device__ __forceinline__ void load_values_range(const AttnBf16Args& a, const GroupCtx& gc, int part,
                                                  u32x4 (&out)[NDT][2]) {
  const int key0 = part * ATT_PART;
  const size_t vpage = (size_t)a.kv_heads * HD * a.page_size;
#pragma unroll
  for (int w = 0; w < 2; ++w)
#pragma unroll
    for (int hseg = 0; hseg < 2; ++hseg) {
      const int kA = key0 + 32 * w + 16 * hseg + 4 * gc.g;   // 4 consecutive keys
      const bool ok = kA <= gc.kmax && kA + 3 >= gc.kmin;
      const int pidx = kA / a.page_size;
      const int page = gc.table[pidx < a.table_stride ? pidx : a.table_stride - 1];
      const bf16_t* vp = a.v_cache + (size_t)page * vpage + (size_t)gc.kvh * HD * a.page_size + kA % a.page_size;
      uint32_t m0 = ok ? 0xffffffffu : 0u, m1 = m0;
      const int over = kA + 3 - gc.kmax;                      // keys kA+4-over .. kA+3 are unwritten
      if (over >= 1) m1 &= (over >= 2) ? 0u : 0x0000ffffu;
      if (over >= 3) m0 &= (over >= 4) ? 0u : 0x0000ffffu;
      const int under = gc.kmin - kA;                         // keys kA .. kA+under-1 are gone
      if (under >= 1) m0 &= (under >= 2) ? 0u : 0xffff0000u;
      if (under >= 3) m1 &= (under >= 4) ? 0u : 0xffff0000u;
#pragma unroll
      for (int dt = 0; dt < NDT; ++dt) {
        u32x2 v2 = {0u, 0u};
        if (ok) v2 = *reinterpret_cast<const u32x2*>(vp + (size_t)(16 * (DT0 + dt) + gc.r) * a.page_size);
        out[dt][w][2 * hseg] = v2[0] & m0;
        out[dt][w][2 * hseg + 1] = v2[1] & m1;
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
__device__ __forceinline__ void load_values(const AttnBf16Args& a, const GroupCtx& gc, int part, VFrags<HD>& vf) {
  if constexpr (VFrags<HD>::EARLY) load_values_range<HD, 0, HD / 16>(a, gc, part, vf.v);
}

template <int HD, int DT>
__device__ __forceinline__ void pv_step(const AttnBf16Args& a, const GroupCtx& gc, int part, const VFrags<HD>& vf,
                                        const u32x4 (&pf)[2], f32x4 (&o_p)[HD / 16]) {
  if constexpr (DT < HD / 16) {
    o_p[DT] = (f32x4){0.f, 0.f, 0.f, 0.f};
    if constexpr (VFrags<HD>::EARLY) {
#pragma unroll
      for (int w = 0; w < 2; ++w)
        o_p[DT] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(vf.v[DT][w]), as_bf16x8(pf[w]), o_p[DT], 0, 0, 0);
    } else {
      u32x4 v[1][2];
      load_values_range<HD, DT, 1>(a, gc, part, v);
#pragma unroll
      for (int w = 0; w < 2; ++w)
        o_p[DT] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(v[0][w]), as_bf16x8(pf[w]), o_p[DT], 0, 0, 0);
    }
    pv_step<HD, DT + 1>(a, gc, part, vf, pf, o_p);
  }
}

// One partition's partial for one tile: per column m_p, l_p (replicated over the 4 lane
// groups) and O_p[dt][i] = element d = 16dt + 4g + i of the column.
template <int HD>
__device__ __forceinline__ void partition_partial(const AttnBf16Args& a, const GroupCtx& gc, const TileCtx<HD>& t,
                                                  int part, const KFrags<HD>& kf, const VFrags<HD>& vf, float& m_p,
                                                  float& l_p, f32x4 (&o_p)[HD / 16]) {
  constexpr int KS = (HD + 31) / 32;
  const int key0 = part * ATT_PART;
  f32x4 st[4];
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    st[u] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
      st[u] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(kf.k[u][ks]), as_bf16x8(t.qf[ks]), st[u], 0, 0, 0);
  }
  // scale, mask, column maximum
  float mx = -INFINITY;
  bool vis[4][4];
#pragma unroll
  for (int u = 0; u < 4; ++u)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int key = key0 + 16 * u + 4 * gc.g + i;
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
  pv_step<HD, 0>(a, gc, part, vf, pf, o_p);
}

// The fold step, element by element; the combine kernel runs the same statements.
__device__ __forceinline__ void fold_scalars(float m, float m_p, float& mn, float& fa, float& fb) {
  mn = fmaxf(m, m_p);
  fa = fast_exp(m - mn);
  fb = fast_exp(m_p - mn);
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
  float mn, fa, fb;
  fold_scalars(m, m_p, mn, fa, fb);
  l = fmaf(l, fa, l_p * fb);
#pragma unroll
  for (int dt = 0; dt < NT; ++dt)
#pragma unroll
    for (int i = 0; i < 4; ++i) o[dt][i] = fmaf(o[dt][i], fa, o_p[dt][i] * fb);
  m = mn;
}

// Route 1: one wave folds all partitions of its group of QT tiles.
template <int HD, int QT>
__global__ __launch_bounds__(64) void attention_fold_kernel(AttnBf16Args a) {
  constexpr int NT = HD / 16;
  GroupCtx gc;
  TileCtx<HD> tc[QT];
  if (!group_setup<HD, QT>(a, blockIdx.x * QT, blockIdx.y, gc, tc)) return;
  float m[QT], l[QT];
  f32x4 o[QT][NT];
#pragma unroll
  for (int t = 0; t < QT; ++t) {
    m[t] = -INFINITY;
    l[t] = 0.0f;
#pragma unroll
    for (int dt = 0; dt < NT; ++dt) o[t][dt] = (f32x4){0.f, 0.f, 0.f, 0.f};
  }
  const int first = gc.kmin / ATT_PART, last = gc.kmax / ATT_PART;
  constexpr bool PREFETCH = HD <= 128;      // the next partition's keys are loaded while this one is worked on
  KFrags<HD> kf, kf_next;
  VFrags<HD> vf;
  if constexpr (PREFETCH) load_keys<HD>(a, gc, first, kf);
  for (int part = first; part <= last; ++part) {
    if constexpr (!PREFETCH) load_keys<HD>(a, gc, part, kf);
    load_values<HD>(a, gc, part, vf);
    if constexpr (PREFETCH) {
      if (part < last) load_keys<HD>(a, gc, part + 1, kf_next);
    }
#pragma unroll
    for (int t = 0; t < QT; ++t) {
      float m_p, l_p;
      f32x4 o_p[NT];
      partition_partial<HD>(a, gc, tc[t], part, kf, vf, m_p, l_p, o_p);
      fold<NT>(m[t], l[t], o[t], m_p, l_p, o_p);
    }
    if constexpr (PREFETCH) kf = kf_next;
  }
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
template <int HD, int W>
__global__ __launch_bounds__(64 * W) void attention_decode_kernel(AttnBf16Args a, int pcap) {
  constexpr int NT = HD / 16;
  constexpr int THREADS = 64 * W;
  constexpr int EPT = (16 * HD + THREADS - 1) / THREADS;   // output elements per thread at most (16 live columns)
  constexpr int CELL = HD + 2;                              // m, l, then hd values
  constexpr bool PREFETCH = HD <= 64;
  extern __shared__ float parts[];                          // [pcap][hpt][CELL]
  GroupCtx gc;
  TileCtx<HD> tc[1];
  if (!group_setup<HD, 1>(a, blockIdx.x, blockIdx.y, gc, tc)) return;   // uniform over the workgroup
  const int wave = threadIdx.x >> 6;
  const int first = gc.kmin / ATT_PART, last = gc.kmax / ATT_PART;
  const int elems = a.hpt * HD;
  float m[EPT], l[EPT], o[EPT];
#pragma unroll
  for (int j = 0; j < EPT; ++j) {
    m[j] = -INFINITY;
    l[j] = 0.0f;
    o[j] = 0.0f;
  }
  for (int pass0 = first; pass0 <= last; pass0 += pcap) {
    const int pass_last = (last - pass0) < pcap ? last : pass0 + pcap - 1;
    KFrags<HD> kf, kf_next;
    VFrags<HD> vf;
    int part = pass0 + wave;
    if constexpr (PREFETCH) {
      if (part <= pass_last) load_keys<HD>(a, gc, part, kf);
    }
    for (; part <= pass_last; part += W) {
      if constexpr (!PREFETCH) load_keys<HD>(a, gc, part, kf);
      load_values<HD>(a, gc, part, vf);
      if constexpr (PREFETCH) {
        if (part + W <= pass_last) load_keys<HD>(a, gc, part + W, kf_next);
      }
      float m_p, l_p;
      f32x4 o_p[NT];
      partition_partial<HD>(a, gc, tc[0], part, kf, vf, m_p, l_p, o_p);
      if (gc.r < a.hpt) {
        float* cell = parts + ((size_t)(part - pass0) * a.hpt + gc.r) * CELL;
        if (gc.g == 0) {
          cell[0] = m_p;
          cell[1] = l_p;
        }
#pragma unroll
        for (int dt = 0; dt < NT; ++dt)
#pragma unroll
          for (int i = 0; i < 4; ++i) cell[2 + 16 * dt + 4 * gc.g + i] = o_p[dt][i];
      }
      if constexpr (PREFETCH) kf = kf_next;
    }
    __syncthreads();
    const int count = pass_last - pass0 + 1;
#pragma unroll
    for (int j = 0; j < EPT; ++j) {
      const int e = threadIdx.x + j * THREADS;
      if (e >= elems) continue;
      const int col = e / HD, d = e % HD;
      for (int wv = 0; wv < count; ++wv) {
        const float* cell = parts + ((size_t)wv * a.hpt + col) * CELL;
        const float m_p = cell[0], l_p = cell[1], o_p = cell[2 + d];
        if (m_p == -INFINITY) continue;
        if (m[j] == -INFINITY) {
          m[j] = m_p;
          l[j] = l_p;
          o[j] = o_p;
          continue;
        }
        float mn, fa, fb;
        fold_scalars(m[j], m_p, mn, fa, fb);
        l[j] = fmaf(l[j], fa, l_p * fb);
        o[j] = fmaf(o[j], fa, o_p * fb);
        m[j] = mn;
      }
    }
    __syncthreads();
  }
  // columns of a one-token tile: column c is head sub*hpt + c of the kv head's group
  const int group = a.heads / a.kv_heads;
  const int row = a.tiles != nullptr ? a.tiles[blockIdx.x * 4] : blockIdx.x;
#pragma unroll
  for (int j = 0; j < EPT; ++j) {
    const int e = threadIdx.x + j * THREADS;
    if (e >= elems) continue;
    const int col = e / HD, d = e % HD;
    if (gc.sub * a.hpt + col >= group) continue;
    const float inv = 1.0f / l[j];
    a.out[(size_t)row * a.out_stride + (size_t)(gc.kvh * group + gc.sub * a.hpt + col) * HD + d] = f32_to_bf16(o[j] * inv);
  }
}

template <int HD>
static void launch_attention(const AttnBf16Args& a, int decode, hipStream_t s) {
  const int items = a.kv_heads * a.nsub;
  if (decode) {
    constexpr int W = 8;
    const size_t cell = (size_t)a.hpt * (HD + 2) * sizeof(float);
    int pcap = (int)((48 * 1024) / cell);          // partitions whose partials fit 48 KB of LDS
    pcap = pcap < W ? W : (pcap > 256 ? 256 : pcap);
    hipLaunchKernelGGL((attention_decode_kernel<HD, W>), dim3(a.num_tiles, items), dim3(64 * W), pcap * cell, s, a, pcap);
  } else {
    constexpr int QT = HD <= 64 ? 4 : (HD <= 128 ? 2 : 1);
    hipLaunchKernelGGL((attention_fold_kernel<HD, QT>), dim3((a.num_tiles + QT - 1) / QT, items), dim3(64), 0, s, a);
  }
}

extern "C" int bw_attention_bf16(const void* q, int q_stride, const int32_t* positions, const int32_t* block_table,
                                 int table_stride, const int32_t* tiles, int num_tiles, const void* k_cache,
                                 const void* v_cache, void* out, int out_stride, int heads, int kv_heads,
                                 int head_dim, int page_size, int window, float scale, int decode, void* stream) {
  if (num_tiles <= 0) return 0;
  if (kv_heads <= 0 || heads % kv_heads) return -2;
  if (page_size < 4 || (page_size & (page_size - 1)) || page_size > ATT_PART) return -5;  // 4-key loads stay inside a page
  if ((q_stride % 8) || (out_stride % 4)) return -3;
  const int group = heads / kv_heads;
  AttnBf16Args a;
  a.q = (const bf16_t*)q; a.positions = positions; a.block_table = block_table; a.tiles = tiles;
  a.k_cache = (const bf16_t*)k_cache; a.v_cache = (const bf16_t*)v_cache; a.out = (bf16_t*)out;
  a.heads = heads; a.kv_heads = kv_heads; a.page_size = page_size; a.table_stride = table_stride;
  a.q_stride = q_stride; a.out_stride = out_stride; a.window = window;
  a.hpt = group < 16 ? group : 16;
  a.nsub = (group + a.hpt - 1) / a.hpt;
  a.num_tiles = num_tiles;
  a.scale = scale;
  if (kv_heads * a.nsub > 65535) return -2;
  hipStream_t s = (hipStream_t)stream;
#define BW_CASE(HD) case HD: launch_attention<HD>(a, decode, s); break;
  switch (head_dim) {
    BW_CASE(16) BW_CASE(32) BW_CASE(48) BW_CASE(64) BW_CASE(80) BW_CASE(96) BW_CASE(112) BW_CASE(128)
    BW_CASE(160) BW_CASE(192) BW_CASE(224) BW_CASE(256)
    default: return -4;
  }
#undef BW_CASE
  return BW_LAUNCH_CHECK();
}
