// True 32-bit causal attention over the paged cache, in the reference's operation order
// (src/kernels.cpp:312-368): for the query at position p of head h,
//   pass 1: s_j = dot_canonical(q, K_j) * scale for j = lo..p, mx = max s_j;
//   pass 2: for j = lo..p in key order: e = exp(s_j - mx); sum += e; acc[d] = fma(e, V_j[d], acc[d]);
//   out[d] = acc[d] * (1/sum).
// dot_canonical is the 16-chain split with the fixed tree (src/kernels.cpp:57-64, :86-101).
// lo is 0, or p-window+1 for a windowed cache.  A workgroup of 256 threads per (row, head): in pass 1 each
// thread takes keys j = lo+t, lo+t+256, ...; in pass 2 the threads recompute the scores of 256 keys at a
// time (the same deterministic function, so the same bits), park e_j in LDS, and then thread d walks
// the 256 keys in order for its own d.  The same code runs for a row of a prompt portion and for a
// decoded token, so the bits cannot differ.
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
};

template <int HD>
__device__ __forceinline__ float dot_canonical(const float* __restrict__ q_lds, const float* __restrict__ k) {
  float lane[16];
#pragma unroll
  for (int i = 0; i < 16; ++i) lane[i] = 0.0f;
#pragma unroll
  for (int c = 0; c < HD / 16; ++c) {
    float kv[16];
#pragma unroll
    for (int v4 = 0; v4 < 4; ++v4) {
      const f32x4 t = *reinterpret_cast<const f32x4*>(k + c * 16 + v4 * 4);
      kv[v4 * 4 + 0] = t[0]; kv[v4 * 4 + 1] = t[1]; kv[v4 * 4 + 2] = t[2]; kv[v4 * 4 + 3] = t[3];
    }
#pragma unroll
    for (int i = 0; i < 16; ++i) lane[i] = fmaf(q_lds[c * 16 + i], kv[i], lane[i]);
  }
  float s8[8], s4[4];
#pragma unroll
  for (int i = 0; i < 8; ++i) s8[i] = lane[i] + lane[i + 8];
#pragma unroll
  for (int i = 0; i < 4; ++i) s4[i] = s8[i] + s8[i + 4];
  const float a = s4[0] + s4[2];
  const float b = s4[1] + s4[3];
  return a + b;
}

// Element offset of key j of this kv head in either cache.
__device__ __forceinline__ size_t key_offset(const AttnF32Args& a, const int32_t* table, int j, size_t head_off,
                                             size_t page_stride, int hd) {
  const int page = a.page_shift >= 0 ? j >> a.page_shift : j / a.page_size;
  const int slot = a.page_shift >= 0 ? j & (a.page_size - 1) : j % a.page_size;
  return (size_t)table[page] * page_stride + head_off + (size_t)slot * hd;
}

#define ATT32_THREADS 256

// Keys of a chunk of pass 2: as many as 32 KB of value rows hold, at most one a thread.
template <int HD>
struct Att32Shape {
  static constexpr int T = ATT32_THREADS;
  static constexpr int KC = (8192 / HD) < T ? (8192 / HD) : T;
  static constexpr int SEGS = HD / 4;                              // 16-byte pieces of a key's row
  static constexpr int VJ = (KC * SEGS + T - 1) / T;               // pieces of a chunk's value rows a thread
  static constexpr int LDS_BYTES = 2 * KC * HD * (int)sizeof(float);
};

template <int HD>
__global__ __launch_bounds__(ATT32_THREADS) void attention_f32_kernel(AttnF32Args a) {
  using S = Att32Shape<HD>;
  constexpr int T = S::T, KC = S::KC, SEGS = S::SEGS, VJ = S::VJ;
  extern __shared__ __attribute__((aligned(16))) float v_lds[];    // [2][KC][HD]: value rows of a chunk of keys
  __shared__ float q_lds[HD];
  __shared__ float e_lds[2][KC];
  __shared__ float red[T / 64];
  const int row = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
  const int pos = a.positions[row];
  if (pos < 0) return;
  const int kvh = h / (a.heads / a.kv_heads);
  const int32_t* table = a.block_table + (size_t)a.row_seq[row] * a.table_stride;
  const float* qh = a.q + (size_t)row * a.q_stride + (size_t)h * HD;
  for (int i = tid; i < HD; i += T) q_lds[i] = qh[i];
  __syncthreads();
  const int lo = (a.window > 0 && pos - a.window + 1 > 0) ? pos - a.window + 1 : 0;
  const size_t head_off = (size_t)kvh * a.page_size * HD;
  const size_t page_stride = (size_t)a.kv_heads * a.page_size * HD;

  // pass 1: the maximum (exact whatever the order), a key a thread at a time
  float mx = -INFINITY;
  for (int j = lo + tid; j <= pos; j += T)
    mx = fmaxf(mx, dot_canonical<HD>(q_lds, a.k_cache + key_offset(a, table, j, head_off, page_stride, HD)) * a.scale);
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
      const int c = tid + T * i, j = j0 + c / SEGS;
      vreg[i] = (f32x4){0.f, 0.f, 0.f, 0.f};
      if (c < KC * SEGS && j <= pos)
        vreg[i] = *reinterpret_cast<const f32x4*>(a.v_cache + key_offset(a, table, j, head_off, page_stride, HD) + 4 * (c % SEGS));
    }
  };
  auto stash = [&](int buf) {
#pragma unroll
    for (int i = 0; i < VJ; ++i) {
      const int c = tid + T * i;                           // piece c = key c / SEGS, elements 4 * (c % SEGS)..: float 4c of the buffer
      if (c < KC * SEGS) *reinterpret_cast<f32x4*>(v_lds + buf * KC * HD + 4 * c) = vreg[i];
    }
  };
  auto park = [&](int j0, int buf) {
    const int t = tid - (T - KC);
    if (t < 0) return;
    const int j = j0 + t;
    float e = 0.0f;
    if (j <= pos)
      e = expf(dot_canonical<HD>(q_lds, a.k_cache + key_offset(a, table, j, head_off, page_stride, HD)) * a.scale - mx);
    e_lds[buf][t] = e;
  };
  float acc = 0.0f, sum = 0.0f;
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
    if (tid < HD) {
      const int cnt = (pos - j0 + 1) < KC ? (pos - j0 + 1) : KC;
      const float* vd = v_lds + buf * KC * HD + tid;
      const float* ed = e_lds[buf];
#pragma unroll 8
      for (int jj = 0; jj < cnt; ++jj) {
        const float ej = ed[jj];
        sum += ej;
        acc = fmaf(ej, vd[jj * HD], acc);
      }
    }
    if (more) stash(buf ^ 1);
    __syncthreads();
    buf ^= 1;
  }
  if (tid < HD) a.out[(size_t)row * a.out_stride + (size_t)h * HD + tid] = acc * (1.0f / sum);
}

template <int HD>
static void launch_attention_f32(const AttnF32Args& a, dim3 grid, hipStream_t s) {
  static bool allowed = false;                         // 64 KB of dynamic LDS has to be asked for once
  if (!allowed) {
    (void)hipFuncSetAttribute((const void*)attention_f32_kernel<HD>, hipFuncAttributeMaxDynamicSharedMemorySize,
                              Att32Shape<HD>::LDS_BYTES);
    allowed = true;
  }
  hipLaunchKernelGGL(attention_f32_kernel<HD>, grid, dim3(ATT32_THREADS), Att32Shape<HD>::LDS_BYTES, s, a);
}

extern "C" int bw_attention_f32(const float* q, int q_stride, const int32_t* positions, const int32_t* row_seq,
                                const int32_t* block_table, int table_stride, const float* k_cache,
                                const float* v_cache, float* out, int out_stride, int rows, int heads,
                                int kv_heads, int head_dim, int page_size, int window, float scale, void* stream) {
  if (rows <= 0) return 0;
  if (kv_heads <= 0 || heads % kv_heads || heads > 65535) return -2;
  AttnF32Args a{q, positions, row_seq, block_table, k_cache, v_cache, out, rows, heads, kv_heads, head_dim,
                page_size, table_stride, q_stride, out_stride, window, scale,
                (page_size & (page_size - 1)) == 0 ? __builtin_ctz((unsigned)page_size) : -1};
  dim3 grid(rows, heads);
  hipStream_t s = (hipStream_t)stream;
#define BW_CASE(HD) case HD: launch_attention_f32<HD>(a, grid, s); break;
  switch (head_dim) {
    BW_CASE(16) BW_CASE(32) BW_CASE(48) BW_CASE(64) BW_CASE(80) BW_CASE(96) BW_CASE(112) BW_CASE(128)
    BW_CASE(160) BW_CASE(192) BW_CASE(224) BW_CASE(256)
    default: return -4;  // head size not compiled in
  }
#undef BW_CASE
  return BW_LAUNCH_CHECK();
}
