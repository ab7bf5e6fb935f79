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

template <int HD>
__global__ __launch_bounds__(ATT32_THREADS) void attention_f32_kernel(AttnF32Args a) {
  constexpr int T = ATT32_THREADS;
  __shared__ float q_lds[HD];
  __shared__ float e_lds[2][T];
  __shared__ unsigned long long off_lds[2][T];
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

  // pass 2: the threads compute e_j of T keys at a time (the same deterministic function of the key as in pass
  // 1) and park them with the keys' cache offsets; thread d < HD then walks the T keys in order for element d.
  // The next T keys' e_j are computed before the walk, into the other buffer: one barrier per T keys.
  auto park = [&](int j0, int buf) {
    const int j = j0 + tid;
    float e = 0.0f;
    size_t off = 0;
    if (j <= pos) {
      off = key_offset(a, table, j, head_off, page_stride, HD);
      e = expf(dot_canonical<HD>(q_lds, a.k_cache + off) * a.scale - mx);
    }
    e_lds[buf][tid] = e;
    off_lds[buf][tid] = off;
  };
  float acc = 0.0f, sum = 0.0f;
  park(lo, 0);
  __syncthreads();
  int buf = 0;
  for (int j0 = lo; j0 <= pos; j0 += T) {
    if (j0 + T <= pos) park(j0 + T, buf ^ 1);
    if (tid < HD) {
      const int cnt = (pos - j0 + 1) < T ? (pos - j0 + 1) : T;
      const float* vd = a.v_cache + tid;
#pragma unroll 8
      for (int jj = 0; jj < cnt; ++jj) {
        const float ej = e_lds[buf][jj];
        sum += ej;
        acc = fmaf(ej, vd[off_lds[buf][jj]], acc);
      }
    }
    __syncthreads();
    buf ^= 1;
  }
  if (tid < HD) a.out[(size_t)row * a.out_stride + (size_t)h * HD + tid] = acc * (1.0f / sum);
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
  dim3 grid(rows, heads), block(ATT32_THREADS);
  hipStream_t s = (hipStream_t)stream;
#define BW_CASE(HD) case HD: hipLaunchKernelGGL(attention_f32_kernel<HD>, grid, block, 0, s, a); break;
  switch (head_dim) {
    BW_CASE(16) BW_CASE(32) BW_CASE(48) BW_CASE(64) BW_CASE(80) BW_CASE(96) BW_CASE(112) BW_CASE(128)
    BW_CASE(160) BW_CASE(192) BW_CASE(224) BW_CASE(256)
    default: return -4;  // head size not compiled in
  }
#undef BW_CASE
  return BW_LAUNCH_CHECK();
}
