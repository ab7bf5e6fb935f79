// True 32-bit causal attention over the paged cache, in the reference's operation order
// (src/kernels.cpp:312-368): for the query at position p of head h,
//   pass 1: s_j = dot_canonical(q, K_j) * scale for j = lo..p, mx = max s_j;
//   pass 2: for j = lo..p in key order: e = exp(s_j - mx); sum += e; acc[d] = fma(e, V_j[d], acc[d]);
//   out[d] = acc[d] * (1/sum).
// dot_canonical is the 16-chain split with the fixed tree (src/kernels.cpp:57-64, :86-101).
// lo is 0, or p-window+1 for a windowed cache.  One wave per (row, head): in pass 1 each
// lane takes keys j = lo+lane, lo+lane+64, ...; in pass 2 the lanes recompute the scores of
// 64 keys at a time (the same deterministic function, so the same bits), park e_j in LDS,
// and then every lane walks the 64 keys in order for its own d.  The same code runs for a
// row of a prompt portion and for a decoded token, so the bits cannot differ.
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

template <int HD>
__global__ __launch_bounds__(64) void attention_f32_kernel(AttnF32Args a) {
  __shared__ float q_lds[HD];
  __shared__ float e_lds[64];
  const int row = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const int pos = a.positions[row];
  if (pos < 0) return;
  const int kvh = h / (a.heads / a.kv_heads);
  const int32_t* table = a.block_table + (size_t)a.row_seq[row] * a.table_stride;
  const float* qh = a.q + (size_t)row * a.q_stride + (size_t)h * HD;
  for (int i = lane; i < HD; i += 64) q_lds[i] = qh[i];
  __syncthreads();
  const int lo = (a.window > 0 && pos - a.window + 1 > 0) ? pos - a.window + 1 : 0;
  const size_t head_off = (size_t)kvh * a.page_size * HD;
  const size_t page_stride = (size_t)a.kv_heads * a.page_size * HD;

  float mx = -INFINITY;
  for (int j = lo + lane; j <= pos; j += 64) {
    const float* k = a.k_cache + (size_t)table[j / a.page_size] * page_stride + head_off + (size_t)(j % a.page_size) * HD;
    mx = fmaxf(mx, dot_canonical<HD>(q_lds, k) * a.scale);
  }
  mx = wave_max(mx);

  constexpr int DPL = (HD + 63) / 64;  // output elements per lane
  float acc[DPL];
#pragma unroll
  for (int t = 0; t < DPL; ++t) acc[t] = 0.0f;
  float sum = 0.0f;
  for (int j0 = lo; j0 <= pos; j0 += 64) {
    const int j = j0 + lane;
    float e = 0.0f;
    if (j <= pos) {
      const float* k = a.k_cache + (size_t)table[j / a.page_size] * page_stride + head_off + (size_t)(j % a.page_size) * HD;
      e = expf(dot_canonical<HD>(q_lds, k) * a.scale - mx);
    }
    __syncthreads();
    e_lds[lane] = e;
    __syncthreads();
    const int cnt = (pos - j0 + 1) < 64 ? (pos - j0 + 1) : 64;
    for (int jj = 0; jj < cnt; ++jj) {
      const int key = j0 + jj;
      const float ej = e_lds[jj];
      sum += ej;
      const float* v = a.v_cache + (size_t)table[key / a.page_size] * page_stride + head_off + (size_t)(key % a.page_size) * HD;
#pragma unroll
      for (int t = 0; t < DPL; ++t) {
        const int d = lane + 64 * t;
        if (d < HD) acc[t] = fmaf(ej, v[d], acc[t]);
      }
    }
  }
  const float inv = 1.0f / sum;
  float* o = a.out + (size_t)row * a.out_stride + (size_t)h * HD;
#pragma unroll
  for (int t = 0; t < DPL; ++t) {
    const int d = lane + 64 * t;
    if (d < HD) o[d] = acc[t] * inv;
  }
}

extern "C" int bw_attention_f32(const float* q, int q_stride, const int32_t* positions, const int32_t* row_seq,
                                const int32_t* block_table, int table_stride, const float* k_cache,
                                const float* v_cache, float* out, int out_stride, int rows, int heads,
                                int kv_heads, int head_dim, int page_size, int window, float scale, void* stream) {
  if (rows <= 0) return 0;
  if (kv_heads <= 0 || heads % kv_heads || heads > 65535) return -2;
  AttnF32Args a{q, positions, row_seq, block_table, k_cache, v_cache, out, rows, heads, kv_heads, head_dim,
                page_size, table_stride, q_stride, out_stride, window, scale};
  dim3 grid(rows, heads), block(64);
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
