// Row-wise kernels around the matrix products: embedding gather, RMSNorm, rotary
// position encoding fused with the cache write, SwiGLU, residual add, row gather.
//
// 32-bit variants follow the reference's operation order exactly
// (src/kernels.cpp:57-103, :264-298; src/model.cpp:285-297); the bfloat16 variants keep
// sums of squares, rotation and the residual in 32-bit and round once when they store.
#include "common.h"
#include "api.h"

// ------------------------------------------------------------------------- embedding

// A token of -2 stands for "the token the last step sampled for this row": it is read from ``feedback`` (the
// sampling kernel's output), so that a decode step can be launched before the host has seen the token.
#define BW_TOKEN_FROM_FEEDBACK (-2)

template <typename TableT>
__global__ void embed_kernel(const int32_t* __restrict__ tokens, const int32_t* __restrict__ feedback,
                             const TableT* __restrict__ table, float* __restrict__ out, int width, int vocab) {
  const int row = blockIdx.x;
  int tok = tokens[row];
  if (tok == BW_TOKEN_FROM_FEEDBACK && feedback != nullptr) tok = feedback[row];
  float* o = out + (size_t)row * width;
  if (tok < 0 || tok >= vocab) {  // padding rows of a fixed-size batch carry token -1
    for (int i = threadIdx.x; i < width; i += blockDim.x) o[i] = 0.0f;
    return;
  }
  const TableT* e = table + (size_t)tok * width;
  for (int i = threadIdx.x; i < width; i += blockDim.x) {
    if constexpr (sizeof(TableT) == 2) o[i] = bf16_to_f32(e[i]);
    else o[i] = e[i];
  }
}

extern "C" int bw_embed(const int32_t* tokens, const int32_t* feedback, const void* table, int table_is_bf16, float* out,
                        int rows, int width, int vocab, void* stream) {
  if (rows <= 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  if (table_is_bf16)
    hipLaunchKernelGGL(embed_kernel<bf16_t>, dim3(rows), dim3(256), 0, s, tokens, feedback, (const bf16_t*)table, out, width, vocab);
  else
    hipLaunchKernelGGL(embed_kernel<float>, dim3(rows), dim3(256), 0, s, tokens, feedback, (const float*)table, out, width, vocab);
  return BW_LAUNCH_CHECK();
}

// ------------------------------------------------------------------------- RMSNorm, 32-bit

// 16 lanes per row: lane j runs the fused multiply-add chain over i = j, j+16, ... and the
// lanes are joined by the tree (v[i]+v[i+8]), (+4), (s4[0]+s4[2])+(s4[1]+s4[3])
// (src/kernels.cpp:57-64, :86-101).  Then inv = 1/sqrt(ss/dim + eps), y = (x*inv)*w
// (src/kernels.cpp:264-271).
template <typename WT>
__global__ void rmsnorm_f32_kernel(const float* __restrict__ x, const WT* __restrict__ w,
                                   float* __restrict__ y, int rows, int dim, float eps) {
  const int sub = threadIdx.x & 15;
  const int row = blockIdx.x * (blockDim.x >> 4) + (threadIdx.x >> 4);
  const bool live = row < rows;
  const float* xr = x + (size_t)(live ? row : 0) * dim;
  float acc = 0.0f;
  if (live)
    for (int i = sub; i < dim; i += 16) acc = fmaf(xr[i], xr[i], acc);
  acc = row16_sum(acc);
  if (!live) return;
  const float inv = 1.0f / sqrtf(acc / (float)dim + eps);
  float* yr = y + (size_t)row * dim;
  for (int i = sub; i < dim; i += 16) {
    float wi;
    if constexpr (sizeof(WT) == 2) wi = bf16_to_f32(w[i]);
    else wi = w[i];
    yr[i] = (xr[i] * inv) * wi;
  }
}

// The same chains and tree for rows of up to RMS32_MAX elements, a workgroup a row: its 256 threads bring the row
// into LDS together, 16 of them run the chains from there (nothing between two steps of a chain but an LDS
// read), and all write the result.
#define RMS32_MAX 8192
template <typename WT>
__global__ __launch_bounds__(256) void rmsnorm_f32_row_kernel(const float* __restrict__ x, const WT* __restrict__ w,
                                                              float* __restrict__ y, int dim, float eps) {
  __shared__ float row_lds[RMS32_MAX];
  __shared__ float inv_lds;
  const float* xr = x + (size_t)blockIdx.x * dim;
  for (int i = threadIdx.x; i < dim; i += 256) row_lds[i] = xr[i];
  __syncthreads();
  if (threadIdx.x < 16) {
    float acc = 0.0f;
#pragma unroll 8
    for (int i = threadIdx.x; i < dim; i += 16) acc = fmaf(row_lds[i], row_lds[i], acc);
    acc = row16_sum(acc);
    if (threadIdx.x == 0) inv_lds = 1.0f / sqrtf(acc / (float)dim + eps);
  }
  __syncthreads();
  const float inv = inv_lds;
  float* yr = y + (size_t)blockIdx.x * dim;
  for (int i = threadIdx.x; i < dim; i += 256) {
    float wi;
    if constexpr (sizeof(WT) == 2) wi = bf16_to_f32(w[i]);
    else wi = w[i];
    yr[i] = (row_lds[i] * inv) * wi;
  }
}

// ------------------------------------------------------------------------- RMSNorm, bfloat16 out

// One wave per row.  Rows whose width is a multiple of 4 are read as 16-byte vectors: lane l
// takes vectors l, l+64, ... and runs one fused multiply-add chain over its elements in
// ascending order; other widths take elements l, l+64, ...  The lanes are joined by xor
// butterflies (32, 16, ..., 1).  All in 32-bit; one rounding at the store.  The order depends
// on the width alone, so a row's result depends on that row alone.
template <typename WT>
__global__ __launch_bounds__(256) void rmsnorm_bf16_kernel(const float* __restrict__ x, const WT* __restrict__ w,
                                                           bf16_t* __restrict__ y, int rows, int dim, int ldy,
                                                           float eps) {
  const int lane = threadIdx.x & 63;
  const int row = blockIdx.x * (blockDim.x >> 6) + wave_index();
  if (row >= rows) return;
  const float* xr = x + (size_t)row * dim;
  bf16_t* yr = y + (size_t)row * ldy;
  float acc = 0.0f;
  if ((dim & 3) == 0 && (ldy & 3) == 0) {
    const int nvec = dim >> 2;
    const f32x4* xv = reinterpret_cast<const f32x4*>(xr);
    if (dim <= 2048) {      // the whole row fits the wave's registers: one round of loads
      rmsnorm_row_small(xv, w, sizeof(WT) == 2, nvec, dim, eps, lane,
                        [&](int c, u32x2 pk) { *reinterpret_cast<u32x2*>(yr + 4 * c) = pk; });
      return;
    }
    if (dim <= 4096) {      // sixteen vectors a lane: still one round of loads (two cost a second trip to memory)
      rmsnorm_row_small<16>(xv, w, sizeof(WT) == 2, nvec, dim, eps, lane,
                            [&](int c, u32x2 pk) { *reinterpret_cast<u32x2*>(yr + 4 * c) = pk; });
      return;
    }
    acc = row_sumsq_vec(xv, nvec, lane);
    const float inv = 1.0f / sqrtf(acc / (float)dim + eps);
    // eight vectors of the row and of the weight asked for before the first is used (a loop of one load and its
    // store waits a memory round trip for every vector: 9 us for rows of 4096)
    constexpr int UN = 8;
    for (int c0 = 0; c0 < nvec; c0 += 64 * UN) {
      f32x4 v[UN];
      u32x4 wr[UN];
#pragma unroll
      for (int j = 0; j < UN; ++j) {
        const int c = c0 + 64 * j + lane < nvec ? c0 + 64 * j + lane : nvec - 1;
        v[j] = xv[c];
        wr[j] = load_norm_w_raw(w, sizeof(WT) == 2, c);
      }
#pragma unroll
      for (int j = 0; j < UN; ++j) {
        const int c = c0 + 64 * j + lane;
        if (c >= nvec) continue;
        const f32x4 wv = norm_w_floats(wr[j], sizeof(WT) == 2);
        u32x2 pk = {pack_bf16x2((v[j][0] * inv) * wv[0], (v[j][1] * inv) * wv[1]),
                    pack_bf16x2((v[j][2] * inv) * wv[2], (v[j][3] * inv) * wv[3])};
        *reinterpret_cast<u32x2*>(yr + 4 * c) = pk;
      }
    }
    return;
  }
  for (int i = lane; i < dim; i += 64) acc = fmaf(xr[i], xr[i], acc);
  acc = wave_sum(acc);
  const float inv = 1.0f / sqrtf(acc / (float)dim + eps);
  for (int i = lane; i < dim; i += 64) {
    float wi;
    if constexpr (sizeof(WT) == 2) wi = bf16_to_f32(w[i]);
    else wi = w[i];
    yr[i] = f32_to_bf16((xr[i] * inv) * wi);
  }
}

extern "C" int bw_rmsnorm(const float* x, const void* weight, int weight_is_bf16, void* y, int out_is_bf16,
                          int rows, int dim, int ldy, float eps, void* stream) {
  if (rows <= 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  if (out_is_bf16) {
    dim3 grid((rows + 3) / 4), block(256);
    if (weight_is_bf16)
      hipLaunchKernelGGL(rmsnorm_bf16_kernel<bf16_t>, grid, block, 0, s, x, (const bf16_t*)weight, (bf16_t*)y, rows, dim, ldy, eps);
    else
      hipLaunchKernelGGL(rmsnorm_bf16_kernel<float>, grid, block, 0, s, x, (const float*)weight, (bf16_t*)y, rows, dim, ldy, eps);
  } else {
    if (ldy != dim) return -2;
    if (dim <= RMS32_MAX) {
      if (weight_is_bf16)
        hipLaunchKernelGGL(rmsnorm_f32_row_kernel<bf16_t>, dim3(rows), dim3(256), 0, s, x, (const bf16_t*)weight, (float*)y, dim, eps);
      else
        hipLaunchKernelGGL(rmsnorm_f32_row_kernel<float>, dim3(rows), dim3(256), 0, s, x, (const float*)weight, (float*)y, dim, eps);
      return BW_LAUNCH_CHECK();
    }
    dim3 grid((rows + 15) / 16), block(256);
    if (weight_is_bf16)
      hipLaunchKernelGGL(rmsnorm_f32_kernel<bf16_t>, grid, block, 0, s, x, (const bf16_t*)weight, (float*)y, rows, dim, eps);
    else
      hipLaunchKernelGGL(rmsnorm_f32_kernel<float>, grid, block, 0, s, x, (const float*)weight, (float*)y, rows, dim, eps);
  }
  return BW_LAUNCH_CHECK();
}

// ------------------------------------------------------------------------- small row ops

__global__ void add_kernel(float* __restrict__ x, const float* __restrict__ y, size_t n) {
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) x[i] += y[i];
}

extern "C" int bw_add(float* x, const float* y, long long n, void* stream) {
  if (n <= 0) return 0;
  hipLaunchKernelGGL(add_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, (hipStream_t)stream, x, y, (size_t)n);
  return BW_LAUNCH_CHECK();
}

// x[r, c] += bias[c] in 32-bit: a projection's bias, one addition behind the product's sum.
__global__ void add_bias_kernel(float* __restrict__ x, const float* __restrict__ bias, int rows, int cols, int ldx) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= (size_t)rows * cols) return;
  const int r = (int)(i / cols), c = (int)(i % cols);
  x[(size_t)r * ldx + c] += bias[c];
}

extern "C" int bw_add_bias(float* x, const float* bias, int rows, int cols, int ldx, void* stream) {
  if (rows <= 0 || cols <= 0) return 0;
  if (ldx < cols) return -2;
  const size_t n = (size_t)rows * cols;
  hipLaunchKernelGGL(add_bias_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, (hipStream_t)stream, x, bias, rows, cols, ldx);
  return BW_LAUNCH_CHECK();
}

// dst[r, c] = src[r, c] between 32-bit and bfloat16 rows (widening is exact; narrowing rounds to nearest even
// with the hardware conversion).  For the routes on which a weight's dtype is not the mode's.
template <typename S, typename D>
__global__ void convert_kernel(const S* __restrict__ src, D* __restrict__ dst, int rows, int cols, int lds, int ldd) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= (size_t)rows * cols) return;
  const int r = (int)(i / cols), c = (int)(i % cols);
  const S v = src[(size_t)r * lds + c];
  if constexpr (sizeof(S) == 4 && sizeof(D) == 2) dst[(size_t)r * ldd + c] = f32_to_bf16(v);
  else if constexpr (sizeof(S) == 2 && sizeof(D) == 4) dst[(size_t)r * ldd + c] = bf16_to_f32(v);
  else dst[(size_t)r * ldd + c] = v;
}

extern "C" int bw_convert(const void* src, int src_is_bf16, void* dst, int dst_is_bf16, int rows, int cols, int lds,
                          int ldd, void* stream) {
  if (rows <= 0 || cols <= 0) return 0;
  if (lds < cols || ldd < cols) return -2;
  const size_t n = (size_t)rows * cols;
  const dim3 grid((unsigned)((n + 255) / 256)), block(256);
  hipStream_t s = (hipStream_t)stream;
  if (src_is_bf16 && dst_is_bf16)
    hipLaunchKernelGGL((convert_kernel<bf16_t, bf16_t>), grid, block, 0, s, (const bf16_t*)src, (bf16_t*)dst, rows, cols, lds, ldd);
  else if (src_is_bf16)
    hipLaunchKernelGGL((convert_kernel<bf16_t, float>), grid, block, 0, s, (const bf16_t*)src, (float*)dst, rows, cols, lds, ldd);
  else if (dst_is_bf16)
    hipLaunchKernelGGL((convert_kernel<float, bf16_t>), grid, block, 0, s, (const float*)src, (bf16_t*)dst, rows, cols, lds, ldd);
  else
    hipLaunchKernelGGL((convert_kernel<float, float>), grid, block, 0, s, (const float*)src, (float*)dst, rows, cols, lds, ldd);
  return BW_LAUNCH_CHECK();
}

// h = g * (1/(1+exp(-g))) * u over rows laid out [gate | up] (src/kernels.cpp:291-298).
__global__ void swiglu_f32_kernel(const float* __restrict__ gate_up, float* __restrict__ h, int rows, int inter) {
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= (size_t)rows * inter) return;
  const int r = (int)(i / inter), c = (int)(i % inter);
  const float g = gate_up[(size_t)r * 2 * inter + c];
  const float u = gate_up[(size_t)r * 2 * inter + inter + c];
  h[i] = g * (1.0f / (1.0f + bw_expf(-g))) * u;
}

extern "C" int bw_swiglu_f32(const float* gate_up, float* h, int rows, int inter, void* stream) {
  if (rows <= 0) return 0;
  size_t n = (size_t)rows * inter;
  hipLaunchKernelGGL(swiglu_f32_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, (hipStream_t)stream, gate_up, h, rows, inter);
  return BW_LAUNCH_CHECK();
}

template <typename T>
__global__ void gather_rows_kernel(const T* __restrict__ x, const int32_t* __restrict__ idx, T* __restrict__ out,
                                   int width, int ldx) {
  const T* src = x + (size_t)idx[blockIdx.x] * ldx;
  T* dst = out + (size_t)blockIdx.x * width;
  for (int i = threadIdx.x; i < width; i += blockDim.x) dst[i] = src[i];
}

extern "C" int bw_gather_rows_f32(const float* x, const int32_t* idx, float* out, int count, int width, int ldx,
                                  void* stream) {
  if (count <= 0) return 0;
  hipLaunchKernelGGL(gather_rows_kernel<float>, dim3(count), dim3(256), 0, (hipStream_t)stream, x, idx, out, width, ldx);
  return BW_LAUNCH_CHECK();
}

// ------------------------------------------------------------------------- rotary + cache write

// The tables hold cos and sin of float(pos) * inv_freq[i] (src/kernels.cpp:277-279), built once
// on the host.  Pairs are (i, i + hd/2): out[i] = x1*c - x2*s, out[i+hd/2] = x2*c + x1*s, as
// separate products and one subtraction or addition (src/kernels.cpp:283-287).
// A row whose position is negative is padding and is skipped.

struct RopeArgs {
  const float* qkv;         // [rows, q_dim + 2*kv_dim] 32-bit, row = [q | k | v]
  const int32_t* positions;  // [rows]
  const int32_t* row_seq;    // [rows] -> row of the block table
  const int32_t* block_table;
  const float* cos_table;    // [max_pos, hd/2]
  const float* sin_table;
  int rows, heads, kv_heads, head_dim, page_size, table_stride, write_cache;
};

// 32-bit: q and k are rotated in place; k and v go to cache[page][kv_head][slot][hd]
// (src/model.cpp:291-296, src/kernels.h:97-99).
__global__ void rope_kvwrite_f32_kernel(RopeArgs a, float* qkv_rw, float* __restrict__ k_cache,
                                        float* __restrict__ v_cache) {
  const int row = blockIdx.x;
  const int pos = a.positions[row];
  if (pos < 0) return;
  const int hd = a.head_dim, half = hd / 2;
  const int q_dim = a.heads * hd, kv_dim = a.kv_heads * hd;
  float* r = qkv_rw + (size_t)row * (q_dim + 2 * kv_dim);
  const int page = a.block_table[(size_t)a.row_seq[row] * a.table_stride + pos / a.page_size];
  const int slot = pos % a.page_size;
  const float* ct = a.cos_table + (size_t)pos * half;
  const float* st = a.sin_table + (size_t)pos * half;
  const int pairs = (a.heads + a.kv_heads) * half;
  for (int e = threadIdx.x; e < pairs; e += blockDim.x) {
    const int hh = e / half, i = e % half;
    float* v = r + hh * hd;
    const float x1 = v[i], x2 = v[i + half];
    const float c = ct[i], s = st[i];
    const float o1 = x1 * c - x2 * s;
    const float o2 = x2 * c + x1 * s;
    v[i] = o1;
    v[i + half] = o2;
    if (hh >= a.heads && a.write_cache) {
      const int h = hh - a.heads;
      float* dst = k_cache + (((size_t)page * a.kv_heads + h) * a.page_size + slot) * hd;
      dst[i] = o1;
      dst[i + half] = o2;
    }
  }
  if (a.write_cache) {
    const float* vsrc = r + q_dim + kv_dim;
    for (int e = threadIdx.x; e < kv_dim; e += blockDim.x) {
      const int h = e / hd, d = e % hd;
      v_cache[(((size_t)page * a.kv_heads + h) * a.page_size + slot) * hd + d] = vsrc[e];
    }
  }
}

// bfloat16: rotation in 32-bit from the 32-bit projections; q goes to q_out [rows, q_dim],
// k to cache[page][kv_head][slot][hd], v transposed to cache[page][kv_head][hd][slot], each
// rounded once.
__global__ void rope_kvwrite_bf16_kernel(RopeArgs a, bf16_t* __restrict__ q_out, bf16_t* __restrict__ k_cache,
                                         bf16_t* __restrict__ v_cache) {
  const int row = blockIdx.x;
  const int pos = a.positions[row];
  if (pos < 0) return;
  const int hd = a.head_dim, half = hd / 2;
  const int q_dim = a.heads * hd, kv_dim = a.kv_heads * hd;
  const float* r = a.qkv + (size_t)row * (q_dim + 2 * kv_dim);
  const int page = a.block_table[(size_t)a.row_seq[row] * a.table_stride + pos / a.page_size];
  const int slot = pos % a.page_size;
  const float* ct = a.cos_table + (size_t)pos * half;
  const float* st = a.sin_table + (size_t)pos * half;
  const int pairs = (a.heads + a.kv_heads) * half;
  for (int e = threadIdx.x; e < pairs; e += blockDim.x) {
    const int hh = e / half, i = e % half;
    const float* v = r + hh * hd;
    const float x1 = v[i], x2 = v[i + half];
    const float c = ct[i], s = st[i];
    const float o1 = x1 * c - x2 * s;
    const float o2 = x2 * c + x1 * s;
    if (hh < a.heads) {
      bf16_t* dst = q_out + (size_t)row * q_dim + hh * hd;
      dst[i] = f32_to_bf16(o1);
      dst[i + half] = f32_to_bf16(o2);
    } else if (a.write_cache) {
      const int h = hh - a.heads;
      bf16_t* dst = k_cache + (((size_t)page * a.kv_heads + h) * a.page_size + slot) * hd;
      dst[i] = f32_to_bf16(o1);
      dst[i + half] = f32_to_bf16(o2);
    }
  }
  if (a.write_cache) {
    const float* vsrc = r + q_dim + kv_dim;
    for (int e = threadIdx.x; e < kv_dim; e += blockDim.x) {
      const int h = e / hd, d = e % hd;
      v_cache[(((size_t)page * a.kv_heads + h) * hd + d) * a.page_size + slot] = f32_to_bf16(vsrc[e]);
    }
  }
}

extern "C" int bw_rope_kvwrite(float* qkv, void* q_out, const int32_t* positions, const int32_t* row_seq,
                               const int32_t* block_table, int table_stride, const float* cos_table,
                               const float* sin_table, void* k_cache, void* v_cache, int is_bf16, int rows,
                               int heads, int kv_heads, int head_dim, int page_size, int write_cache,
                               void* stream) {
  if (rows <= 0) return 0;
  if (head_dim % 2 || page_size <= 0) return -2;
  RopeArgs a{qkv, positions, row_seq, block_table, cos_table, sin_table,
             rows, heads, kv_heads, head_dim, page_size, table_stride, write_cache};
  hipStream_t s = (hipStream_t)stream;
  if (is_bf16)
    hipLaunchKernelGGL(rope_kvwrite_bf16_kernel, dim3(rows), dim3(256), 0, s, a, (bf16_t*)q_out, (bf16_t*)k_cache, (bf16_t*)v_cache);
  else
    hipLaunchKernelGGL(rope_kvwrite_f32_kernel, dim3(rows), dim3(256), 0, s, a, qkv, (float*)k_cache, (float*)v_cache);
  return BW_LAUNCH_CHECK();
}
