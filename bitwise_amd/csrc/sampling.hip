// Token choice and logits fingerprints on the device, one workgroup per logits row.
//
// Greedy: the first maximum wins (the reference scans with a strict '>', src/engine.cpp:40-45).
// Temperature: w[i] = bw_expf((l[i] - max) / T) in 32-bit, sums in double, the token is the first
// i whose running sum exceeds u * total, else the last i with positive weight
// (src/engine.cpp:50-73).  The reference adds the weights one after the other; here each of
// the 256 threads adds its own contiguous stretch of the vocabulary in order and the
// stretches are joined in thread order, which moves the running sum by a few units of
// 2^-53 and depends on nothing but the row itself.  u comes from the host's counter-based
// generator keyed by (seed, position, stream).
#include "common.h"
#include "api.h"

#define SMP_THREADS 256

__global__ __launch_bounds__(SMP_THREADS) void sample_kernel(const float* __restrict__ logits, int vocab, int ld,
                                                             const float* __restrict__ temperature,
                                                             const double* __restrict__ uniform,
                                                             int32_t* __restrict__ out) {
  __shared__ float s_val[SMP_THREADS];
  __shared__ int s_idx[SMP_THREADS];
  __shared__ double s_sum[SMP_THREADS];
  __shared__ int s_pick[SMP_THREADS];
  __shared__ int s_lastpos[SMP_THREADS];
  __shared__ double s_total;
  const int row = blockIdx.x, tid = threadIdx.x;
  const float* l = logits + (size_t)row * ld;
  const int chunk = (vocab + SMP_THREADS - 1) / SMP_THREADS;
  const int begin = tid * chunk < vocab ? tid * chunk : vocab;
  const int end = begin + chunk < vocab ? begin + chunk : vocab;

  // maximum and its first index: every thread scans an interleaved share of the row in ascending
  // order (16-byte loads where the row allows), the shares are joined below with ties going to
  // the smaller index, so the first maximum of the whole row wins whatever the split
  float best = -INFINITY;
  int best_i = 0x7fffffff;
  if ((vocab & 3) == 0 && (ld & 3) == 0 && (reinterpret_cast<uintptr_t>(logits) & 15) == 0) {
    const f32x4* lv = reinterpret_cast<const f32x4*>(l);
    const int nv = vocab >> 2;
    auto scan = [&](const f32x4& x, int v) {
#pragma unroll
      for (int e = 0; e < 4; ++e)
        if (x[e] > best || best_i == 0x7fffffff) {  // the share's first element, or strictly greater
          best = x[e];
          best_i = 4 * v + e;
        }
    };
    int v = tid;
    for (; v + 3 * SMP_THREADS < nv; v += 4 * SMP_THREADS) {   // four loads in flight, scanned in ascending order
      const f32x4 x0 = lv[v], x1 = lv[v + SMP_THREADS], x2 = lv[v + 2 * SMP_THREADS], x3 = lv[v + 3 * SMP_THREADS];
      scan(x0, v);
      scan(x1, v + SMP_THREADS);
      scan(x2, v + 2 * SMP_THREADS);
      scan(x3, v + 3 * SMP_THREADS);
    }
    for (; v < nv; v += SMP_THREADS) scan(lv[v], v);
  } else {
    for (int i = tid; i < vocab; i += SMP_THREADS)
      if (l[i] > best || best_i == 0x7fffffff) {
        best = l[i];
        best_i = i;
      }
  }
  s_val[tid] = best;
  s_idx[tid] = best_i;
  __syncthreads();
  for (int off = SMP_THREADS / 2; off >= 1; off >>= 1) {
    if (tid < off) {
      const float ov = s_val[tid + off];
      const int oi = s_idx[tid + off];
      if (oi != 0x7fffffff && (s_idx[tid] == 0x7fffffff || ov > s_val[tid] || (ov == s_val[tid] && oi < s_idx[tid]))) {
        s_val[tid] = ov;
        s_idx[tid] = oi;
      }
    }
    __syncthreads();
  }
  const float mx = s_val[0];
  const float T = temperature[row];
  if (T <= 0.0f) {
    if (tid == 0) out[row] = s_idx[0];
    return;
  }

  double part = 0.0;
  int lastpos = -1;
  for (int i = begin; i < end; ++i) {
    const float w = bw_expf((l[i] - mx) / T);
    if (w > 0.0f) {
      part += (double)w;
      lastpos = i;
    }
  }
  s_sum[tid] = part;
  s_lastpos[tid] = lastpos;
  s_pick[tid] = -1;
  __syncthreads();
  if (tid == 0) {  // exclusive prefix in thread order; s_sum[t] becomes the sum before stretch t
    double run = 0.0;
    int last = 0;
    for (int t = 0; t < SMP_THREADS; ++t) {
      const double p = s_sum[t];
      s_sum[t] = run;
      run += p;
      if (s_lastpos[t] >= 0) last = s_lastpos[t];
    }
    s_lastpos[0] = last;
    s_total = run;
  }
  __syncthreads();
  const double total = s_total;
  const double target = uniform[row] * total;
  double cum = s_sum[tid];
  if (cum <= target) {
    for (int i = begin; i < end; ++i) {
      const float w = bw_expf((l[i] - mx) / T);
      if (w <= 0.0f) continue;
      cum += (double)w;
      if (cum > target) {
        s_pick[tid] = i;
        break;
      }
    }
  }
  __syncthreads();
  if (tid == 0) {
    int pick = s_lastpos[0];
    for (int t = 0; t < SMP_THREADS; ++t)
      if (s_pick[t] >= 0) {
        pick = s_pick[t];
        break;
      }
    out[row] = pick;
  }
}

extern "C" int bw_sample(const float* logits, int vocab, int ld, int rows, const float* temperature,
                         const double* uniform, int32_t* out, void* stream) {
  if (rows <= 0) return 0;
  if (vocab <= 0 || ld < vocab) return -2;
  hipLaunchKernelGGL(sample_kernel, dim3(rows), dim3(SMP_THREADS), 0, (hipStream_t)stream, logits, vocab, ld,
                     temperature, uniform, out);
  return BW_LAUNCH_CHECK();
}

// Fingerprint chain of the reference (src/engine.cpp:18-29): h = (h ^ word) * 1099511628211
// over the row's 8-byte words, single trailing bytes likewise, then the splitmix64 finaliser.
// The chain is sequential by construction (an exclusive or, then a product modulo 2^64: no algebra in which both
// are linear), so a row's time is its number of words times the latency of one link.  A wave takes a row: the row's
// address is the same for every lane, so the words arrive through the scalar unit, sixteen of them a load and the
// next sixteen asked for before these are used, and the chain runs in scalar registers, a link every dozen clocks;
// rows run beside each other on as many compute units.  (One lane a row with loads of its own, as this kernel
// was first written, spent a memory latency a word: 6.4 ms for 64 rows of 128,256 logits.)
#define FP_BLOCK 16        // words of 8 bytes a block
__device__ __forceinline__ uint64_t fp_link(uint64_t h, uint32_t lo, uint32_t hi) {
  return (h ^ ((uint64_t)lo | ((uint64_t)hi << 32))) * 1099511628211ull;
}

struct FpBlock {
  uint32_t d[2 * FP_BLOCK];
};

__device__ __forceinline__ void fp_load(FpBlock& blk, const uint32_t* __restrict__ p) {
#pragma unroll
  for (int j = 0; j < 2 * FP_BLOCK; ++j) blk.d[j] = p[j];
}

__device__ __forceinline__ uint64_t fp_chain(uint64_t h, const FpBlock& blk) {
#pragma unroll
  for (int j = 0; j < FP_BLOCK; ++j) h = fp_link(h, blk.d[2 * j], blk.d[2 * j + 1]);
  return h;
}

__global__ __launch_bounds__(64) void fingerprint_kernel(const float* __restrict__ logits, int vocab, int ld, int rows,
                                                         const uint64_t* __restrict__ h_in, uint64_t* __restrict__ h_out) {
  const int row = blockIdx.x;                                         // the same for every lane: scalar from here on
  if (row >= rows) return;
  const uint32_t* __restrict__ p = reinterpret_cast<const uint32_t*>(logits + (size_t)row * ld);
  uint64_t h = h_in[row];
  const int words = vocab >> 1;
  const int blocks = words / FP_BLOCK;
  // two blocks in turn: while one is chained the other is on its way (scalar loads come back in any order, so a
  // wait is for all of them; each block is asked for a whole chain of sixteen links before it is needed)
  FpBlock even, odd;
  if (blocks > 0) fp_load(even, p);
  int b = 0;
  for (; b + 2 <= blocks; b += 2) {
    __builtin_amdgcn_s_waitcnt(0xc07f);                                // lgkmcnt(0): the block to be chained now is there ...
    __builtin_amdgcn_sched_barrier(0);
    fp_load(odd, p + (size_t)(b + 1) * 2 * FP_BLOCK);                  // ... before the next one is asked for
    __builtin_amdgcn_sched_barrier(0);
    h = fp_chain(h, even);
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_waitcnt(0xc07f);
    __builtin_amdgcn_sched_barrier(0);
    fp_load(even, p + (size_t)(b + 2 < blocks ? b + 2 : b) * 2 * FP_BLOCK);      // (past the end: a block once more, unused)
    __builtin_amdgcn_sched_barrier(0);
    h = fp_chain(h, odd);
    __builtin_amdgcn_sched_barrier(0);
  }
  if (b < blocks) h = fp_chain(h, even);                               // an odd number of blocks: the last one
  for (int i = blocks * FP_BLOCK; i < words; ++i) h = fp_link(h, p[2 * i], p[2 * i + 1]);
  if (vocab & 1) {
    const uint32_t t = p[vocab - 1];
    for (int k = 0; k < 4; ++k) h = (h ^ ((t >> (8 * k)) & 0xffu)) * 1099511628211ull;
  }
  h = (h ^ (h >> 30)) * 0xBF58476D1CE4E5B9ull;
  h = (h ^ (h >> 27)) * 0x94D049BB133111EBull;
  if (threadIdx.x == 0) h_out[row] = h ^ (h >> 31);
}

extern "C" int bw_fingerprint(const float* logits, int vocab, int ld, int rows, const void* h_in, void* h_out,
                              void* stream) {
  if (rows <= 0) return 0;
  hipLaunchKernelGGL(fingerprint_kernel, dim3(rows), dim3(64), 0, (hipStream_t)stream, logits, vocab, ld,
                     rows, (const uint64_t*)h_in, (uint64_t*)h_out);
  return BW_LAUNCH_CHECK();
}
