// C entry points of the kernel library.  Every function launches on the given stream and
// returns 0, a HIP error code (> 0), or a negative code for arguments it refuses:
//   -2 sizes or strides out of range, -3 misaligned pointer or stride,
//   -4 head size not compiled in, -5 page size not supported, -6 scratch smaller than asked for,
//   -7 sizes beyond what the library's own static scratch holds (inside the library also: not this kernel's shape),
//   -8 a decode attention whose partials do not fit a workgroup's LDS (a context too long for the kernel).
// All pointers are device pointers.  Nothing here allocates.
#pragma once
#include <stdint.h>

extern "C" {
int bw_embed(const int32_t* tokens, const int32_t* feedback, const void* table, int table_is_bf16, float* out,
             int rows, int width, int vocab, void* stream);
int bw_rmsnorm(const float* x, const void* weight, int weight_is_bf16, void* y, int out_is_bf16, int rows,
               int dim, int ldy, float eps, void* stream);
int bw_add(float* x, const float* y, long long n, void* stream);
int bw_add_bias(float* x, const float* bias, int rows, int cols, int ldx, void* stream);
int bw_convert(const void* src, int src_is_bf16, void* dst, int dst_is_bf16, int rows, int cols, int lds, int ldd,
               void* stream);
int bw_swiglu_f32(const float* gate_up, float* h, int rows, int inter, void* stream);
int bw_gather_rows_f32(const float* x, const int32_t* idx, float* out, int count, int width, int ldx, void* stream);
int bw_rope_kvwrite(float* qkv, void* q_out, const int32_t* positions, const int32_t* row_seq,
                    const int32_t* block_table, int table_stride, const float* cos_table, const float* sin_table,
                    void* k_cache, void* v_cache, int is_bf16, int rows, int heads, int kv_heads, int head_dim,
                    int page_size, int write_cache, void* stream);
int bw_gemm_f32(const float* x, const void* w, int w_is_bf16, float* y, int M, int N, int K, int ldx, int ldy,
                int accumulate, void* stream);
int bw_gemm_bf16(const void* x, const void* w, void* out, int M, int N, int K, int ldx, int ldo, int epilogue,
                 void* stream);
int bw_gemm_add_scratch(int M, int N, int K, long long* scratch_floats, int* counters);
int bw_gemm_add_bf16(const void* x, const void* w, void* out, int M, int N, int K, int ldx, int ldo, float* scratch,
                     long long scratch_floats, int32_t* counters, int num_counters, void* stream);
// No counterpart in the reference.  For callers that cannot allocate device memory and cannot bring a
// workspace either (code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc):
// bw_gemm_add_bf16 with its scratch (the segments' sums, the tiles' counters) in a static array of the
// library's device image, 8 MB + 4 KB on every GPU the library runs on, held until the process ends.
// Shapes whose scratch would exceed that (bw_gemm_add_bf16_static_max gives the limits, bw_gemm_add_scratch
// what a shape needs) are refused with -7.  It calls no hipMalloc, no hipFree and no allocating library
// routine.  All calls on one GPU share that GPU's array: calls that overlap on one GPU race; calls on one
// stream, one after the other, do not.  The bits are those of bw_gemm_add_bf16.
int bw_gemm_add_bf16_static(const void* x, const void* w, void* out, int M, int N, int K, int ldx, int ldo,
                            void* stream);
int bw_gemm_add_bf16_static_max(long long* scratch_floats, int* counters);
int bw_gemm_qkv_rope_bf16(const void* x, int ldx, const void* w_qkv, void* q_out, const int32_t* positions,
                          const int32_t* row_seq, const int32_t* block_table, int table_stride, const float* cos_table,
                          const float* sin_table, void* k_cache, void* v_cache, int M, int heads, int kv_heads,
                          int head_dim, int K, int page_size, int write_cache, void* stream);
int bw_attention_f32(const float* q, int q_stride, const int32_t* positions, const int32_t* row_seq,
                     const int32_t* block_table, int table_stride, const float* k_cache, const float* v_cache,
                     float* out, int out_stride, int rows, int heads, int kv_heads, int head_dim, int page_size,
                     int window, float scale, void* stream);
int bw_attention_f32_tiles(const float* q, int q_stride, const int32_t* positions, const int32_t* block_table,
                           int table_stride, const int32_t* tiles, int num_tiles, int tiled, const float* k_cache,
                           const float* v_cache, float* out, int out_stride, int heads, int kv_heads, int head_dim,
                           int page_size, int window, float scale, void* stream);
int bw_attention_bf16(const void* q, int q_stride, const int32_t* positions, const int32_t* block_table,
                      int table_stride, const int32_t* tiles, int num_tiles, const void* k_cache,
                      const void* v_cache, int num_pages, void* out, int out_stride, int heads, int kv_heads,
                      int head_dim, int page_size, int window, float scale, int decode, float* scratch,
                      long long scratch_floats, int32_t* counters, int num_counters, void* stream);
int bw_attention_decode_scratch(int num_tiles, int heads, int kv_heads, int head_dim, int table_stride,
                                int page_size, long long* scratch_floats, int* counters);
int bw_attention_fold_group_tiles(int head_dim);
int bw_norm_gemm_supported(int M, int K);
// rows wider than one 2048-segment of K: whether the fused norm + product kernel with ``cols`` columns a workgroup takes them
int bw_norm_gemm_wide_supported(int M, int N, int K, int cols);
int bw_norm_gemm_bf16(const float* x, int ldx, const void* norm_w, int norm_w_is_bf16, float eps, const void* w,
                      void* out, int ldo, int M, int N, int K, int epilogue, void* stream);
int bw_norm_qkv_rope_bf16(const float* x, int ldx, const void* norm_w, int norm_w_is_bf16, float eps,
                          const void* w_qkv, void* q_out, const int32_t* positions, const int32_t* row_seq,
                          const int32_t* block_table, int table_stride, const float* cos_table,
                          const float* sin_table, void* k_cache, void* v_cache, int M, int heads, int kv_heads,
                          int head_dim, int K, int page_size, int write_cache, void* stream);
// Between bw_chain_begin and bw_chain_end (in the calling thread) the decode products of up to 16 rows that can run as
// phases of one launch (bw_norm_gemm_bf16 with SwiGLU or a 32-bit store, bw_norm_qkv_rope_bf16, the residual adds of
// bw_gemm_bf16 / bw_gemm_add_bf16 of few columns) are not launched when they are asked for: they wait, and leave as one
// launch whose phases wait for each other inside the kernel when anything else of gemm_bf16.hip or fused_decode.hip is
// launched, at bw_chain_flush, or at the end.  A caller that launches anything else on the stream meanwhile (this
// library's other entry points included) calls bw_chain_flush first.  sync: bw_chain_sync_words() 32-bit words, zero
// before the first chain (every launch leaves them zero); err: a word that gets a bit for every phase one of whose
// bounded waits gave up after spin_limit looks (then the results are void and the caller clears sync).  The same bits.
int bw_chain_sync_words();
int bw_chain_begin(void* sync, int sync_words, void* err, int spin_limit);
int bw_chain_flush(void* stream);
int bw_chain_end(void* stream);
int bw_sample(const float* logits, int vocab, int ld, int rows, const float* temperature, const double* uniform,
              int32_t* out, void* stream);
int bw_fingerprint(const float* logits, int vocab, int ld, int rows, const void* h_in, void* h_out, void* stream);
}
