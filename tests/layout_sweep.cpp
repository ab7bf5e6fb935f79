// Host-side sweep over the index arithmetic of the kernels that normalise rows into LDS in front of a matrix
// product (bitwise_amd/csrc/layout.h, which the kernels call for these addresses): for every shape a launcher
// admits, every wave, lane, register and step,
//   * every vector a lane loads from a row lies inside the row, and the lanes' vectors cover the row exactly once;
//   * every store of a normalised vector lies inside the rows' area of the launch's LDS, no two stores overlap,
//     and what lane (g, r) of a matrix instruction reads for step s is exactly what was stored for row r, elements
//     64 s + 32 kk + 8 g .. + 7 (a model of LDS holds, for every byte, which row and element was stored there);
//   * every load of the weights' ring lands inside the ring, the loads of a stage tile the stage exactly, and the
//     operand reads of a step stay inside the step.
// It is compiled with -fsanitize=address,undefined, so an index that leaves the model's arrays aborts the run.
// A second part applies the same checks to a variant that is not in the library any more (rows of up to 4096
// elements in every fused kernel, up to 16 rows, two rows a wave, sixteen vectors a lane) in the two forms it may
// have had, and prints what they show.  Output: lines "ok <what> <count>" / "FAIL <what> <detail>" / "note ...".
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <vector>

#include "../bitwise_amd/csrc/layout.h"

static long failures = 0;
static bool quiet = false;       // count only (the variant that is not in the library)
#define CHECK(cond, ...)                                 \
  do {                                                   \
    if (!(cond)) {                                       \
      if (failures < 40 && !quiet) { std::printf("FAIL "); std::printf(__VA_ARGS__); std::printf("\n"); } \
      ++failures;                                        \
    }                                                    \
  } while (0)

// ------------------------------------------------------------------------------ a row in a wave's registers
static long sweep_row_vectors(int nv, int max_k) {
  long n = 0;
  for (int K = 64; K <= max_k; K += 64) {
    const int nvec = K / 4;
    std::vector<int> seen(nvec, 0);
    for (int lane = 0; lane < 64; ++lane)
      for (int j = 0; j < nv; ++j) {
        const int c = norm_vec_index(j, lane, nvec);
        CHECK(c >= 0 && c < nvec, "row vector: K %d lane %d j %d -> %d of %d", K, lane, j, c, nvec);
        if (norm_vec_in_row(j, lane, nvec)) {
          CHECK(c == 64 * j + lane, "row vector: K %d lane %d j %d kept but clamped", K, lane, j);
          if (c >= 0 && c < nvec) ++seen[c];
        }
        ++n;
      }
    for (int c = 0; c < nvec; ++c) CHECK(seen[c] == 1, "row vector %d of K %d is held %d times with %d registers a lane", c, K, seen[c], nv);
  }
  return n;
}

// ------------------------------------------------------------------------------ gemm_bf16_mid_kernel, the ring
template <class S, int NRB>
static long sweep_mid_ring(const char* what) {
  long n = 0;
  std::vector<int> owner(S::RING, -1);                // per KB of a stage: which (wave, load) fills it
  CHECK(S::RING <= BW_LDS_LIMIT, "%s: ring of %d bytes", what, S::RING);
  std::vector<int> filled(S::STAGE / 1024, 0);
  for (int wave = 0; wave < S::NW; ++wave) {
    for (int t = 0; t < S::A_LOADS; ++t) {
      int sub, block;
      if (!mid_a_load<S, NRB>(wave, t, sub, block)) continue;     // a padding load: behind the ring
      const int dst = mid_a_dst<S>(sub, block);
      CHECK(dst >= 0 && dst % 1024 == 0 && dst + 1024 <= S::STAGE, "%s: x load of wave %d, %d lands at %d of a stage of %d", what, wave, t, dst, S::STAGE);
      CHECK(sub < S::SUB && dst - sub * S::STEP_BYTES < S::A_BYTES, "%s: x load of wave %d, %d leaves the step's rows of x", what, wave, t);
      if (dst >= 0 && dst + 1024 <= S::STAGE) ++filled[dst / 1024];
      ++n;
    }
    for (int t = 0; t < S::B_LOADS; ++t) {
      int sub, blk;
      mid_b_load<S>(wave, t, sub, blk);
      const int dst = mid_b_dst<S>(sub, blk);
      CHECK(sub >= 0 && sub < S::SUB && blk >= 0 && blk < S::B_ROWS / 8, "%s: W load of wave %d, %d is block %d of step %d", what, wave, t, blk, sub);
      CHECK(dst >= 0 && dst % 1024 == 0 && dst + 1024 <= S::STAGE, "%s: W load of wave %d, %d lands at %d of a stage of %d", what, wave, t, dst, S::STAGE);
      if (dst >= 0 && dst + 1024 <= S::STAGE) ++filled[dst / 1024];
      ++n;
    }
  }
  for (int kb = 0; kb < S::STAGE / 1024; ++kb) CHECK(filled[kb] == 1, "%s: KB %d of a stage is filled %d times", what, kb, filled[kb]);
  for (int step = 0; step < 3 * S::STAGES; ++step) {
    const int off = mid_stage_offset<S>(step);
    CHECK(off >= 0 && off + S::STAGE <= mid_padding_offset<S>(), "%s: stage of step %d at %d", what, step, off);
  }
  CHECK(mid_padding_offset<S>() + 1024 <= S::RING, "%s: the padding loads' KB ends at %d of %d", what, mid_padding_offset<S>() + 1024, S::RING);
  // operand reads of W: inside the step, inside the wave's own strip(s)
  for (int wave = 0; wave < S::NW; ++wave)
    for (int j = 0; j < S::NJ; ++j)
      for (int lane = 0; lane < 64; ++lane)
        for (int kk = 0; kk < 2; ++kk) {
          const int off = mid_b_read_offset<S>(wave % S::STRIPS, j, lane & 15, lane >> 4, kk);
          CHECK(off >= S::A_BYTES && off + 16 <= S::STEP_BYTES, "%s: W operand read of wave %d lane %d at %d of a step of %d", what, wave, lane, off, S::STEP_BYTES);
          ++n;
        }
  // operand reads of x (not NORM): the wave's blocks of rows inside the step's rows of x
  if (S::A_BYTES > 0)
    for (int wave = 0; wave < S::NW; ++wave) {
      const int b0 = mid_first_block<S>(wave);
      if (b0 >= NRB) continue;                                     // a wave that only loads
      for (int i = 0; i < S::NI; ++i)
        for (int lane = 0; lane < 64; ++lane)
          for (int kk = 0; kk < 2; ++kk) {
            const int off = (b0 + i) * 2048 + mid_operand_offset(lane & 15, lane >> 4, kk);
            CHECK(off >= 0 && off + 16 <= S::A_BYTES, "%s: x operand read of wave %d at %d of %d", what, wave, off, S::A_BYTES);
            ++n;
          }
    }
  return n;
}

// ------------------------------------------------------------------------------ gemm_bf16_mid_kernel, NORM rows
// One launch: rows_a_wave / vectors_a_lane / row_step / rows' bytes are parameters, so that a variant which is
// not the library's can be put through the same checks.  Returns the number of addresses checked.
struct RowsModel {
  std::vector<int32_t> who;          // per 2 bytes of the rows' area: row * 65536 + element, or -1
  explicit RowsModel(size_t bytes) : who(bytes / 2, -1) {}
};

template <class S>
static long sweep_mid_norm_launch(const char* what, int M, int K, int rows_a_wave, int nv, int row_step, int lds_bytes, bool clamp) {
  long n = 0;
  const int nvec = K / 4, rows_bytes = lds_bytes - S::RING;
  CHECK(lds_bytes <= BW_LDS_LIMIT, "%s: M %d K %d asks for %d bytes of LDS", what, M, K, lds_bytes);
  if (rows_bytes <= 0) return n;
  RowsModel lds((size_t)rows_bytes);
  CHECK(rows_a_wave * S::NW >= M, "%s: M %d rows, %d a wave on %d waves", what, M, rows_a_wave, S::NW);
  CHECK(nv * 64 >= nvec, "%s: K %d has %d vectors, a lane holds %d", what, K, nvec, nv);
  for (int wave = 0; wave < S::NW && wave < M; ++wave)
    for (int i = 0; i < rows_a_wave; ++i) {
      const int m = mid_norm_row_of(wave, i, S::NW);
      if (m >= M) continue;
      for (int lane = 0; lane < 64; ++lane)
        for (int j = 0; j < nv; ++j) {
          const int c_load = clamp ? norm_vec_index(j, lane, nvec) : 64 * j + lane;
          CHECK(c_load >= 0 && c_load < nvec, "%s: M %d K %d: load of vector %d of a row of %d (row %d, lane %d, register %d): %d bytes past the row",
                what, M, K, c_load, nvec, m, lane, j, (c_load - nvec + 1) * 16);
          ++n;
          if (!norm_vec_in_row(j, lane, nvec)) continue;
          const int c = 64 * j + lane, off = mid_norm_store_offset(c, m, row_step);
          const bool in = off >= 0 && off % 8 == 0 && off + 8 <= rows_bytes;
          CHECK(in, "%s: M %d K %d: store of row %d vector %d at %d of %d", what, M, K, m, c, off, rows_bytes);
          if (!in) continue;
          for (int e = 0; e < 4; ++e) {
            CHECK(lds.who[off / 2 + e] == -1, "%s: M %d K %d: row %d element %d lands on row %d element %d", what, M, K, m, 4 * c + e,
                  lds.who[off / 2 + e] >> 16, lds.who[off / 2 + e] & 0xffff);
            lds.who[off / 2 + e] = m * 65536 + 4 * c + e;
          }
          ++n;
        }
    }
  // the product's reads: the waves that work on block 0 (the only block with rows)
  for (int wave = 0; wave < S::NW; ++wave) {
    const int b0 = mid_first_block<S>(wave);
    if (b0 >= 1) continue;                                         // (NRB is 1 with NORM)
    for (int ks = 0; ks < K / 64; ++ks)
      for (int lane = 0; lane < 64; ++lane)
        for (int kk = 0; kk < 2; ++kk) {
          const int r = lane & 15, g = lane >> 4;
          const int off = mid_norm_read_offset(ks, b0, row_step, r, g, kk);
          const bool in = off >= 0 && off % 16 == 0 && off + 16 <= rows_bytes;
          CHECK(in, "%s: M %d K %d: read of lane %d step %d at %d of %d", what, M, K, lane, ks, off, rows_bytes);
          ++n;
          if (!in || r >= M) continue;                             // rows past M: whatever LDS holds, never stored
          for (int e = 0; e < 8; ++e) {
            const int want = r * 65536 + 64 * ks + 32 * kk + 8 * g + e;
            CHECK(lds.who[off / 2 + e] == want, "%s: M %d K %d: lane %d step %d half %d reads row %d element %d, wants row %d element %d", what, M,
                  K, lane, ks, kk, lds.who[off / 2 + e] >> 16, lds.who[off / 2 + e] & 0xffff, r, want & 0xffff);
          }
        }
  }
  return n;
}

// every (M, K) the launcher admits for this instantiation, with the choices the kernel makes
template <class S>
static long sweep_mid_norm(const char* what, bool eight) {
  long n = 0;
  for (int K = 64; K <= 2 * GEMM_SEG; K += 64) {
    const bool whole_stages = K % (64 * S::SUB) == 0;
    // launch_mid: the eight-wave variant where K is whole stages of it, else the four-wave one
    if (eight != whole_stages && eight) continue;
    if (!eight) {
      // the four-wave variant runs only where the eight-wave one of the same product does not take K
      // (its SUB is 2 for narrow tiles and 1 otherwise)
      using E = MidShape<S::ROPE_NARROW ? EPI_QKV_ROPE : (S::GLU ? EPI_SWIGLU_BF16 : EPI_F32), 1, true, S::ROPE_NARROW, true>;
      if (K % (64 * E::SUB) == 0) continue;
    }
    for (int M = 1; M <= 16; ++M) {
      if (!mid_norm_admits(M, K, 64)) continue;
      const int row_step = mid_norm_row_step(K);
      n += sweep_mid_norm_launch<S>(what, M, K, mid_norm_rows_a_wave(M, S::NW), mid_norm_vectors_a_lane(K), row_step,
                                    mid_norm_lds_bytes(S::RING, K, row_step), true);
    }
  }
  return n;
}

// ------------------------------------------------------------------------------ decode_gemm_kernel
static long sweep_decode(int waves, int stages, int stage_bytes, int rope_lw) {
  long n = 0;
  for (int K = 64; K <= DEC_SEG; K += 64)
    for (int M = 1; M <= 16; ++M) {
      if (!decode_gemm_admits(M, 16, K, K)) continue;
      const size_t lds = decode_lds_bytes(M, K, waves, stages, stage_bytes);
      if (lds > DEC_MAX_LDS) continue;                              // the launcher refuses (-2)
      const size_t rows_elems = (size_t)M * decode_lds_row(K);
      CHECK(rows_elems * 2 <= decode_rows_bytes(M, K), "decode: rows of M %d K %d", M, K);
      std::vector<int32_t> who(rows_elems, -1);
      const int nvec = K / 4, rows_a_wave = (M + waves - 1) / waves;
      CHECK(8 * 64 >= nvec, "decode: K %d has %d vectors, a lane holds 8", K, nvec);
      for (int wave = 0; wave < waves; ++wave)
        for (int m = wave; m < M; m += waves)                       // rows dealt round robin, rows_a_wave (at most 4) at a time
          for (int c = 0; c < nvec; ++c) {
            const size_t e0 = decode_norm_store_elem(m, c, K);
            const bool in = e0 % 4 == 0 && e0 + 4 <= rows_elems;
            CHECK(in, "decode: M %d K %d store of row %d vector %d at element %zu of %zu", M, K, m, c, e0, rows_elems);
            if (!in) continue;
            for (int e = 0; e < 4; ++e) {
              CHECK(who[e0 + e] == -1, "decode: M %d K %d two stores at element %zu", M, K, e0 + e);
              who[e0 + e] = m * 65536 + 4 * c + e;
            }
            ++n;
          }
      (void)rows_a_wave;                                            // (more than four rows a wave: the kernel takes them four at a time)
      for (int step = 0; step < K / 64; ++step)
        for (int lane = 0; lane < 64; ++lane)
          for (int kk = 0; kk < 2; ++kk) {
            const int r = lane & 15, g = lane >> 4;
            const size_t e0 = decode_operand_elem(r, M, g, step, kk, K);
            CHECK(e0 == decode_operand_elem(r, M, g, 0, 0, K) + 64 * step + 32 * kk, "decode: the operand address is not linear in the step");
            const bool in = e0 % 8 == 0 && e0 + 8 <= rows_elems;
            CHECK(in, "decode: M %d K %d read of lane %d step %d at element %zu of %zu", M, K, lane, step, e0, rows_elems);
            ++n;
            if (!in) continue;
            const int row = r < M ? r : 0;
            for (int e = 0; e < 8; ++e)
              CHECK(who[e0 + e] == row * 65536 + 64 * step + 32 * kk + 8 * g + e, "decode: M %d K %d lane %d step %d reads row %d element %d", M, K,
                    lane, step, who[e0 + e] >> 16, who[e0 + e] & 0xffff);
          }
      for (int wave = 0; wave < waves; ++wave) {
        const size_t ring = decode_ring_offset(M, K, wave, stages, stage_bytes);
        CHECK(ring % 16 == 0 && ring >= rows_elems * 2 && ring + (size_t)stages * stage_bytes <= lds, "decode: ring of wave %d at %zu of %zu", wave, ring, lds);
        for (int lane = 0; lane < 64; ++lane)
          for (int kk = 0; kk < 2; ++kk) {
            const int off = decode_ring_operand_offset(lane & 15, lane >> 4, kk);
            CHECK(off >= 0 && off + 16 <= 2048, "decode: ring operand read at %d", off);
            ++n;
          }
      }
      // the rotary epilogue parks M rows of rope_lw 32-bit products where the rows were (the launcher checks the row size)
      if (rope_lw && (size_t)rope_lw * 4 <= (size_t)decode_lds_row(K) * 2)
        CHECK((size_t)M * rope_lw * 4 <= decode_rows_bytes(M, K), "decode: rotary epilogue of M %d K %d", M, K);
    }
  return n;
}

int main() {
  std::printf("ok row-vectors-8 %ld\n", sweep_row_vectors(8, GEMM_SEG));
  std::printf("ok row-vectors-16 %ld\n", sweep_row_vectors(16, 2 * GEMM_SEG));

  long ring = 0;
#define RING(EPI, NRB, NORM, NARROW, EIGHT) ring += sweep_mid_ring<MidShape<EPI, NRB, NORM, NARROW, EIGHT>, NRB>(#EPI " " #NRB " " #NORM " " #NARROW " " #EIGHT)
  // every instantiation the launchers name: plain epilogues, SwiGLU and the rotary one, 1, 2 and 4 blocks of rows,
  // narrow tiles where they exist, four and eight waves where launch_mid picks between them
  RING(EPI_F32, 1, true, false, true);  RING(EPI_BF16, 1, true, false, true);  RING(EPI_ADD_F32, 1, true, false, true);
  RING(EPI_SWIGLU_BF16, 1, true, false, true);
  RING(EPI_F32, 1, true, false, false); RING(EPI_SWIGLU_BF16, 1, true, false, false);
  RING(EPI_QKV_ROPE, 1, true, false, true);  RING(EPI_QKV_ROPE, 1, true, false, false);
  RING(EPI_QKV_ROPE, 1, true, true, true);   RING(EPI_QKV_ROPE, 1, true, true, false);
  RING(EPI_F32, 1, false, false, false); RING(EPI_SWIGLU_BF16, 1, false, false, false); RING(EPI_ADD_F32, 1, false, false, false);
  RING(EPI_F32, 2, false, false, false); RING(EPI_F32, 2, false, false, true); RING(EPI_F32, 4, false, false, false); RING(EPI_F32, 4, false, false, true);
  RING(EPI_SWIGLU_BF16, 2, false, false, false); RING(EPI_SWIGLU_BF16, 2, false, false, true);
  RING(EPI_SWIGLU_BF16, 4, false, false, false); RING(EPI_SWIGLU_BF16, 4, false, false, true);
  RING(EPI_ADD_F32, 2, false, true, false); RING(EPI_ADD_F32, 2, false, true, true); RING(EPI_ADD_F32, 4, false, true, false); RING(EPI_ADD_F32, 4, false, true, true);
  RING(EPI_QKV_ROPE, 1, false, false, false); RING(EPI_QKV_ROPE, 2, false, false, false); RING(EPI_QKV_ROPE, 2, false, false, true);
  RING(EPI_QKV_ROPE, 4, false, false, false); RING(EPI_QKV_ROPE, 4, false, false, true);
  RING(EPI_QKV_ROPE, 1, false, true, false); RING(EPI_QKV_ROPE, 2, false, true, false); RING(EPI_QKV_ROPE, 2, false, true, true);
  RING(EPI_QKV_ROPE, 4, false, true, false); RING(EPI_QKV_ROPE, 4, false, true, true);
  std::printf("ok mid-ring %ld\n", ring);

  long rows = 0;
  rows += sweep_mid_norm<MidShape<EPI_F32, 1, true, false, true>>("norm+product, 64 columns, eight waves", true);
  rows += sweep_mid_norm<MidShape<EPI_SWIGLU_BF16, 1, true, false, true>>("norm+gate|up, eight waves", true);
  rows += sweep_mid_norm<MidShape<EPI_QKV_ROPE, 1, true, false, true>>("norm+q|k|v, a head a workgroup, eight waves", true);
  rows += sweep_mid_norm<MidShape<EPI_QKV_ROPE, 1, true, true, true>>("norm+q|k|v, half a head a workgroup, eight waves", true);
  rows += sweep_mid_norm<MidShape<EPI_QKV_ROPE, 1, true, true, false>>("norm+q|k|v, half a head a workgroup, four waves", false);
  rows += sweep_mid_norm<MidShape<EPI_F32, 1, true, false, false>>("norm+product, 64 columns, four waves", false);
  std::printf("ok mid-norm-rows %ld\n", rows);

  long dec = 0;
  dec += sweep_decode(4, 8, 2048, 0);       // plain epilogues: four strips a workgroup, eight stages
  dec += sweep_decode(4, 4, 4096, 0);       // SwiGLU: gate and up strip a stage, four stages
  dec += sweep_decode(2, 10, 2048, 32);     // rotary, a strip and its partner
  for (int w = 1; w <= 4; ++w) dec += sweep_decode(w, 10, 2048, 16 * w);   // rotary, a whole head of 16 w
  std::printf("ok decode-rows %ld\n", dec);
  const long in_library = failures;

  // ---------------------------------------------------------------------------- the variant that was taken out
  // Rows of up to 4096 elements in every fused kernel, up to 16 rows, two rows a wave, sixteen vectors a lane.
  // (a) with the library's layout of 16-row blocks (2048 bytes a step): what the launch would ask of LDS
  using S = MidShape<EPI_SWIGLU_BF16, 1, true, false, true>;
  const int lds_a = mid_norm_lds_bytes(S::RING, 4096, 2048);
  std::printf("note removed-variant 16 rows x 4096 in 16-row blocks: %d bytes of LDS (limit %d): %s\n", lds_a, BW_LDS_LIMIT,
              lds_a > BW_LDS_LIMIT ? "the launch is refused before any kernel runs" : "fits");
  const size_t lds_d = decode_lds_bytes(16, 4096, 4, 8, 2048);
  std::printf("note removed-variant 16 rows x 4096 in the few-columns kernel: %zu bytes of LDS (limit %d): %s\n", lds_d, DEC_MAX_LDS,
              lds_d > (size_t)DEC_MAX_LDS ? "refused" : "fits");
  // (b) sixteen vectors a lane applied to rows of one segment too (K <= 2048), loads not clamped into the row:
  // the farthest byte a lane reads past its row and past the norm's weights
  failures = 0;
  quiet = true;
  long before = failures;
  sweep_mid_norm_launch<S>("removed variant, unclamped", 16, 2048, 2, 16, 2048, mid_norm_lds_bytes(S::RING, 2048, 2048), false);
  std::printf("note removed-variant unclamped, 16 rows x 2048 with sixteen vectors a lane: %ld loads leave their row, the farthest %d bytes past its end "
              "(of the residual stream's last row and of the norm's weights: past the allocation)\n", failures - before, (64 * 15 + 63 - 512 + 1) * 16);
  failures = 0;
  sweep_mid_norm_launch<S>("removed variant, clamped", 16, 2048, 2, 16, 2048, mid_norm_lds_bytes(S::RING, 2048, 2048), true);
  std::printf("note removed-variant clamped, 16 rows x 2048 with sixteen vectors a lane: %ld failures\n", failures);
  failures = 0;
  sweep_mid_norm_launch<S>("removed variant, 8 rows x 4096, 16-row blocks", 8, 4096, 1, 16, 2048, mid_norm_lds_bytes(S::RING, 4096, 2048), true);
  std::printf("note removed-variant 8 rows x 4096 in 16-row blocks: %ld failures (LDS %d bytes)\n", failures, mid_norm_lds_bytes(S::RING, 4096, 2048));

  std::printf("%s in-library failures %ld\n", in_library ? "FAIL" : "ok", in_library);
  return in_library ? 1 : 0;
}
