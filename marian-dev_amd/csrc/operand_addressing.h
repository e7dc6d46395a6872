// Where the GEMM kernels read their operands: every byte offset a lane computes for a weight or
// activation load, as functions that compile for the host as well.  The kernels call them, and a
// CPU program (tests/addressing_check.cpp) walks all lanes, waves, tiles and K steps of edge shapes
// through the same functions and checks that every 16-byte load stays inside its operand.
#pragma once

#include <stddef.h>
#include <stdint.h>

#if !defined(__HIPCC__)
#define __host__
#define __device__
#define __forceinline__ inline
#endif

namespace marian_hip {

__host__ __device__ __forceinline__ int addr_min(int a, int b) { return a < b ? a : b; }

// Prepared weights ("K-blocked"): the K*N int8 values of W^T are stored by K sub-step of 32 values;
// within a sub-step the N columns follow each other, 32 bytes (the sub-step's 32 K values) each:
//   byte of (column n, k) = (k / 32) * 32 * N + n * 32 + k % 32
// The operand of one matrix instruction for 32 (or 16) consecutive columns is then 1 KB (512 bytes)
// of consecutive memory, which a wave fetches with one fully coalesced load; advancing along K adds
// 32 * N bytes for every column alike.  (With the plain [N x K] rows every lane of such a load reads
// a different 128-byte line: the address unit then takes four times as long per load, measured as
// 2 k of 16 k clocks of the dominant decode call.  A gathered column - shortlist - still finds the
// two 16-byte halves of a sub-step side by side.)
__host__ __device__ __forceinline__ unsigned b_column_offset(int n) { return (unsigned)n * 32u; }
// 16-byte chunk k16 (K values 16 * k16 .. + 15) of column n
__host__ __device__ __forceinline__ size_t b_chunk_offset(int n, int k16, int N) {
  return (size_t)(k16 >> 1) * 32u * (size_t)N + b_column_offset(n) + (unsigned)(k16 & 1) * 16u;
}

// ---- small-M kernels on 32x32x32 instructions (gemm_stream32_kernel, proj_attention_kernel) ----
// Lane (li, lg) of the wave that owns output columns n0 .. n0 + 31 reads half lg of column
// min(n0 + li, n_out - 1) (through the shortlist ids when there are any), sub-step after sub-step.
__host__ __device__ __forceinline__ int stream32_lane_column(int n0, int li, int n_out) {
  return addr_min(n0 + li, n_out - 1);
}
__host__ __device__ __forceinline__ unsigned stream32_lane_offset(int src_column, int lg) {
  return b_column_offset(src_column) + (unsigned)lg * 16u;
}
// A chunk is CS sub-steps; wave kw of the K split takes sub-steps kw * PW .. + PW - 1 of it.  When
// they all exist the loads use one pointer and constant offsets, otherwise every sub-step is
// clamped to the last one (and its weights are replaced by zeros afterwards).
__host__ __device__ __forceinline__ bool stream32_chunk_is_whole(int chunk, int CS, int kw, int PW, int S) {
  return chunk * CS + (kw + 1) * PW <= S;
}
__host__ __device__ __forceinline__ int stream32_clamped_substep(int s, int S) { return addr_min(s, S - 1); }

// ---- small-M kernel on 16x16x64 instructions (gemm_stream_kernel) ----
// Lane (li, lg) reads 16-byte chunk lg of a K step of 64 of column n (column 0 stands in for columns
// past the output; K steps past the end are not loaded at all).
__host__ __device__ __forceinline__ size_t stream16_lane_offset(int src_column, int lg, int N) {
  return b_chunk_offset(src_column, lg, N);
}

// ---- large-M kernels (gemm_mfma32_kernel, gemm_pair_kernel): global -> LDS staging ----
// Activations: load j of wave `wave` (of `waves`) fills rows (j * waves + wave) * 8 .. + 7 of a stage;
// a lane takes the 16-byte chunk that the XOR swizzle of its row puts at its place.  Rows past the
// matrix re-read the last one.  Offset within a K block of 128 bytes.
__host__ __device__ __forceinline__ int stage_a_row(int j, int waves, int wave, int lane) {
  return (j * waves + wave) * 8 + lane / 8;
}
__host__ __device__ __forceinline__ int stage_a_chunk(int row, int lane) { return (lane % 8) ^ ((row >> 1) & 7); }
__host__ __device__ __forceinline__ int stage_a_offset(int j, int waves, int wave, int lane, int m0, int M, int K) {
  const int row = stage_a_row(j, waves, wave, lane);
  return addr_min(m0 + row, M - 1) * K + stage_a_chunk(row, lane) * 16;
}
// A last block of 64 instead of 128 columns has no chunks 4 .. 7: such lanes go 64 bytes back.
// (The chunk of a lane is the same for all its loads when the number of waves is even.)
__host__ __device__ __forceinline__ int stage_a_tail_adjust(int wave, int lane) {
  return stage_a_chunk(stage_a_row(0, 0, wave, lane), lane) >= 4 ? 64 : 0;
}
// Weights: load g of a stage brings sub-step g / tiles_n of the 32 columns of tile g % tiles_n; lane q
// fetches half q >> 5 of column q & 31 of the tile (clamped to the last output column).
__host__ __device__ __forceinline__ int stage_b_column(int g, int tiles_n, int lane, int n0, int n_out) {
  return addr_min(n0 + (g % tiles_n) * 32 + (lane & 31), n_out - 1);
}
__host__ __device__ __forceinline__ size_t stage_b_offset(int g, int tiles_n, int lane, int src_column, int N) {
  return b_chunk_offset(src_column, 2 * (g / tiles_n) + (lane >> 5), N);
}
// A last block of 64 columns has no sub-steps 2, 3: such loads go two sub-steps (64 * N bytes) back.
__host__ __device__ __forceinline__ bool stage_b_goes_back(int g, int tiles_n) { return g / tiles_n >= 2; }

// ---- projections + attention in one launch (proj_attention_kernel): which input rows a workgroup takes ----
// Caches that are complete and shared - `sentences` entries per head, row m attends to sentence
// m % sentences, M = hypotheses * sentences - let a workgroup take `per_wg` hypotheses of
// 1 << shift neighbouring sentences (per_wg << shift <= 8) instead of eight consecutive rows, so
// that the waves reading the same keys and values sit on one CU; the hypotheses of a sentence are
// taken in `chunks` of per_wg.  Row r of a workgroup: hypothesis chunk * per_wg + (r >> shift) of
// sentence first + (r & ((1 << shift) - 1)); rows whose hypothesis does not exist are idle.
// shift < 0: eight consecutive rows.
struct ProjRowPlan {
  int shift;       // log2 of the sentences per workgroup, or -1
  int sentences;
  int hyps;        // hypotheses per sentence
  int per_wg;      // hypotheses of a sentence a workgroup takes
  int stage;       // the sentences' keys and values are staged in LDS (shift 0 or 1, len <= stage_len)
  long long blocks_y;   // workgroups per head
};
__host__ __device__ __forceinline__ ProjRowPlan proj_row_plan(long long n_proj, long long M, long long heads, long long batchKV,
                                                              long long len, int stage_len, size_t lds_without,
                                                              size_t lds_max) {
  ProjRowPlan plan = {-1, 0, 0, 0, 0, (M + 7) / 8};
  if(n_proj != 1 || heads <= 0 || batchKV % heads != 0) return plan;
  const long long nb = batchKV / heads;
  if(nb <= 0 || nb >= M || M % nb != 0 || nb > 2147483647LL) return plan;
  const long long hyps = M / nb;
  if(hyps > 2147483647LL) return plan;
  // the fewest workgroups (each reads the head's weights), then the fewest chunks (each reads the
  // sentences' keys and values); two hypotheses a sentence keep four sentences per workgroup
  int best_shift = -1, best_per = 0;
  long long best_blocks = 0, best_chunks = 0;
  for(int shift = 2; shift >= 0; --shift) {
    if(nb % (1 << shift) != 0) continue;
    const int room = 8 >> shift;                        // hypotheses a workgroup has rows for
    const long long chunks = (hyps + room - 1) / room;
    const int per = (int)((hyps + chunks - 1) / chunks);
    if(per < 2 || (per << shift) < 4) continue;         // (at least half of a workgroup's rows in use)
    if(shift == 2 && hyps != 2) continue;               // (four sentences are not staged: only where nothing else fits)
    const long long blocks = chunks * (nb >> shift);
    if(best_shift < 0 || blocks < best_blocks || (blocks == best_blocks && chunks < best_chunks)) {
      best_shift = shift; best_per = per; best_blocks = blocks; best_chunks = chunks;
    }
  }
  if(best_shift < 0) return plan;
  plan.shift = best_shift;
  plan.sentences = (int)nb;
  plan.hyps = (int)hyps;
  plan.per_wg = best_per;
  plan.blocks_y = best_blocks;
  const size_t kv_bytes = (size_t)(2 << best_shift) * (size_t)len * 256;
  plan.stage = best_shift <= 1 && len <= stage_len && lds_without + kv_bytes <= lds_max;
  return plan;
}
// input row r (0 .. 7) of workgroup block_y; rows that do not exist: a value of at least M (= hyps * sentences)
__host__ __device__ __forceinline__ int proj_row_of(int shift, int sentences, int hyps, int per_wg, int block_y, int r) {
  if(shift < 0) return block_y * 8 + r;
  const int groups = sentences >> shift;
  const int j = r >> shift, hyp = (block_y / groups) * per_wg + j;
  if(j >= per_wg || hyp >= hyps) return 0x7fffffff;
  return hyp * sentences + ((block_y % groups) << shift) + (r & ((1 << shift) - 1));
}
// first sentence of workgroup block_y (shift >= 0)
__host__ __device__ __forceinline__ int proj_first_sentence(int shift, int sentences, int block_y) {
  return (block_y % (sentences >> shift)) << shift;
}

}  // namespace marian_hip
