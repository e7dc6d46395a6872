// CPU walk over the operand addresses of the GEMM kernels.  The byte offsets, the clamps at the
// matrix edges and the detours of a 64-column last K block come from the header the kernels
// themselves compile (marian-dev_amd/csrc/operand_addressing.h); this program supplies what a
// launch supplies - grid, waves, lanes, loads per wave, K steps - for edge shapes and checks that
//   * every 16-byte load lies inside its operand (weights: K * N bytes, activations: M * K bytes),
//   * an activation load stays inside the row it was clamped to,
//   * the loads that are multiplied (not clamped duplicates, not detours) cover every 16-byte
//     chunk of the columns / rows of the tile exactly once.
// Built and run by tests/test_operand_addressing.py; prints one line per kernel family.
#include <cstdio>
#include <cstdlib>
#include <vector>

#include "operand_addressing.h"

using namespace marian_hip;

static long long g_checked = 0;
static int g_failures = 0;

static void fail(const char* what, long long off, long long limit, const char* where) {
  if(g_failures < 20) std::fprintf(stderr, "FAIL %s: offset %lld (+16) vs limit %lld in %s\n", what, off, limit, where);
  ++g_failures;
}

static void inside(long long off, long long limit, const char* what, const char* where) {
  ++g_checked;
  if(off < 0 || off + 16 > limit) fail(what, off, limit, where);
}

// shortlists of n_out ids out of N columns: the first, the last and a spread
static std::vector<std::vector<uint32_t>> shortlists(int N, int n_out) {
  std::vector<std::vector<uint32_t>> r(3);
  for(int i = 0; i < n_out; ++i) {
    r[0].push_back((uint32_t)i);
    r[1].push_back((uint32_t)(N - n_out + i));
    r[2].push_back((uint32_t)((long long)i * (N - 1) / (n_out > 1 ? n_out - 1 : 1)));
  }
  return r;
}

// ---- gemm_stream32_kernel<MT32, WN, KW, PW, ...>: weights straight into registers ----
static void stream32(int WN, int KW, int PW, int K, int N, const std::vector<uint32_t>* idx) {
  char where[160];
  const int n_out = idx ? (int)idx->size() : N;
  const int S = K / 32, CS = PW * KW, n_chunks = (S + CS - 1) / CS;
  const int gx = (n_out + WN * 32 - 1) / (WN * 32);
  const long long bytes = (long long)K * N;
  std::snprintf(where, sizeof where, "stream32 WN=%d KW=%d PW=%d K=%d N=%d n_out=%d", WN, KW, PW, K, N, n_out);
  std::vector<int> seen((size_t)n_out * 2 * S, 0);   // (output column, 16-byte chunk of K)
  for(int bx = 0; bx < gx; ++bx)
    for(int wn = 0; wn < WN; ++wn)
      for(int kw = 0; kw < KW; ++kw)
        for(int lane = 0; lane < 64; ++lane) {
          const int li = lane % 32, lg = lane / 32;
          const int n0 = (bx * WN + wn) * 32;
          const int col = stream32_lane_column(n0, li, n_out);
          const int src = idx ? (int)(*idx)[col] : col;
          const long long lane_off = stream32_lane_offset(src, lg);
          for(int chunk = 0; chunk < n_chunks; ++chunk) {
            const bool whole = stream32_chunk_is_whole(chunk, CS, kw, PW, S);
            for(int p = 0; p < PW; ++p) {
              const int s = chunk * CS + kw * PW + p;
              const int s_load = whole ? s : stream32_clamped_substep(s, S);
              inside(lane_off + (long long)s_load * 32 * N, bytes, "weights", where);
              if(s < S && n0 + li < n_out) ++seen[((size_t)(n0 + li) * S + s) * 2 + lg];   // multiplied
            }
          }
        }
  for(size_t i = 0; i < seen.size(); ++i)
    if(seen[i] != 1) { fail("coverage", (long long)i, seen[i], where); break; }
}

// ---- gemm_stream_kernel<MT, NT, WN, KW, PF>: 16x16x64 instructions ----
static void stream16(int NT, int WN, int KW, int PF, int K, int N, const std::vector<uint32_t>* idx) {
  char where[160];
  const int n_out = idx ? (int)idx->size() : N;
  const int KS = K / 64, chunk_steps = PF * KW, n_chunks = (KS + chunk_steps - 1) / chunk_steps;
  const int cols = WN * NT * 16, gx = (n_out + cols - 1) / cols;
  const long long bytes = (long long)K * N;
  std::snprintf(where, sizeof where, "stream16 NT=%d WN=%d KW=%d PF=%d K=%d N=%d n_out=%d", NT, WN, KW, PF, K, N, n_out);
  std::vector<int> seen((size_t)n_out * 4 * KS, 0);
  for(int bx = 0; bx < gx; ++bx)
    for(int wn = 0; wn < WN; ++wn)
      for(int kw = 0; kw < KW; ++kw)
        for(int lane = 0; lane < 64; ++lane)
          for(int nt = 0; nt < NT; ++nt) {
            const int li = lane % 16, lg = lane / 16;
            const int n = (bx * WN + wn) * NT * 16 + nt * 16 + li;
            int src = 0;
            if(n < n_out) src = idx ? (int)(*idx)[n] : n;
            const long long lane_off = (long long)stream16_lane_offset(src, lg, N);
            for(int chunk = 0; chunk < n_chunks; ++chunk)
              for(int p = 0; p < PF; ++p) {
                const int s = chunk * chunk_steps + p * KW + kw;
                if(s >= KS) continue;   // not loaded
                inside(lane_off + (long long)s * 64 * N, bytes, "weights", where);
                if(n < n_out) ++seen[((size_t)n * KS + s) * 4 + lg];
              }
          }
  for(size_t i = 0; i < seen.size(); ++i)
    if(seen[i] != 1) { fail("coverage", (long long)i, seen[i], where); break; }
}

// ---- gemm_mfma32_kernel<BM, BN, WAVES_M, WAVES_N, ...>: operands staged through LDS ----
static void staged(int BM, int BN, int waves, int M, int K, int N, const std::vector<uint32_t>* idx) {
  char where[160];
  const int n_out = idx ? (int)idx->size() : N;
  const int BK = 128, tiles_n = BN / 32;
  const int loads = (BM + BN) / 8 / waves, loads_a = BM / 8 / waves;
  const bool half = K % BK != 0;          // K % 128 == 64: a last block of 64 columns
  const int KB = (K + BK - 1) / BK;
  const long long a_bytes = (long long)M * K, b_bytes = (long long)K * N;
  std::snprintf(where, sizeof where, "staged %dx%d waves=%d M=%d K=%d N=%d n_out=%d", BM, BN, waves, M, K, N, n_out);
  for(int m0 = 0; m0 < M; m0 += BM)
    for(int n0 = 0; n0 < n_out; n0 += BN) {
      std::vector<int> seen_a((size_t)BM * (K / 16), 0), seen_b((size_t)BN * (K / 16), 0);
      for(int wave = 0; wave < waves; ++wave)
        for(int lane = 0; lane < 64; ++lane)
          for(int j = 0; j < loads; ++j)
            for(int kb = 0; kb < KB; ++kb) {
              const bool last_half = half && kb == KB - 1;
              if(j < loads_a) {
                const int row = stage_a_row(j, waves, wave, lane);
                const int chunk = stage_a_chunk(row, lane);
                long long off = (long long)kb * BK + stage_a_offset(j, waves, wave, lane, m0, M, K);
                const bool detour = last_half && stage_a_tail_adjust(wave, lane) != 0;
                if(last_half) off -= stage_a_tail_adjust(wave, lane);
                // (the adjustment of a lane must be the one its chunk asks for, whatever the load index)
                if(last_half && (chunk >= 4) != detour) fail("tail adjust vs chunk", off, chunk, where);
                inside(off, a_bytes, "activations", where);
                const int m = addr_min(m0 + row, M - 1);
                if(off / K != m || off % K + 16 > K) fail("activation load leaves its row", off, (long long)m * K, where);
                if(!detour && m0 + row < M) ++seen_a[(size_t)row * (K / 16) + kb * 8 + chunk];
              } else {
                const int g = (j - loads_a) * waves + wave;
                const int col = stage_b_column(g, tiles_n, lane, n0, n_out);
                const int src = idx ? (int)(*idx)[col] : col;
                long long off = (long long)kb * BK * N + (long long)stage_b_offset(g, tiles_n, lane, src, N);
                const bool detour = last_half && stage_b_goes_back(g, tiles_n);
                if(detour) off -= 64LL * N;
                inside(off, b_bytes, "weights", where);
                const int c = n0 + (g % tiles_n) * 32 + (lane & 31);
                if(!detour && c < n_out) ++seen_b[(size_t)(c - n0) * (K / 16) + kb * 8 + 2 * (g / tiles_n) + (lane >> 5)];
              }
            }
      for(int r = 0; r < BM && m0 + r < M; ++r)
        for(int c16 = 0; c16 < K / 16; ++c16)
          if(seen_a[(size_t)r * (K / 16) + c16] != 1) { fail("activation coverage", r, c16, where); r = BM; break; }
      for(int c = 0; c < BN && n0 + c < n_out; ++c)
        for(int c16 = 0; c16 < K / 16; ++c16)
          if(seen_b[(size_t)c * (K / 16) + c16] != 1) { fail("weight coverage", c, c16, where); c = BN; break; }
    }
}

// The rows the workgroups of the one-launch projections + attention take: every row exactly once,
// the rows of a workgroup that share a sentence slot attend to that sentence, and every staged
// key/value load (and LDS slot) lies inside the caches (the staging area).
static void proj_rows(long long hyps, long long sentences, long long heads, long long len, long long cap) {
  const long long M = hyps * sentences, batchKV = sentences * heads;
  const int stage_len = 96;
  const size_t lds_without = 32 * 1024 + 8 * 8 * 128 + 8 * 64 * 4 + 8 * (size_t)(((len + 3) & ~3LL) + 256) * 4;
  const size_t lds_max = 160 * 1024 - 256;
  const ProjRowPlan plan = proj_row_plan(1, M, heads, batchKV, len, stage_len, lds_without, lds_max);
  char where[160];
  std::snprintf(where, sizeof(where), "proj rows hyps %lld sentences %lld len %lld shift %d per %d stage %d", hyps, sentences,
                len, plan.shift, plan.per_wg, plan.stage);
  const int blocks = (int)plan.blocks_y;
  if(plan.shift < 0 && plan.blocks_y != (M + 7) / 8) fail("workgroups of the plain form", plan.blocks_y, (M + 7) / 8, where);
  if(plan.shift >= 0 && ((plan.per_wg << plan.shift) > 8 || (plan.per_wg << plan.shift) < 4 || plan.hyps != hyps))
    fail("hypotheses per workgroup", plan.per_wg, plan.shift, where);
  std::vector<int> seen((size_t)M, 0);
  for(int by = 0; by < blocks; ++by)
    for(int r = 0; r < 8; ++r) {
      const int m = proj_row_of(plan.shift, plan.sentences, plan.hyps, plan.per_wg, by, r);
      ++g_checked;
      if(m < 0) { fail("negative row", by, r, where); continue; }
      if(m >= M) continue;   // rows past the end are skipped by the kernel
      ++seen[(size_t)m];
      if(plan.shift >= 0) {
        const int slot = r & ((1 << plan.shift) - 1);
        const int sentence = proj_first_sentence(plan.shift, plan.sentences, by) + slot;
        if(sentence >= sentences || m % sentences != sentence) fail("row outside its sentence", by, r, where);
        if(plan.stage) {   // the loads of segment 2 * slot (keys) and 2 * slot + 1 (values)
          const long long entry = (long long)sentence * heads + (heads - 1);
          const long long last = (entry * cap + (len - 1)) * 64 + 63;
          if(entry >= batchKV || last >= batchKV * cap * 64) fail("staged load outside the cache", by, r, where);
          const size_t lds_end = lds_without + (size_t)(2 * slot + 2) * (size_t)len * 256;
          if(lds_end > lds_max) fail("staging area past the LDS", by, r, where);
          if(plan.shift > 1 || len > stage_len) fail("staged beyond what the kernels hold", by, r, where);
        }
      }
    }
  for(long long m = 0; m < M; ++m)
    if(seen[(size_t)m] != 1) { fail("row coverage", (int)m, seen[(size_t)m], where); break; }
}

int main() {
  const int Ks[] = {64, 192, 576, 1088, 1024};
  const int Ns[] = {8, 24, 1000, 1032};
  // (WN, KW, PW) of the small-M instantiations in use
  const int s32[][3] = {{1, 4, 4}, {4, 2, 8}, {1, 8, 2}, {1, 8, 8}, {2, 4, 8}, {1, 8, 4}, {4, 1, 8}, {1, 4, 8}, {2, 2, 8}};
  for(auto& c : s32)
    for(int K : Ks)
      for(int N : Ns) {
        stream32(c[0], c[1], c[2], K, N, nullptr);
        for(auto& sl : shortlists(N, 8)) stream32(c[0], c[1], c[2], K, N, &sl);
      }
  std::printf("stream32: %lld loads checked\n", g_checked);
  long long before = g_checked;
  // (NT, WN, KW, PF)
  const int s16[][4] = {{1, 1, 4, 2}, {1, 2, 4, 2}, {2, 1, 4, 2}, {1, 4, 2, 2}, {1, 1, 8, 1}};
  for(auto& c : s16)
    for(int K : Ks)
      for(int N : Ns) {
        stream16(c[0], c[1], c[2], c[3], K, N, nullptr);
        for(auto& sl : shortlists(N, 8)) stream16(c[0], c[1], c[2], c[3], K, N, &sl);
      }
  std::printf("stream16: %lld loads checked\n", g_checked - before);
  before = g_checked;
  // (BM, BN, waves): whole tiles and the edge tiles of the ragged launches
  const int big[][3] = {{128, 128, 4}, {128, 128, 8}, {256, 256, 8}, {128, 64, 4}, {64, 128, 4}, {64, 128, 8}, {128, 64, 8}, {256, 128, 4}};
  const int Ms[] = {129, 130, 257, 300};
  for(auto& c : big)
    for(int M : Ms)
      for(int K : Ks)
        for(int N : Ns) {
          if(c[0] == 256 && c[1] == 256 && K % 128 != 0) continue;   // no 64-column last block in this form
          staged(c[0], c[1], c[2], M, K, N, nullptr);
          if(N >= 1000)
            for(auto& sl : shortlists(N, 8)) staged(c[0], c[1], c[2], M, K, N, &sl);
        }
  std::printf("staged: %lld loads checked\n", g_checked - before);
  before = g_checked;
  for(long long hyps : {1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 12, 16, 17})
    for(long long sentences : {1, 2, 3, 4, 5, 8, 10, 32, 33})
      for(long long len : {1, 31, 32, 33, 60, 96, 97, 300})
        proj_rows(hyps, sentences, 16, len, len + 3);
  std::printf("projection rows: %lld rows checked\n", g_checked - before);
  if(g_failures) {
    std::fprintf(stderr, "%d failures\n", g_failures);
    return 1;
  }
  std::printf("ok\n");
  return 0;
}
