// Persistent compute-bound int8 GEMM for large M (encoder shapes).
//
// One workgroup per CU walks a list of BM x BN output tiles.  The K blocks of all its tiles form
// one continuous stream through a ring of NSTAGE LDS buffers, filled by global_load_lds_dwordx4
// (global -> LDS without passing through registers) NSTAGE blocks ahead, so the first
// operand blocks of the next tile are already in flight while the current tile is finished and
// written out; the output stores of a tile drain while the next tile is multiplied.
//
//   * v_mfma_i32_32x32x32_i8 (32 cycles per 32x32x32 MACs) is the int8 instruction that runs at
//     the full matrix rate on gfx950.
//   * A K block is 128 bytes per row = one full line in global memory (both operands are
//     K-contiguous).  One wave load moves 8 rows (1 KB); the lane that fills 16-byte slot p of
//     row r fetches chunk p ^ ((r >> 1) & 7), so LDS rows are XOR-swizzled and the MFMA fragment
//     reads (32 consecutive rows, one chunk each) are bank-conflict free.
//   * Fragments for two 32-wide K sub-steps are requested two sub-steps ahead and interleaved
//     with MFMAs, so LDS latency is covered by a full sub-step of MFMA time.
//   * Epilogue: each 32x32 accumulator tile is dequantized, transposed through a small per-wave
//     LDS buffer and written as 16-byte stores covering full 128-byte lines of the output rows.
// Activations are the row operand, weights the column operand.  Requires K % 128 == 0.
#pragma once

#include "gemm_mfma32_kernel.h"

namespace marian_hip {

// DIRECT_: write accumulators straight from registers (4-byte stores, a half-wave covers 128 bytes
// of an output row) instead of transposing through LDS; needs no LDS buffer, so two workgroups fit
// on a CU, but its 16 stores per 32x32 tile are too many to count in vmcnt, so the loads of the
// next tile are only confirmed after the stores have retired.
template <int BM_, int BN_, int WAVES_M, int WAVES_N, int NSTAGE_, bool DIRECT_ = false>
struct PersistCfg {
  static constexpr int BM = BM_, BN = BN_, BK = 128, NSTAGE = NSTAGE_;
  static constexpr int kWaves = WAVES_M * WAVES_N;
  static constexpr int kThreads = kWaves * kWave;
  static constexpr int WTM = BM / WAVES_M / 32;
  static constexpr int WTN = BN / WAVES_N / 32;
  static constexpr int kRows = BM + BN;
  static constexpr int kStageBytes = kRows * BK;
  static constexpr int kLoads = (kRows / 8) / kWaves;     // wave loads per K block
  static constexpr int kLoadsA = (BM / 8) / kWaves;
  static constexpr int kStoresPerTile = 4 * WTM * WTN;    // 16-byte stores per lane per tile
  static constexpr bool DIRECT = DIRECT_;
  static constexpr int kEpiBytes = DIRECT ? 0 : kWaves * 4096;   // one 32x32 fp32 tile per wave
  static constexpr int kBiasBytes = 2 * 1024;              // bias of two consecutive tiles
  static constexpr int kLdsBytes = NSTAGE * kStageBytes + kEpiBytes + kBiasBytes;
  static_assert(BN <= 256, "one wave load stages the bias of a tile");
  static_assert((BM / 8) % kWaves == 0 && (BN / 8) % kWaves == 0, "tile rows vs waves");
  static_assert(BM % (WAVES_M * 32) == 0 && BN % (WAVES_N * 32) == 0, "tile vs wave grid");
  static_assert(NSTAGE >= 2 && NSTAGE <= 4, "two to four LDS stages");
  static_assert(DIRECT || (NSTAGE - 2) * kLoads + kStoresPerTile <= 63, "vmcnt is a 6-bit counter");
  static_assert(kLoads % 2 == 0 && kStoresPerTile % 2 == 0, "wait counts are even");
};

// Waits until at most n vector-memory operations of this wave are outstanding (n even, <= 62).
__device__ __forceinline__ void wait_vmcnt_dyn(int n) {
  switch(n >> 1) {
#define MH_CASE(i) case i: wait_vmcnt<2 * i>(); break;
    MH_CASE(0) MH_CASE(1) MH_CASE(2) MH_CASE(3) MH_CASE(4) MH_CASE(5) MH_CASE(6) MH_CASE(7)
    MH_CASE(8) MH_CASE(9) MH_CASE(10) MH_CASE(11) MH_CASE(12) MH_CASE(13) MH_CASE(14) MH_CASE(15)
    MH_CASE(16) MH_CASE(17) MH_CASE(18) MH_CASE(19) MH_CASE(20) MH_CASE(21) MH_CASE(22) MH_CASE(23)
    MH_CASE(24) MH_CASE(25) MH_CASE(26) MH_CASE(27) MH_CASE(28) MH_CASE(29) MH_CASE(30) MH_CASE(31)
#undef MH_CASE
    default: wait_vmcnt<0>(); break;
  }
}

// Tile t of the launch -> tile coordinates.  Workgroups of one XCD (ids congruent mod 8 under
// round-robin dispatch) work at the same time on a compact block of tiles (4 along n by a run
// along m), so that XCD's L2 holds few weight panels and few activation panels at a time.
__device__ __forceinline__ void persistent_tile_coords(int round, int block, int grid, int tiles_n,
                                                       int tiles_m, int& tn, int& tm) {
  int slot = block;
  if(grid % 8 == 0) slot = (block % 8) * (grid / 8) + block / 8;
  const int t = round * grid + slot;
  const int band = 4;
  const int b = t / (band * tiles_m);
  const int r = t % (band * tiles_m);
  const int bw = (tiles_n - b * band) < band ? (tiles_n - b * band) : band;
  tn = b * band + r % bw;
  tm = r / bw;
}

// GATHER selects the shortlist form (weight rows and bias picked through args.idx).  It is a
// separate instantiation because its index and bias reads are ordinary vector loads inside the
// tile loop; the dense form keeps every in-loop load under manual vmcnt control.
template <int BM, int BN, int WAVES_M, int WAVES_N, int NSTAGE, bool GATHER, bool DIRECT = false>
__global__ __launch_bounds__(WAVES_M * WAVES_N * kWave) void gemm_persistent_kernel(
    GemmArgs args, int tiles_n, int tiles_m, int stagger) {
  using Cfg = PersistCfg<BM, BN, WAVES_M, WAVES_N, NSTAGE, DIRECT>;
  extern __shared__ __attribute__((aligned(16))) int8_t lds[];
  const unsigned lds_base = (unsigned)(size_t)lds;  // LDS byte address of the ring

  const long long t_start = MH_CLOCK();
  long long t_epi = 0;
  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);
  const int lane = tid % kWave;
  const int wm = wave / WAVES_N, wn = wave % WAVES_N;
  const int li = lane % 32, lg = lane / 32;
  const int K = args.K, M = args.M;
  const int KB = K / Cfg::BK;
  const int total_tiles = tiles_n * tiles_m;
  const int grid = gridDim.x;
  // tiles of this workgroup: round r -> the (slot of blockIdx)'th tile of [r*grid, (r+1)*grid);
  // the slot permutation is a bijection on [0, grid), so count the rounds whose tile exists
  int my_slot = blockIdx.x;
  if(grid % 8 == 0) my_slot = (blockIdx.x % 8) * (grid / 8) + blockIdx.x / 8;
  const int n_my = (total_tiles - my_slot + grid - 1) / grid;
  const int total_blocks = n_my * KB;

  // ---------------- load side: its own tile cursor, runs NSTAGE - 1 blocks ahead ----------------
  const bool has_bias = args.bias != nullptr && !args.dump;
  const unsigned bias_lds = lds_base + NSTAGE * Cfg::kStageBytes + Cfg::kEpiBytes;
  int goff[Cfg::kLoads];
  int ld_round = 0, ld_kb = 0, ld_count = 0, ld_n0 = 0;
  auto load_tile_setup = [&](int round) {
    int tn, tm;
    persistent_tile_coords(round, blockIdx.x, grid, tiles_n, tiles_m, tn, tm);
    const int m0 = tm * BM, n0 = tn * BN;
    ld_n0 = n0;
#pragma unroll
    for(int j = 0; j < Cfg::kLoads; ++j) {
      const int row = (j * Cfg::kWaves + wave) * 8 + lane / 8;
      const int chunk = (lane % 8) ^ ((row >> 1) & 7);
      int src;
      if(j < Cfg::kLoadsA) {
        src = min(m0 + row, M - 1);   // rows past the edge re-read the last valid row
      } else {
        const int n = min(n0 + row - BM, args.n_out - 1);
        src = GATHER ? (int)args.idx[n] : n;
      }
      goff[j] = src * K + chunk * 16;
    }
  };
  auto issue_next = [&]() {   // loads the next K block of the stream into its ring slot
    const int stage = ld_count % NSTAGE;
#pragma unroll
    for(int j = 0; j < Cfg::kLoads; ++j) {
      const int8_t* base = (j < Cfg::kLoadsA) ? args.Aq : args.Bq;
      const int8_t* src = base + (size_t)(unsigned)goff[j] + (size_t)ld_kb * Cfg::BK;
      global_load_lds16(src, lds_base + stage * Cfg::kStageBytes + (j * Cfg::kWaves + wave) * 1024);
    }
    if(!GATHER && ld_kb == 0 && has_bias && wave == 0) {
      // dense bias of this tile's columns, 256 floats, into the half of the bias buffer that
      // belongs to the tile's parity; retired before the tile's second K block is waited for
      const int n = min(ld_n0 + 4 * lane, args.N - 4);
      global_load_lds16(args.bias + n, bias_lds + (ld_round & 1) * 1024);
    }
    ++ld_count;
    if(++ld_kb == KB) {
      ld_kb = 0;
      ++ld_round;
      if(ld_round < n_my) load_tile_setup(ld_round);
    }
  };

  // ---------------- compute side ----------------
  int frag_off[4];
#pragma unroll
  for(int kk = 0; kk < 4; ++kk) frag_off[kk] = li * 128 + (((kk * 2 + lg) ^ ((li >> 1) & 7)) * 16);
  const int a_row0 = wm * Cfg::WTM * 32;
  const int b_row0 = BM + wn * Cfg::WTN * 32;

  v4i af[4][Cfg::WTM], bf[4][Cfg::WTN];
  auto read_frags = [&](int stage, int kk, int set) {
    const int8_t* buf = lds + stage * Cfg::kStageBytes + frag_off[kk];
#pragma unroll
    for(int a = 0; a < Cfg::WTM; ++a)
      af[set][a] = *reinterpret_cast<const v4i*>(buf + (a_row0 + a * 32) * 128);
#pragma unroll
    for(int b = 0; b < Cfg::WTN; ++b)
      bf[set][b] = *reinterpret_cast<const v4i*>(buf + (b_row0 + b * 32) * 128);
  };
  v16i acc[Cfg::WTM][Cfg::WTN];
  auto zero_acc = [&]() {
#pragma unroll
    for(int a = 0; a < Cfg::WTM; ++a)
#pragma unroll
      for(int b = 0; b < Cfg::WTN; ++b)
#pragma unroll
        for(int v = 0; v < 16; ++v) acc[a][b][v] = 0;
  };
  auto multiply = [&](int set) {
#pragma unroll
    for(int a = 0; a < Cfg::WTM; ++a)
#pragma unroll
      for(int b = 0; b < Cfg::WTN; ++b)
        acc[a][b] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[set][a], bf[set][b], acc[a][b], 0, 0, 0);
  };
  auto interleave = [&]() {   // scheduler hint: a few LDS reads after each MFMA
    constexpr int kMfma = Cfg::WTM * Cfg::WTN;
    constexpr int kReads = 2 * (Cfg::WTM + Cfg::WTN);
    constexpr int kPer = (kReads + kMfma - 1) / kMfma;
#pragma unroll
    for(int i = 0; i < kMfma; ++i) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, kPer, 0);
    }
  };
  auto mfma_only = [&]() { __builtin_amdgcn_sched_group_barrier(0x008, Cfg::WTM * Cfg::WTN, 0); };

  float unquant = 0.0f;
  if(!args.dump) {
    float aqm = tail_quant_mult(args.Aq, (size_t)M * (size_t)K);
    float bqm = tail_quant_mult(args.Bq, (size_t)K * (size_t)args.N);
    unquant = unquant_mult(aqm, bqm, args.scale);
  }
  float* epi = reinterpret_cast<float*>(lds + NSTAGE * Cfg::kStageBytes + wave * 4096);

  // Dequantize one tile's accumulators and write them out.  A 32x32 tile goes through the wave's
  // 4 KB LDS buffer: element v of lane (li, lg) is row 8*(v/4) + 4*lg + v%4, column li; it is read
  // back as rows of 32 floats, 16 bytes per lane, and stored with 8 rows x 128 bytes per store.
  bool last_tile_interior = false;   // every lane of every wave issued all its stores
  auto epilogue = [&](int round) {
    int tn, tm;
    persistent_tile_coords(round, blockIdx.x, grid, tiles_n, tiles_m, tn, tm);
    const int m0 = tm * BM, n0 = tn * BN;
    last_tile_interior = (m0 + BM <= M) && (n0 + BN <= args.n_out) && !(MH_DBG(args, 2));
    if(DIRECT) {
      const bool interior = last_tile_interior;
      const size_t row_bytes = (size_t)args.n_out * 4;
#pragma unroll
      for(int b = 0; b < Cfg::WTN; ++b) {
        const int n = n0 + (wn * Cfg::WTN + b) * 32 + li;
        const bool nvalid = n < args.n_out;
        float bias_v = 0.0f;
        if(has_bias) {
          if(GATHER) {
            bias_v = args.bias[args.idx[min(n, args.n_out - 1)]];
          } else {
            const float* staged = reinterpret_cast<const float*>(lds + NSTAGE * Cfg::kStageBytes + Cfg::kEpiBytes);
            bias_v = staged[(round & 1) * 256 + (wn * Cfg::WTN + b) * 32 + li];
          }
        }
#pragma unroll
        for(int a = 0; a < Cfg::WTM; ++a) {
          const int mbase = m0 + (wm * Cfg::WTM + a) * 32 + 4 * lg;
          char* outp = reinterpret_cast<char*>(args.out) + ((size_t)mbase * (size_t)args.n_out + (size_t)n) * 4;
          if(MH_DBG(args, 2)) continue;
          if(interior)
            store_tile32_any<false>(acc[a][b], outp, row_bytes, unquant, bias_v, 32, true, args.dump, has_bias, args.relu);
          else
            store_tile32_any<true>(acc[a][b], outp, row_bytes, unquant, bias_v, M - mbase, nvalid, args.dump, has_bias, args.relu);
        }
      }
      return;
    }
#pragma unroll
    for(int b = 0; b < Cfg::WTN; ++b) {
      const int ncol0 = n0 + (wn * Cfg::WTN + b) * 32;
      float bias_v = 0.0f;
      if(has_bias) {
        if(GATHER) {
          const int n = min(ncol0 + li, args.n_out - 1);
          bias_v = args.bias[args.idx[n]];
        } else {
          const float* staged = reinterpret_cast<const float*>(lds + NSTAGE * Cfg::kStageBytes + Cfg::kEpiBytes);
          bias_v = staged[(round & 1) * 256 + (wn * Cfg::WTN + b) * 32 + li];
        }
      }
#pragma unroll
      for(int a = 0; a < Cfg::WTM; ++a) {
        const int mrow0 = m0 + (wm * Cfg::WTM + a) * 32;
#pragma unroll
        for(int v = 0; v < 16; ++v) {
          const int r = 8 * (v / 4) + 4 * lg + (v % 4);
          float y;
          if(args.dump) {
            y = __int_as_float(acc[a][b][v]);
          } else {
            y = (float)acc[a][b][v] * unquant;
            if(has_bias) y = y + bias_v;
            if(args.relu) y = y > 0.0f ? y : 0.0f;
          }
          epi[r * 32 + li] = y;
        }
        wait_lgkmcnt0();
#pragma unroll
        for(int q = 0; q < 4; ++q) {
          const int r = q * 8 + lane / 8, c = (lane % 8) * 4;
          v4f y = *reinterpret_cast<const v4f*>(epi + r * 32 + c);
          const int m = mrow0 + r, n = ncol0 + c;
          if(m < M && n < args.n_out && !(MH_DBG(args, 2)))
            *reinterpret_cast<v4f*>(reinterpret_cast<float*>(args.out) + (size_t)m * (size_t)args.n_out + n) = y;
        }
        wait_lgkmcnt0();   // the buffer is rewritten by the next tile
      }
    }
  };

  // ---------------- prologue ----------------
  if(n_my <= 0) return;
  // Two workgroups share a CU; the second half of the grid starts late so that one of the two is
  // in its main loop while the other loads its first blocks or writes a tile out.
  if(stagger > 0 && blockIdx.x >= (unsigned)(grid / 2))
    for(int i = 0; i < stagger; ++i) __builtin_amdgcn_s_sleep(127);
  load_tile_setup(0);
#pragma unroll
  for(int s = 0; s < NSTAGE; ++s)
    if(ld_count < total_blocks) issue_next();
  zero_acc();
  // block 0 has landed once at most the later blocks' loads are outstanding
  wait_vmcnt_dyn((min(total_blocks, NSTAGE) - 1) * Cfg::kLoads);
  __builtin_amdgcn_s_barrier();
  const long long t_prologue = MH_CLOCK();
  read_frags(0, 0, 0);
  read_frags(0, 1, 1);

  int pos = 0, round = 0;       // K block within the tile, tile index of the compute side
  // K blocks since the last tile was written out.  The loads of block g+1 went out at the barrier
  // of block g+1-NSTAGE, so the stores of a tile finished 1 .. NSTAGE-1 blocks ago are younger
  // than them.  (With fewer K blocks per tile than stages several tiles could fall into that
  // window; then the stores are simply waited for.)
  int since_store = NSTAGE;
  const bool count_stores = KB >= NSTAGE && !DIRECT;
  for(int g = 0; g < total_blocks; ++g) {
    const int stage = g % NSTAGE;
    read_frags(stage, 2, 2);
    read_frags(stage, 3, 3);
    multiply(0);
    interleave();
    multiply(1);
    mfma_only();
    const bool more = g + 1 < total_blocks;
    if(more) {
      // All reads of block g were issued a sub-step ago; when they have returned its ring slot
      // may be refilled.  Block g+1 (this wave's share) has landed once only younger vector
      // memory operations remain: the loads of blocks g+2 .. g+NSTAGE-1 and the stores of a tile
      // finished since block g+1 was requested (counted only for a tile that lies fully inside
      // the matrix, where no store is skipped).  Loads and stores retire in issue order; counting
      // too few younger operations only waits longer.
      __builtin_amdgcn_sched_barrier(0);
      wait_lgkmcnt0();
      const int later_blocks = min(NSTAGE - 2, total_blocks - 2 - g);
      const int young_stores =
          (count_stores && last_tile_interior && since_store >= 1 && since_store <= NSTAGE - 1)
              ? Cfg::kStoresPerTile
              : 0;
      wait_vmcnt_dyn(later_blocks * Cfg::kLoads + young_stores);
      __builtin_amdgcn_s_barrier();
      __builtin_amdgcn_sched_barrier(0);
      // block g + NSTAGE takes the ring slot of block g, which every wave has finished reading
      if(ld_count < total_blocks && !(MH_DBG(args, 1))) issue_next();
      read_frags((g + 1) % NSTAGE, 0, 0);
      read_frags((g + 1) % NSTAGE, 1, 1);
    }
    multiply(2);
    interleave();
    multiply(3);
    mfma_only();
    if(since_store < NSTAGE) ++since_store;
    if(++pos == KB) {
      __builtin_amdgcn_sched_barrier(0);
      if(!more) {   // last tile: nothing later has waited for its staged bias yet
        wait_vmcnt<0>();
        __builtin_amdgcn_s_barrier();
      }
      long long te0 = 0;
      if(MH_PROF(args)) te0 = MH_CLOCK();
      epilogue(round);
      if(MH_PROF(args)) t_epi += MH_CLOCK() - te0;
      zero_acc();
      pos = 0;
      ++round;
      since_store = 0;
    }
  }
  if(MH_PROF(args) && tid == 0) {
    long long* p = MH_PROF(args) + (size_t)blockIdx.x * 8;
    p[0] = t_start; p[1] = t_prologue; p[2] = MH_CLOCK() - t_epi; p[3] = MH_CLOCK(); p[4] = t_epi; p[5] = total_blocks;
  }
}

}  // namespace marian_hip
