// Compute-bound int8 GEMM for large M (encoder shapes): 32x32x32 i8 MFMA, operands streamed
// global -> LDS without passing through registers.
//
// v_mfma_i32_32x32x32_i8 is the int8 instruction that runs at the full matrix rate on gfx950
// (32 cycles for 32x32x32 MACs; the 16x16x64 form issues at roughly half that rate).  Operand
// traffic into a CU (about 64 bytes per clock through the vector L1) is the limit, so a
// workgroup owns a large BM x BN output tile and each operand byte enters the CU once per tile:
//   * K advances in 128-byte blocks.  A row of a block is one full 128-byte line of the
//     activations in global memory.  One global_load_lds_dwordx4 per wave moves 8 rows (1 KB)
//     straight into LDS; the lane that fills 16-byte slot p of row r fetches chunk p ^ ((r >> 1) & 7)
//     of that row, so LDS holds each row with its chunks XOR-swizzled and the MFMA fragment reads
//     (32 consecutive rows, one chunk each) are bank-conflict free.  The K-blocked weights need no
//     swizzle: 32 columns x one sub-step are 1 KB of consecutive memory in operand order, one wave
//     load brings them into LDS in the lane order of the operand, and a fragment read covers that
//     1 KB once.
//   * NSTAGE LDS buffers; the loads of block k + NSTAGE are issued as soon as block k has been
//     read, so they have NSTAGE - 1 blocks of MFMA time to land.
//   * Fragments are double-buffered in registers: the ds_reads of sub-step s + 1 (also across
//     the barrier into the next block) are issued before the MFMAs of sub-step s.
// Activations are the row operand and weights the column operand, so a lane ends up with one
// output column and the 32 lanes of a half-wave write 128 contiguous bytes of an output row.
// Requires K % 128 == 0.
#pragma once

#include <type_traits>

#include "int8_common.h"
#include "quantize_kernels.h"

namespace marian_hip {

typedef int v16i __attribute__((ext_vector_type(16)));

template <int BM_, int BN_, int WAVES_M, int WAVES_N, int NSTAGE_>
struct BigCfg {
  static constexpr int BM = BM_, BN = BN_, BK = 128, NSTAGE = NSTAGE_;
  static constexpr int kWaves = WAVES_M * WAVES_N;
  static constexpr int kThreads = kWaves * kWave;
  static constexpr int WTM = BM / WAVES_M / 32;  // 32x32 MFMA tiles per wave along m
  static constexpr int WTN = BN / WAVES_N / 32;  // and along n
  static constexpr int kRows = BM + BN;
  static constexpr int kStageBytes = kRows * BK;
  static constexpr int kGroups = kRows / 8;            // 8-row groups, one wave load each
  static constexpr int kLoads = kGroups / kWaves;      // loads per wave per K block
  static constexpr int kLoadsA = (BM / 8) / kWaves;    // the first of them are activation rows
  static constexpr int kLdsBytes = NSTAGE * kStageBytes;
  // A last K block of 64 columns is supported unless the eight-wave 256x256 tile is chosen: that
  // one uses 242 of its 256 registers and the few more that the half block needs made it spill.
  static constexpr bool kHalfTailOk = !(BM == 256 && BN == 256 && kWaves == 8);
  static_assert((BM / 8) % kWaves == 0 && (BN / 8) % kWaves == 0, "tile rows vs waves");
  static_assert(BM % (WAVES_M * 32) == 0 && BN % (WAVES_N * 32) == 0, "tile vs wave grid");
  static_assert(NSTAGE >= 2 && NSTAGE <= 4, "two to four LDS stages (four: the split form only)");
};

// s_waitcnt with only vmcnt (up to 63) or only lgkmcnt constrained (gfx9 encoding).
template <int N>
__device__ __forceinline__ void wait_vmcnt() {
  __builtin_amdgcn_s_waitcnt((N & 0xF) | ((N >> 4) << 14) | (0x7 << 4) | (0xF << 8));
}
__device__ __forceinline__ void wait_lgkmcnt0() { __builtin_amdgcn_s_waitcnt(0xC07F); }

// 16 bytes per lane from global memory straight into LDS: lane l of the wave writes LDS bytes
// lds_addr + 16*l .. +15 (lds_addr is wave-uniform and travels in M0).  Issued as inline assembly
// on purpose: for the builtin form the compiler assumes that every later LDS read may alias the
// incoming data and inserts s_waitcnt vmcnt(0) in front of it, which serialises the K pipeline.
// Completion is tracked by hand with vmcnt (loads and stores of a wave retire in issue order).
__device__ __forceinline__ void global_load_lds16(const void* gptr, unsigned lds_addr) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off"
               :
               : "s"(lds_addr), "v"(gptr)
               : "memory", "m0");
}

// The same with the address as a wave-uniform 64-bit base (scalar registers) plus a 32-bit unsigned
// per-lane offset: advancing along K then changes only the scalar base, no vector arithmetic per load.
__device__ __forceinline__ void global_load_lds16(const void* sbase, unsigned voff, unsigned lds_addr) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
               :
               : "s"(lds_addr), "v"(voff), "s"(sbase)
               : "memory", "m0");
}

// Writes one 32x32 accumulator tile.  Element v of the tile is row 8*(v/4) + 4*(lane/32) + v%4,
// column lane%32; `out` points at this lane's element of tile row 4*(lane/32).
//   y = float(acc) * unquant (+ bias) ; relu: y > 0 ? y : 0   (mul and add round separately)
template <bool DUMP, bool BIAS, bool RELU, bool GUARD>
__device__ __forceinline__ void store_tile32(const v16i& acc, char* out, size_t row_bytes,
                                             float unquant, float bias_v, int rows_left,
                                             bool col_valid) {
#pragma unroll
  for(int v = 0; v < 16; ++v) {
    const int r = 8 * (v / 4) + (v % 4);
    if(GUARD && (!col_valid || r >= rows_left)) continue;
    char* p = out + (size_t)r * row_bytes;
    if(DUMP) {
      *reinterpret_cast<int32_t*>(p) = acc[v];
    } else {
      float y = (float)acc[v] * unquant;
      if(BIAS) y = y + bias_v;
      if(RELU) y = y > 0.0f ? y : 0.0f;
      *reinterpret_cast<float*>(p) = y;
    }
  }
}

// The WTN 32x32 tiles that sit side by side in a wave's output, written row by row: for every
// accumulator row the stores of the WTN tiles follow each other, so that consecutive stores of a
// wave cover WTN * 128 contiguous bytes of an output row (measured on the store burst alone: tile
// after tile is 50 % slower).  `out` points at this lane's element of row 4*(lane/32) of the first
// tile; tile b starts 128 bytes further per b.
// AMAX: also keeps the maximum of |y| over what this lane stores in `omax` (one more vector
// operation per value; only calls that hand their abs-max to the next call ask for it).
template <int WTN, bool DUMP, bool BIAS, bool RELU, bool GUARD, bool NT, bool AMAX>
__device__ __forceinline__ void store_tiles32_rowwise(const v16i (&acc)[WTN], char* out, size_t row_bytes,
                                                      float unquant, const float (&bias_v)[WTN],
                                                      int rows_left, const bool (&col_valid)[WTN], float& omax) {
#pragma unroll
  for(int v = 0; v < 16; ++v) {
    const int r = 8 * (v / 4) + (v % 4);
    if(GUARD && r >= rows_left) continue;
    char* row = out + (size_t)r * row_bytes;
#pragma unroll
    for(int b = 0; b < WTN; ++b) {
      if(GUARD && !col_valid[b]) continue;
      char* p = row + b * 128;
      if(DUMP) {
        *reinterpret_cast<int32_t*>(p) = acc[b][v];
      } else {
        float y = (float)acc[b][v] * unquant;
        if(BIAS) y = y + bias_v[b];
        if(RELU) y = y > 0.0f ? y : 0.0f;
        if(AMAX) omax = fmaxf(omax, fabsf(y));
        if(NT) __builtin_nontemporal_store(y, reinterpret_cast<float*>(p));
        else *reinterpret_cast<float*>(p) = y;
      }
    }
  }
}

template <int WTN, bool GUARD, bool NT, bool AMAX>
__device__ __forceinline__ void store_tiles32_rowwise_any(const v16i (&acc)[WTN], char* out, size_t row_bytes,
                                                          float unquant, const float (&bias_v)[WTN],
                                                          int rows_left, const bool (&col_valid)[WTN],
                                                          int dump, bool bias, int relu, float& omax) {
  if(dump) store_tiles32_rowwise<WTN, true, false, false, GUARD, NT, false>(acc, out, row_bytes, unquant, bias_v, rows_left, col_valid, omax);
  else if(bias && relu) store_tiles32_rowwise<WTN, false, true, true, GUARD, NT, AMAX>(acc, out, row_bytes, unquant, bias_v, rows_left, col_valid, omax);
  else if(bias) store_tiles32_rowwise<WTN, false, true, false, GUARD, NT, AMAX>(acc, out, row_bytes, unquant, bias_v, rows_left, col_valid, omax);
  else if(relu) store_tiles32_rowwise<WTN, false, false, true, GUARD, NT, AMAX>(acc, out, row_bytes, unquant, bias_v, rows_left, col_valid, omax);
  else store_tiles32_rowwise<WTN, false, false, false, GUARD, NT, AMAX>(acc, out, row_bytes, unquant, bias_v, rows_left, col_valid, omax);
}

template <bool GUARD>
__device__ __forceinline__ void store_tile32_any(const v16i& acc, char* out, size_t row_bytes,
                                                 float unquant, float bias_v, int rows_left,
                                                 bool col_valid, int dump, bool bias, int relu) {
  if(dump) store_tile32<true, false, false, GUARD>(acc, out, row_bytes, unquant, bias_v, rows_left, col_valid);
  else if(bias && relu) store_tile32<false, true, true, GUARD>(acc, out, row_bytes, unquant, bias_v, rows_left, col_valid);
  else if(bias) store_tile32<false, true, false, GUARD>(acc, out, row_bytes, unquant, bias_v, rows_left, col_valid);
  else if(relu) store_tile32<false, false, true, GUARD>(acc, out, row_bytes, unquant, bias_v, rows_left, col_valid);
  else store_tile32<false, false, false, GUARD>(acc, out, row_bytes, unquant, bias_v, rows_left, col_valid);
}

// PAIRED: fragments of two K sub-steps are requested two sub-steps ahead (four fragment sets in
// registers; needed when a sub-step has only a few MFMAs to cover the LDS latency).  Otherwise the
// fragments of sub-step s+1 are requested during sub-step s (two sets; for large wave tiles, whose
// accumulators leave no room for four).
// NT: the outputs are written with non-temporal stores.  An output that fits the L2 caches would
// otherwise sit there dirty until the end of the kernel and be written back then, after the last
// workgroup, in one piece (measured: 24.1 instead of 25.6 us for a 16 MB output; a 64 MB output
// does not fit anyway and is 2 % slower with them).
// HALF: K is a multiple of 64 but not of 128, the last block holds 64 columns (an instantiation of
// its own, so that whole-block calls run code without the checks).
// XCD-aware tile order: workgroups of one XCD (ids congruent mod 8 under round-robin dispatch)
// take a compact block of tiles - 4 tiles along n by a run along m - so that the XCD's L2 holds
// few weight panels and few activation panels at a time.
__device__ __forceinline__ void xcd_tile(int tiles_n, int tiles_m, int block, int& tn, int& tm) {
  const int total = tiles_n * tiles_m;
  int t = block;
  if(total % 8 == 0) t = (block % 8) * (total / 8) + block / 8;
  const int band = 4;
  const int b = t / (band * tiles_m);
  const int r = t % (band * tiles_m);
  const int bw = (tiles_n - b * band) < band ? (tiles_n - b * band) : band;
  tn = b * band + r % bw;
  tm = r / bw;
}

// Abs-max hand-over of a large-M launch: slot `slot` receives the maximum of |y| over the tile this
// workgroup stored (omax: this lane's share), the workgroup of slot 0 zeroes the slots past the
// `used` ones the launch fills.  red: the LDS ring, free once every wave is past its last fragment
// read (the first barrier).  All threads of the workgroup call it.
__device__ __forceinline__ void publish_tile_absmax(float omax, float* absmax_out, int slot, int used, float* red) {
  const int tid = threadIdx.x, lane = tid % kWave, wave = tid / kWave, nw = blockDim.x / kWave;
  omax = wave_max(omax);
  __syncthreads();
  if(lane == 0) red[wave] = omax;
  __syncthreads();
  if(tid == 0) {
    float m = red[0];
    for(int w = 1; w < nw; ++w) m = fmaxf(m, red[w]);
    absmax_out[slot] = m;
  }
  if(slot == 0)
    for(int sl = used + tid; sl < kAbsmaxSlots; sl += (int)blockDim.x) absmax_out[sl] = 0.0f;
}

// One BM x BN output tile at rows m0 .., columns n0 .. (any multiples of 32; the tile may hang over
// the edge of the output).  slot: the workgroup's number among the tiles of the launch (abs-max
// slot, clock record).
// SPLIT: the workgroup has twice the waves of the tile's wave grid.  The first WAVES_M * WAVES_N waves
// multiply and never touch global memory before the write-out; the others ("loaders", one more wave
// per SIMD) issue every global -> LDS load of the tile and wait for them.  Both kinds meet at the one
// workgroup barrier per K block, which says "block kb + 1 has landed" and "stage kb is free" at once.
// The multiplying waves then spend no issue slots on loads and their waits (measured with the
// instruction mixes alone: 90 % instead of 63 % matrix-instruction issue for the 128 x 128 tile).
// Whole blocks only (no HALF).
template <int BM, int BN, int WAVES_M, int WAVES_N, int NSTAGE, bool PAIRED = true, bool NT = false,
          bool HALF = false, bool AMAX = false, bool SPLIT = false>
__device__ __forceinline__ void gemm_mfma32_tile(const GemmArgs& args, const int m0, const int n0, int8_t* lds,
                                                 const int slot) {
  using Cfg = BigCfg<BM, BN, WAVES_M, WAVES_N, NSTAGE>;
  const unsigned lds_base = (unsigned)(size_t)lds;  // LDS byte address of the ring

  const long long t_start = MH_CLOCK();
  const long long w_start = MH_WALL();
  const int tid = threadIdx.x;
  static_assert(!SPLIT || (PAIRED && !HALF), "the split form exists for whole blocks of the paired-fragment form");
  const int wave_of_group = __builtin_amdgcn_readfirstlane(tid / kWave);
  const bool loader = SPLIT && wave_of_group >= Cfg::kWaves;
  const int wave = loader ? wave_of_group - Cfg::kWaves : wave_of_group;   // its number among its kind
  const int lane = tid % kWave;
  const int wm = wave / WAVES_N, wn = wave % WAVES_N;
  const int li = lane % 32, lg = lane / 32;
  const int K = args.K, M = args.M;
  // K is a multiple of 64: the last block may hold 64 columns only (PAIRED form; the launcher sends
  // other K to the plain form only as whole blocks).  Its loads stay inside the rows, see tail_adj.
  static_assert(!HALF || (PAIRED && Cfg::kHalfTailOk), "no half last block in this form");
  const int KB = HALF ? (K + Cfg::BK - 1) / Cfg::BK : K / Cfg::BK;
  constexpr bool half_tail = HALF;

  // ---- global -> LDS: load j of this wave fills rows (j*kWaves + wave)*8 .. +7 of a stage.
  // Rows past the matrix edge re-read the last valid row; their products are never stored.
  // Weights: load g = (j - kLoadsA) * kWaves + wave of a stage brings sub-step g / (BN/32) of the 32
  // columns of tile g % (BN/32): 1 KB that is consecutive in the K-blocked weights (consecutive g:
  // consecutive memory).  Lane q fetches half q >> 5 of column q & 31 of the tile, so the block sits
  // in LDS in the lane order of the matrix operand and a fragment read is 1 KB of consecutive LDS
  // (no bank conflicts).  With a shortlist the lanes gather their
  // columns.
  constexpr int kTilesN = BN / 32;
  int goff[Cfg::kLoads];
#pragma unroll
  for(int j = 0; j < Cfg::kLoads; ++j) {
    if(j < Cfg::kLoadsA) {
      goff[j] = stage_a_offset(j, Cfg::kWaves, wave, lane, m0, M, K);
    } else {
      const int g = (j - Cfg::kLoadsA) * Cfg::kWaves + wave;
      const int n = stage_b_column(g, kTilesN, lane, n0, args.n_out);
      const int src = args.idx ? (int)args.idx[n] : n;
      goff[j] = (int)stage_b_offset(g, kTilesN, lane, src, args.N);   // (K * N < 2^31)
    }
  }
  const size_t b_block = (size_t)Cfg::BK * (size_t)args.N;   // bytes of all columns per K block
  // A half last block: the lanes of the upper four 16-byte chunks of a row would read past the
  // row (past the buffer, for the last row), so they re-read the lower half instead; what they
  // stage is never multiplied.  The chunk of a lane is the same for all its loads (the number of
  // waves is even, so (row >> 1) & 7 does not depend on j).
  static_assert(Cfg::kWaves % 2 == 0, "the chunk of a lane must not depend on the load index");
  const int tail_adj = stage_a_tail_adjust(wave, lane);
  auto issue_one = [&](int kb, int stage, int j, auto check_tail) __attribute__((always_inline)) {
    const bool is_a = j < Cfg::kLoadsA;
    const int8_t* base = is_a ? args.Aq + (size_t)kb * Cfg::BK : args.Bq + (size_t)kb * b_block;
    int voff = goff[j];
    // (a half block has no chunks 4 .. 7 and no sub-steps 2, 3: such loads go two sub-steps back, 64
    // bytes of an activation row or 64 * N bytes of the weights; what they stage is never multiplied)
    if(decltype(check_tail)::value && half_tail && kb == KB - 1) {
      if(is_a) voff -= tail_adj;
      else if(stage_b_goes_back((j - Cfg::kLoadsA) * Cfg::kWaves + wave, kTilesN)) voff -= 64 * args.N;
    }
    global_load_lds16(base, (unsigned)voff,
                      lds_base + stage * Cfg::kStageBytes + (j * Cfg::kWaves + wave) * 1024);
  };
  auto issue = [&](int kb) {
    const int stage = kb % NSTAGE;
#pragma unroll
    for(int j = 0; j < Cfg::kLoads; ++j) issue_one(kb, stage, j, std::true_type());
  };

  // ---- fragment addressing: lane (li, lg) reads row li of a 32-row activation tile, chunk kk*2 + lg;
  //      of the weights, its 16 bytes of the 1 KB block (sub-step kk, column tile), see above ----
  int frag_off[4];
#pragma unroll
  for(int kk = 0; kk < 4; ++kk) frag_off[kk] = li * 128 + (((kk * 2 + lg) ^ ((li >> 1) & 7)) * 16);
  const int a_row0 = wm * Cfg::WTM * 32;          // first activation row of this wave in a stage
  // this lane's 16 bytes of sub-step 0 of the wave's first column tile
  const int b_frag0 = BM * 128 + wn * Cfg::WTN * 1024 + lane * 16;

  v4i af[PAIRED ? 4 : 2][Cfg::WTM], bf[PAIRED ? 4 : 2][Cfg::WTN];
  auto read_frags = [&](int stage, int kk, int set) {
    const int8_t* buf = lds + stage * Cfg::kStageBytes + frag_off[kk];
#pragma unroll
    for(int a = 0; a < Cfg::WTM; ++a)
      af[set][a] = *reinterpret_cast<const v4i*>(buf + (a_row0 + a * 32) * 128);
    const int8_t* bbuf = lds + stage * Cfg::kStageBytes + b_frag0 + kk * kTilesN * 1024;
#pragma unroll
    for(int b = 0; b < Cfg::WTN; ++b) bf[set][b] = *reinterpret_cast<const v4i*>(bbuf + b * 1024);
  };

  // fragment `idx` of the pair of sub-steps (0, 1): idx = set * (WTM + WTN) + f
  auto read_one = [&](int stage, int idx) {
    const int set = idx / (Cfg::WTM + Cfg::WTN), f = idx % (Cfg::WTM + Cfg::WTN);
    const int8_t* buf = lds + stage * Cfg::kStageBytes;
    if(f < Cfg::WTM)
      af[set][f] = *reinterpret_cast<const v4i*>(buf + frag_off[set] + (a_row0 + f * 32) * 128);
    else
      bf[set][f - Cfg::WTM] = *reinterpret_cast<const v4i*>(buf + b_frag0 + (set * kTilesN + f - Cfg::WTM) * 1024);
  };

  v16i acc[Cfg::WTM][Cfg::WTN];
#pragma unroll
  for(int a = 0; a < Cfg::WTM; ++a)
#pragma unroll
    for(int b = 0; b < Cfg::WTN; ++b)
#pragma unroll
      for(int v = 0; v < 16; ++v) acc[a][b][v] = 0;
  // Sub-steps 2 and 3 of a block as 2 * WTM * WTN slots of one MFMA each.  Every slot first issues
  // its share of the global->LDS loads of block kb + NSTAGE and of the LDS reads of the next
  // block's sub-steps 0 and 1; their issue time then hides under the MFMA of the previous slot.
  // (The loads are inline assembly, so the order is pinned slot by slot.)
  auto second_half = [&](auto steady_c, bool may_issue, int kb) __attribute__((always_inline)) {
    // steady: block kb + NSTAGE exists, its loads are issued without a branch between the MFMAs
    const bool do_issue = !SPLIT && (decltype(steady_c)::value || may_issue);
    constexpr int nM = Cfg::WTM * Cfg::WTN;
    constexpr int LPS = (Cfg::kLoads + 2 * nM - 1) / (2 * nM);
    constexpr int nR = 2 * (Cfg::WTM + Cfg::WTN);
    constexpr int RPS = (nR + nM - 1) / nM;
    const int ld_stage = (kb + NSTAGE) % NSTAGE, rd_stage = (kb + 1) % NSTAGE;
#pragma unroll
    for(int slot = 0; slot < 2 * nM; ++slot) {
      if(do_issue) {   // wave-uniform: only the load is skipped, the MFMA code exists once
#pragma unroll
        for(int l = 0; l < LPS; ++l)
          if(slot * LPS + l < Cfg::kLoads)
            issue_one(kb + NSTAGE, ld_stage, slot * LPS + l, std::integral_constant<bool, !decltype(steady_c)::value>());
      }
      if(slot < nM) {
#pragma unroll
        for(int r = 0; r < RPS; ++r)
          if(slot * RPS + r < nR) read_one(rd_stage, slot * RPS + r);
      }
      const int set = slot < nM ? 2 : 3, i = slot % nM, a = i / Cfg::WTN, b = i % Cfg::WTN;
      acc[a][b] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[set][a], bf[set][b], acc[a][b], 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  auto multiply = [&](int set) {
#pragma unroll
    for(int a = 0; a < Cfg::WTM; ++a)
#pragma unroll
      for(int b = 0; b < Cfg::WTN; ++b)
        acc[a][b] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[set][a], bf[set][b], acc[a][b], 0, 0, 0);
  };
  // Scheduler hints.  The fragments of sub-steps 2,3 (and of sub-steps 0,1 of the next block)
  // are requested two sub-steps ahead, `reads_per_mfma` LDS reads after each MFMA of an even
  // sub-step, so that they have a whole odd sub-step of MFMA time to arrive.
  auto interleave = [&]() {
    constexpr int kMfma = Cfg::WTM * Cfg::WTN;
    constexpr int kReads = 2 * (Cfg::WTM + Cfg::WTN);
    constexpr int kPer = (kReads + kMfma - 1) / kMfma;
#pragma unroll
    for(int i = 0; i < kMfma; ++i) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);     // one MFMA
      __builtin_amdgcn_sched_group_barrier(0x100, kPer, 0);  // then a few DS reads
    }
  };
  auto mfma_only = [&]() { __builtin_amdgcn_sched_group_barrier(0x008, Cfg::WTM * Cfg::WTN, 0); };

  // (SPLIT) what a loader wave does instead of everything up to the write-out: all loads of the tile,
  // each K block waited for before the barrier that hands it to the multiplying waves.  `ahead`
  // blocks issued after the one waited for may still be in flight (loads retire in issue order).
  auto wait_for_block = [&](int ahead) {
    if(ahead >= 3) wait_vmcnt<3 * Cfg::kLoads>();
    else if(ahead == 2) wait_vmcnt<2 * Cfg::kLoads>();
    else if(ahead == 1) wait_vmcnt<Cfg::kLoads>();
    else wait_vmcnt<0>();
  };
  static_assert(!SPLIT || 3 * Cfg::kLoads <= 63, "vmcnt holds 63 at most");
  long long t_prologue = 0;
  if(SPLIT && loader) {
#pragma unroll
    for(int s = 0; s < NSTAGE; ++s)
      if(s < KB) issue(s);
    wait_for_block(min(NSTAGE, KB) - 1);
    __builtin_amdgcn_s_barrier();
    t_prologue = MH_CLOCK();
    for(int kb = 0; kb + 1 < KB; ++kb) {
      const int last_issued = min(kb + NSTAGE - 1, KB - 1);
      wait_for_block(last_issued - (kb + 1));   // block kb + 1 has landed ...
      __builtin_amdgcn_s_barrier();              // ... and nobody reads stage kb any more
      if(kb + NSTAGE < KB) issue(kb + NSTAGE);
    }
  } else {
  // ---- prologue: fill all stages, wait for block 0 only ----
  if constexpr(!SPLIT) {
#pragma unroll
    for(int s = 0; s < NSTAGE; ++s)
      if(s < KB) issue(s);
    if(NSTAGE == 3 && KB >= 3) wait_vmcnt<2 * Cfg::kLoads>();
    else if(KB >= 2) wait_vmcnt<Cfg::kLoads>();
    else wait_vmcnt<0>();
  }
  __builtin_amdgcn_s_barrier();
  t_prologue = MH_CLOCK();
  if constexpr(!PAIRED) {
    auto spread = [&]() {   // one LDS read after each MFMA
#pragma unroll
      for(int i = 0; i < Cfg::WTM + Cfg::WTN; ++i) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
      }
    };
    read_frags(0, 0, 0);
    for(int kb = 0; kb < KB; ++kb) {
      const int stage = kb % NSTAGE;
      read_frags(stage, 1, 1);
      multiply(0);
      spread();
      read_frags(stage, 2, 0);
      multiply(1);
      spread();
      read_frags(stage, 3, 1);
      multiply(0);
      spread();
      if(kb + 1 < KB) {
        __builtin_amdgcn_sched_barrier(0);
        wait_lgkmcnt0();
        if(NSTAGE == 3 && kb + 2 < KB) wait_vmcnt<Cfg::kLoads>();
        else wait_vmcnt<0>();
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
        if(!SPLIT && kb + NSTAGE < KB && !(MH_DBG(args, 1))) issue(kb + NSTAGE);
        read_frags((kb + 1) % NSTAGE, 0, 0);
      }
      multiply(1);
      spread();
    }
  } else {
    read_frags(0, 0, 0);
    read_frags(0, 1, 1);

    auto one_block = [&](int kb, auto steady_c) __attribute__((always_inline)) {
      const int stage = kb % NSTAGE;
      read_frags(stage, 2, 2);
      read_frags(stage, 3, 3);
      multiply(0);
      interleave();
      multiply(1);
      mfma_only();
      // All reads of this block were issued one sub-step ago; once they have returned the stage
      // is free.  Block kb+1 must have landed (this wave's share); later blocks may be in flight.
      __builtin_amdgcn_sched_barrier(0);  // keep the MFMAs above on this side of the wait
      wait_lgkmcnt0();
      if constexpr(!SPLIT) {
        if(NSTAGE == 3 && (decltype(steady_c)::value || kb + 2 < KB)) wait_vmcnt<Cfg::kLoads>();
        else wait_vmcnt<0>();
      }
      __builtin_amdgcn_s_barrier();
      __builtin_amdgcn_sched_barrier(0);
      second_half(steady_c, kb + NSTAGE < KB && !(MH_DBG(args, 1)), kb);
    };
    int kb = 0;
    const int KBsteady = half_tail ? KB - 1 : KB;   // the steady body issues whole blocks only
    if(!(MH_DBG(args, 1)))
      for(; kb + NSTAGE < KBsteady; ++kb) one_block(kb, std::true_type());
    for(; kb + 1 < KB; ++kb) one_block(kb, std::false_type());
    if(half_tail) {   // 64 columns: sub-steps 0 and 1 only
      multiply(0);
      multiply(1);
    } else {
      const int stage = (KB - 1) % NSTAGE;
      read_frags(stage, 2, 2);
      read_frags(stage, 3, 3);
      multiply(0);
      interleave();
      multiply(1);
      mfma_only();
      multiply(2);
      mfma_only();
      multiply(3);
      mfma_only();
    }
  }
  }   // (not a loader wave)

  const long long t_main = MH_CLOCK();
  // ---- epilogue: element v of a 32x32 tile is row 8*(v/4) + 4*lg + v%4, column li ----
  float unquant = 0.0f;
  if(!args.dump) {
    float aqm = tail_quant_mult(args.Aq, (size_t)M * (size_t)K);
    float bqm = tail_quant_mult(args.Bq, (size_t)K * (size_t)args.N);
    unquant = unquant_mult(aqm, bqm, args.scale);
  }
  const bool interior = (m0 + BM <= M) && (n0 + BN <= args.n_out);
  const size_t row_bytes = (size_t)args.n_out * 4;
  const bool has_bias = args.bias != nullptr;
  float omax = 0.0f;
  if(!(MH_DBG(args, 2)) && !loader) {
    const int nw = n0 + wn * Cfg::WTN * 32 + li;   // this lane's column in the first of the wave's tiles
    float bias_v[Cfg::WTN];
    bool nvalid[Cfg::WTN];
#pragma unroll
    for(int b = 0; b < Cfg::WTN; ++b) {
      const int n = nw + b * 32;
      nvalid[b] = n < args.n_out;
      bias_v[b] = 0.0f;
      if(has_bias && nvalid[b] && !args.dump) bias_v[b] = args.bias[args.idx ? args.idx[n] : (uint32_t)n];
    }
    // Use the loaded values once here, ahead of the stores: the compiler then waits for them here.
    // Otherwise, in the edge form, it re-inserts a wait for all vector memory operations behind the
    // lane-wise branches, i.e. every store waits for the one before (measured on the edge
    // workgroups of a 4096 x 4000 output: 41 k instead of 17 k clocks for the write-out).
#pragma unroll
    for(int b = 0; b < Cfg::WTN; ++b) asm volatile("" ::"v"(bias_v[b]));
    asm volatile("" ::"v"(unquant));
#pragma unroll
    for(int a = 0; a < Cfg::WTM; ++a) {
      const int mbase = m0 + (wm * Cfg::WTM + a) * 32 + 4 * lg;
      char* outp = reinterpret_cast<char*>(args.out) + ((size_t)mbase * (size_t)args.n_out + (size_t)nw) * 4;
      if(interior)
        store_tiles32_rowwise_any<Cfg::WTN, false, NT, AMAX>(acc[a], outp, row_bytes, unquant, bias_v, 32, nvalid, args.dump, has_bias, args.relu, omax);
      else
        store_tiles32_rowwise_any<Cfg::WTN, true, NT, AMAX>(acc[a], outp, row_bytes, unquant, bias_v, M - mbase, nvalid, args.dump, has_bias, args.relu, omax);
    }
  }
  if(!(MH_DBG(args, 2)) && AMAX && args.absmax_out && !args.dump)   // (all waves: it has barriers)
    publish_tile_absmax(omax, args.absmax_out, slot, args.absmax_used, reinterpret_cast<float*>(lds));
  if(MH_PROF(args) && tid == 0) {
    long long* p = MH_PROF(args) + (size_t)slot * 8;
    p[0] = t_start; p[1] = t_prologue; p[2] = t_main; p[3] = MH_CLOCK(); p[6] = w_start; p[7] = MH_WALL();
  }
}

template <int BM, int BN, int WAVES_M, int WAVES_N, int NSTAGE, bool PAIRED = true, bool NT = false,
          bool HALF = false, bool AMAX = false>
__global__ __launch_bounds__(WAVES_M * WAVES_N * kWave) void gemm_mfma32_kernel(
    GemmArgs args, int tiles_n, int tiles_m) {
  extern __shared__ __attribute__((aligned(16))) int8_t lds[];
  int tn, tm;
  xcd_tile(tiles_n, tiles_m, blockIdx.x, tn, tm);
  gemm_mfma32_tile<BM, BN, WAVES_M, WAVES_N, NSTAGE, PAIRED, NT, HALF, AMAX>(args, tm * BM, tn * BN, lds, blockIdx.x);
}

template <int BM, int BN, int WAVES_M, int WAVES_N, int NSTAGE, bool NT = false, bool AMAX = false>
__global__ __launch_bounds__(2 * WAVES_M * WAVES_N * kWave) void gemm_mfma32_split_kernel(
    GemmArgs args, int tiles_n, int tiles_m) {
  extern __shared__ __attribute__((aligned(16))) int8_t lds[];
  int tn, tm;
  xcd_tile(tiles_n, tiles_m, blockIdx.x, tn, tm);
  gemm_mfma32_tile<BM, BN, WAVES_M, WAVES_N, NSTAGE, true, NT, false, AMAX, true>(args, tm * BM, tn * BN, lds, blockIdx.x);
}

// A launch whose output is not a whole number of main tiles: `main_tiles` whole BM x BN tiles
// (the first workgroups, in the XCD-aware order), then small tiles over the rows below them (EBM x
// EBN tiles: a strip `bottom_tiles_n` tiles wide over all columns, starting at row main_tiles_m * BM)
// and over the columns to their right (RBM x RBN tiles, `right_tiles_m` tiles high, starting at
// column main_tiles_n * BN, over the rows of the main tiles).  The few rows or columns past a whole
// number of main tiles then cost a short tail of small tiles instead of a second round of large
// ones.  All three tile shapes run with the same number of waves.
struct RaggedPlan {
  int main_tiles_n, main_tiles_m;
  int bottom_tiles_n, bottom_tiles_m;   // EBM x EBN tiles below the main tiles (all columns)
  int right_tiles_n, right_tiles_m;     // RBM x RBN tiles to the right of the main tiles (main rows only)
  // 0: the small tiles take the workgroup numbers behind the main tiles.  Otherwise (a multiple of
  // eight, at least the number of small tiles): they take the first `lead` numbers - where a main
  // workgroup fills a CU's LDS, the small tiles then run ahead of the main tiles of a few CUs instead
  // of after the main tiles of all (numbers in between are idle; a multiple of eight keeps every main
  // tile on the XCD its number modulo eight names)
  int lead = 0;
};

template <int BM, int BN, int WAVES_M, int WAVES_N, int NSTAGE, int EBM, int EBN, int EWM, int EWN, int ESTAGE,
          int RBM, int RBN, int RWM, int RWN, int RSTAGE, bool NT = false, bool AMAX = false>
__global__ __launch_bounds__(WAVES_M * WAVES_N * kWave) void gemm_mfma32_ragged_kernel(GemmArgs args, RaggedPlan plan) {
  static_assert(WAVES_M * WAVES_N == EWM * EWN && WAVES_M * WAVES_N == RWM * RWN, "one workgroup size");
  extern __shared__ __attribute__((aligned(16))) int8_t lds[];
  const int block = blockIdx.x;
  const int n_main = plan.main_tiles_n * plan.main_tiles_m;
  const int n_bottom = plan.bottom_tiles_n * plan.bottom_tiles_m;
  if(block < n_main) {
    int tn, tm;
    xcd_tile(plan.main_tiles_n, plan.main_tiles_m, block, tn, tm);
    gemm_mfma32_tile<BM, BN, WAVES_M, WAVES_N, NSTAGE, true, NT, false, AMAX>(args, tm * BM, tn * BN, lds, block);
  } else if(block < n_main + n_bottom) {
    const int t = block - n_main;
    const int tn = t % plan.bottom_tiles_n, tm = t / plan.bottom_tiles_n;
    gemm_mfma32_tile<EBM, EBN, EWM, EWN, ESTAGE, true, NT, false, AMAX>(args, plan.main_tiles_m * BM + tm * EBM, tn * EBN, lds, block);
  } else {
    const int t = block - n_main - n_bottom;
    const int tm = t % plan.right_tiles_m, tn = t / plan.right_tiles_m;
    gemm_mfma32_tile<RBM, RBN, RWM, RWN, RSTAGE, true, NT, false, AMAX>(args, tm * RBM, plan.main_tiles_n * BN + tn * RBN, lds, block);
  }
}

}  // namespace marian_hip
