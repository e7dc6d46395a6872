// Compute-bound int8 GEMM for large M whose fp32 output is most of the bytes (e.g. 4096x1024 times
// 1024x4096: 8 MB of operands, 67 MB of output): the output of one tile is written while the next
// tile is multiplied.
//
// A workgroup of four waves (one per SIMD, up to 512 registers each) computes two 256x128 tiles
// that sit side by side in the output (the same 256 activation rows).  A wave owns a 128x64 piece
// of a tile = 8 accumulator tiles of 32x32 = 128 registers per lane, and there are two such sets:
// while the second tile accumulates into one set, the first tile's set is dequantized and stored,
// one value per lane after every other MFMA of the second tile's last eight K blocks (2 x 128
// values, 8 x 32 MFMAs).  The stores use a wave-uniform row address plus a fixed 32-bit lane offset,
// so a value costs five vector instructions and one store, which fit under the 32 cycles of an MFMA.
// Only the second tile's write-out is exposed.
//
// Operand staging as in the other large-M kernel: K blocks of 128 bytes, global_load_lds_dwordx4
// with XOR-swizzled 16-byte chunks, three LDS stages of 48 KB; the K blocks of the two tiles form
// one stream.  Fragments of two 32-byte sub-steps are requested two sub-steps ahead.  No branch sits
// between two MFMAs: every K block is one of a few straight-line bodies.
//
// Requires: M % 256 == 0, n_out % 256 == 0, K % 128 == 0, K >= 1024, no shortlist, fp32 output.
#pragma once

#include "gemm_mfma32_kernel.h"

namespace marian_hip {

struct PairCfg {
  static constexpr int BM = 256, BN = 128, BK = 128, NSTAGE = 3;
  static constexpr int kWaves = 4, kThreads = kWaves * kWave;
  static constexpr int WTM = 4, WTN = 2;                  // 32x32 tiles per wave
  static constexpr int kStageBytes = (BM + BN) * BK;      // 48 KB
  static constexpr int kLoads = (BM + BN) / 8 / kWaves;   // 12 wave loads per K block
  static constexpr int kLoadsA = BM / 8 / kWaves;         // the first 8 are activation rows
  static constexpr int kRingBytes = NSTAGE * kStageBytes;
  // + per wave: the pair's 256 bias values (1 KB) and the two quantization multipliers (2 x 256 B)
  static constexpr int kLdsBytes = kRingBytes + kWaves * (1024 + 512);
  static constexpr int kSideBlocks = 8;                   // K blocks that carry the first tile's write-out
  static constexpr int kStoresPerBlock = WTM * WTN * 16 / kSideBlocks;   // 16, on the odd MFMA slots
};

// 4-byte store: wave-uniform 64-bit base, 32-bit unsigned lane offset.
template <bool NT>
__device__ __forceinline__ void global_store_f32(const void* sbase, unsigned voff, float y) {
  if(NT) asm volatile("global_store_dword %0, %1, %2 nt" : : "v"(voff), "v"(y), "s"(sbase) : "memory");
  else asm volatile("global_store_dword %0, %1, %2" : : "v"(voff), "v"(y), "s"(sbase) : "memory");
}

// 4 bytes per lane from global memory straight into LDS: lane l writes LDS bytes lds_addr + 4*l .. +3.
__device__ __forceinline__ void global_load_lds4(const void* sbase, unsigned voff, unsigned lds_addr) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, %2"
               :
               : "s"(lds_addr), "v"(voff), "s"(sbase)
               : "memory", "m0");
}

// Vector-memory operations of this wave that are younger than its loads of K block g + 1 when
// side block `kbi` (the kbi-th of the last eight blocks of the stream) reaches its barrier:
// the loads of block g + 2 (issued during block g - 1, blocks 0..4 of the last eight still load)
// and the stores of the first tile issued since (three after the last load of a block, sixteen per
// whole block, eight in the first half of this block).
constexpr int pair_younger_ops(int kbi) {
  int n = 8;
  if(kbi >= 1) n += 16;
  if(kbi >= 2) n += 3;
  if(kbi <= 5) n += PairCfg::kLoads;
  return n;
}

// The two tiles at rows m0 .., columns n0 .. and n0 + 128 .. (whole tiles inside the output).
// slot: the workgroup's number among the workgroups of the launch (abs-max slot, clock record).
// AMAX: the workgroup leaves the maximum of |y| over its two tiles in args.absmax_out[slot].
template <bool NT, bool AMAX>
__device__ __forceinline__ void gemm_pair_tiles(const GemmArgs& args, const int m0, const int n0, int8_t* lds,
                                                const int slot) {
  using Cfg = PairCfg;
  constexpr int BM = Cfg::BM, BN = Cfg::BN, NSTAGE = Cfg::NSTAGE;
  const unsigned lds_base = (unsigned)(size_t)lds;

  const long long t_start = MH_CLOCK();
  const long long w_start = MH_WALL();
  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);
  const int lane = tid % kWave;
  const int wm = wave / 2, wn = wave % 2;
  const int li = lane % 32, lg = lane / 32;
  const int K = args.K;
  const int KB = K / Cfg::BK;
  const int total_blocks = 2 * KB;

  // ---- global -> LDS: activation load j of this wave fills rows (j*4 + wave)*8 .. +7 of a stage;
  //      weight load g = (j - kLoadsA) * 4 + wave brings the 1 KB block (sub-step g / 4, column tile
  //      g % 4) of the K-blocked weights into LDS in operand lane order (see gemm_mfma32_kernel.h) ----
  constexpr int kTilesN = BN / 32;
  unsigned goff[Cfg::kLoads];
#pragma unroll
  for(int j = 0; j < Cfg::kLoads; ++j) {
    if(j < Cfg::kLoadsA) {
      // (whole tiles only: no row or column of a tile lies past the matrix)
      const int row = stage_a_row(j, Cfg::kWaves, wave, lane);
      goff[j] = (unsigned)(m0 + row) * (unsigned)K + stage_a_chunk(row, lane) * 16;
    } else {
      const int g = (j - Cfg::kLoadsA) * Cfg::kWaves + wave;
      goff[j] = (unsigned)stage_b_offset(g, kTilesN, lane, n0 + (g % kTilesN) * 32 + (lane & 31), args.N);
    }
  }
  const int8_t* const b_tile1 = args.Bq + b_column_offset(BN);   // weight columns of the second tile
  const size_t b_block = (size_t)Cfg::BK * (size_t)args.N;        // bytes of all columns per K block
  // K block g of the stream: tile g / KB, block g % KB of its K
  auto issue_one = [&](int g, int stage, int j) __attribute__((always_inline)) {
    const bool second = g >= KB;
    const int kb = second ? g - KB : g;
    const int8_t* base = (j < Cfg::kLoadsA) ? args.Aq + (size_t)kb * Cfg::BK
                                            : (second ? b_tile1 : args.Bq) + (size_t)kb * b_block;
    global_load_lds16(base, goff[j],
                      lds_base + stage * Cfg::kStageBytes + (j * Cfg::kWaves + wave) * 1024);
  };

  // ---- fragments: lane (li, lg) reads row li of a 32-row tile, chunk kk*2 + lg ----
  int frag_off[4];
#pragma unroll
  for(int kk = 0; kk < 4; ++kk) frag_off[kk] = li * 128 + (((kk * 2 + lg) ^ ((li >> 1) & 7)) * 16);
  const int a_row0 = wm * Cfg::WTM * 32;
  // this lane's 16 bytes of sub-step 0 of the wave's first column tile
  const int b_frag0 = BM * 128 + wn * Cfg::WTN * 1024 + lane * 16;
  v4i af[4][Cfg::WTM], bf[4][Cfg::WTN];
  // fragment f (0..5: four activation, two weight) of sub-step / register set kk
  auto read_one = [&](int stage, int kk, int f) __attribute__((always_inline)) {
    const int8_t* buf = lds + stage * Cfg::kStageBytes;
    if(f < Cfg::WTM) af[kk][f] = *reinterpret_cast<const v4i*>(buf + frag_off[kk] + (a_row0 + f * 32) * 128);
    else bf[kk][f - Cfg::WTM] = *reinterpret_cast<const v4i*>(buf + b_frag0 + (kk * kTilesN + f - Cfg::WTM) * 1024);
  };

  // ---- dequantization constants and the write-out addresses of the first tile ----
  const bool has_bias = args.bias != nullptr;
  // max(y, NaN) = y for every y, a NaN included; max(NaN, 0) = 0 like the CPU path's y > 0 ? y : 0
  const float relu_floor = args.relu ? 0.0f : __builtin_nanf("");
  // element e of accumulator tile (a, b): row 32*a + 8*(e/4) + 4*lg + e%4, column 32*b + li
  const unsigned out_voff = ((unsigned)(4 * lg) * (unsigned)args.n_out + (unsigned)li) * 4u;
  const char* const out_base0 = reinterpret_cast<const char*>(args.out) +
      ((size_t)(m0 + wm * Cfg::WTM * 32) * (size_t)args.n_out + (size_t)(n0 + wn * Cfg::WTN * 32)) * 4;
  const size_t row_bytes = (size_t)args.n_out * 4;

  v16i acc[2][Cfg::WTM][Cfg::WTN];
  float bias0[Cfg::WTN], bias1[Cfg::WTN];   // this lane's columns of the first and of the second tile
  float unquant;
  float omax = 0.0f;                        // AMAX: max |y| over what this lane has stored

  // value v (0..127) of the first tile, row by row across the two side-by-side accumulator tiles
  auto side_store = [&](int v) __attribute__((always_inline)) {
    const int b = v % Cfg::WTN, e = (v / Cfg::WTN) % 16, a = v / (Cfg::WTN * 16);
    const int r = 32 * a + 8 * (e / 4) + (e % 4);
    float y = (float)acc[0][a][b][e] * unquant;
    y = y + bias0[b];
    y = fmaxf(y, relu_floor);
    if(AMAX) omax = fmaxf(omax, fabsf(y));
    global_store_f32<NT>(out_base0 + (size_t)r * row_bytes + b * 128, out_voff, y);
  };

  // ---- one K block: 32 slots of one MFMA each (sub-step s/8, accumulator tile (s%8)/2, s%2).
  //   slots 0..11   request the fragments of sub-steps 2 and 3 of this block,
  //   after slot 15 the block's last fragment requests have returned (its stage is free) and block
  //                 g+1 must have landed: wait, barrier,
  //   slots 16..27  issue one global->LDS load each of block g+3 and request the fragments of
  //                 sub-steps 0 and 1 of block g+1,
  //   odd slots     (SIDE >= 0) dequantize and store one value of the first tile.
  // SET: accumulator set; FIRST: first block of a tile (accumulators start from zero);
  // SIDE: -1, or which of the last eight blocks of the stream this is.
  auto block = [&](int g, int stage, auto set_c, auto first_c, auto side_c) __attribute__((always_inline)) {
    constexpr int SET = decltype(set_c)::value;
    constexpr bool FIRST = decltype(first_c)::value;
    constexpr int SIDE = decltype(side_c)::value;
    constexpr bool ISSUE = SIDE < 0 || SIDE + NSTAGE < Cfg::kSideBlocks;   // block g+3 exists
    constexpr bool NEXT = SIDE < Cfg::kSideBlocks - 1;                     // block g+1 exists
    const int st_next = stage == NSTAGE - 1 ? 0 : stage + 1;
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for(int s = 0; s < 32; ++s) {
      if(s == 16) {
        wait_lgkmcnt0();
        if(NEXT) {
          if(SIDE < 0) wait_vmcnt<Cfg::kLoads>();
          else wait_vmcnt<pair_younger_ops(SIDE < 0 ? 0 : SIDE)>();
        }
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
      }
      if(s < 12) read_one(stage, 2 + s / 6, s % 6);
      if(s >= 16 && s < 28) {
        if(ISSUE) issue_one(g + NSTAGE, stage, s - 16);
        if(NEXT) read_one(st_next, (s - 16) / 6, (s - 16) % 6);
      }
      if(SIDE >= 0 && (s % 2) == 1) side_store((SIDE < 0 ? 0 : SIDE) * 16 + s / 2);
      const int kk = s / 8, a = (s % 8) / 2, b = s % 2;
      if(FIRST && kk == 0) {
        const v16i zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
        acc[SET][a][b] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[kk][a], bf[kk][b], zero, 0, 0, 0);
      } else {
        acc[SET][a][b] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[kk][a], bf[kk][b], acc[SET][a][b], 0, 0, 0);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  };

  // ---- prologue: three blocks in flight, wait for the first, request its first fragments ----
  // Every wave first stages the 256 bias values of the pair's columns in its own 1 KB of LDS (the
  // oldest load of the wave, so the first wait covers it; needs a 16-byte aligned bias).
  if(has_bias)
    global_load_lds16(args.bias + n0, (unsigned)lane * 16u, lds_base + Cfg::kRingBytes + wave * 1024);
  // The two quantization multipliers travel the same way (every lane fetches the same 4 bytes):
  // an ordinary load here would be waited for with a count that does not know the hand-issued loads.
  global_load_lds4(args.Aq + (size_t)args.M * (size_t)K, 0u, lds_base + Cfg::kRingBytes + Cfg::kWaves * 1024 + wave * 512);
  global_load_lds4(args.Bq + (size_t)K * (size_t)args.N, 0u, lds_base + Cfg::kRingBytes + Cfg::kWaves * 1024 + wave * 512 + 256);
#pragma unroll
  for(int s = 0; s < NSTAGE; ++s)
#pragma unroll
    for(int j = 0; j < Cfg::kLoads; ++j) issue_one(s, s, j);
  wait_vmcnt<(NSTAGE - 1) * Cfg::kLoads>();
  __builtin_amdgcn_s_barrier();
  const long long t_prologue = MH_CLOCK();
#pragma unroll
  for(int f = 0; f < 12; ++f) read_one(0, f / 6, f % 6);
  {
    const float* tails = reinterpret_cast<const float*>(lds + Cfg::kRingBytes + Cfg::kWaves * 1024 + wave * 512);
    unquant = unquant_mult(tails[0], tails[64], args.scale);
  }
  {
    const float* staged = reinterpret_cast<const float*>(lds + Cfg::kRingBytes + wave * 1024) + wn * Cfg::WTN * 32 + li;
#pragma unroll
    for(int b = 0; b < Cfg::WTN; ++b) {
      bias0[b] = has_bias ? staged[b * 32] : -0.0f;        // y + -0 = y
      bias1[b] = has_bias ? staged[BN + b * 32] : -0.0f;
    }
  }

  using I = std::integral_constant<int, 0>;
  std::integral_constant<int, 0> set0;
  std::integral_constant<int, 1> set1;
  std::integral_constant<int, -1> plain;
  int stage = 0;
  auto advance = [&]() __attribute__((always_inline)) { stage = stage == NSTAGE - 1 ? 0 : stage + 1; };
  int g = 0;
  block(g, stage, set0, std::true_type(), plain); advance();
  for(g = 1; g < KB; ++g) { block(g, stage, set0, std::false_type(), plain); advance(); }
  const int side_begin = total_blocks - Cfg::kSideBlocks;
  if(g < side_begin) {
    block(g, stage, set1, std::true_type(), plain); advance();
    for(++g; g < side_begin; ++g) { block(g, stage, set1, std::false_type(), plain); advance(); }
    block(g, stage, set1, std::false_type(), I()); advance();
  } else {
    block(g, stage, set1, std::true_type(), I()); advance();
  }
  const long long t_side = MH_CLOCK();
  block(g + 1, stage, set1, std::false_type(), std::integral_constant<int, 1>()); advance();
  block(g + 2, stage, set1, std::false_type(), std::integral_constant<int, 2>()); advance();
  block(g + 3, stage, set1, std::false_type(), std::integral_constant<int, 3>()); advance();
  block(g + 4, stage, set1, std::false_type(), std::integral_constant<int, 4>()); advance();
  block(g + 5, stage, set1, std::false_type(), std::integral_constant<int, 5>()); advance();
  block(g + 6, stage, set1, std::false_type(), std::integral_constant<int, 6>()); advance();
  block(g + 7, stage, set1, std::false_type(), std::integral_constant<int, 7>());
  const long long t_main = MH_CLOCK();

  // ---- the second tile's write-out: the same store form, four values in flight ----
  {
    const char* const out_base1 = out_base0 + BN * 4;
#pragma unroll
    for(int v = 0; v < Cfg::WTM * Cfg::WTN * 16; ++v) {
      const int b = v % Cfg::WTN, e = (v / Cfg::WTN) % 16, a = v / (Cfg::WTN * 16);
      const int r = 32 * a + 8 * (e / 4) + (e % 4);
      float y = (float)acc[1][a][b][e] * unquant;
      y = y + bias1[b];
      y = fmaxf(y, relu_floor);
      if(AMAX) omax = fmaxf(omax, fabsf(y));
      global_store_f32<NT>(out_base1 + (size_t)r * row_bytes + b * 128, out_voff, y);
    }
  }
  if(AMAX && args.absmax_out)
    publish_tile_absmax(omax, args.absmax_out, slot, args.absmax_used, reinterpret_cast<float*>(lds));
  if(MH_PROF(args) && tid == 0) {
    long long* p = MH_PROF(args) + (size_t)slot * 8;
    p[0] = t_start; p[1] = t_prologue; p[2] = t_main; p[3] = MH_CLOCK(); p[4] = t_main; p[5] = t_side; p[6] = w_start; p[7] = MH_WALL();
  }
}

template <bool NT, bool AMAX = false>
__global__ __launch_bounds__(PairCfg::kThreads) void gemm_pair_kernel(GemmArgs args, int pairs_n, int tiles_m) {
  extern __shared__ __attribute__((aligned(16))) int8_t lds[];
  int tn, tm;
  xcd_tile(pairs_n, tiles_m, blockIdx.x, tn, tm);   // a compact block of tile pairs per XCD
  gemm_pair_tiles<NT, AMAX>(args, tm * PairCfg::BM, tn * 2 * PairCfg::BN, lds, blockIdx.x);
}

// The same for an output that is not a whole number of tile pairs: pairs over the whole 256 x 256
// blocks, then 64 x 128 tiles over the rows below them and 128 x 64 tiles over the columns to their
// right (see RaggedPlan; main_tiles_n counts pairs).
template <bool NT, bool AMAX = false>
__global__ __launch_bounds__(PairCfg::kThreads) void gemm_pair_ragged_kernel(GemmArgs args, RaggedPlan plan) {
  extern __shared__ __attribute__((aligned(16))) int8_t lds[];
  const int slot = blockIdx.x;
  const int n_main = plan.main_tiles_n * plan.main_tiles_m;
  const int n_bottom = plan.bottom_tiles_n * plan.bottom_tiles_m;
  const int n_small = n_bottom + plan.right_tiles_n * plan.right_tiles_m;
  // number among the main tiles (0 .. n_main - 1) or n_main + number among the small tiles
  int block = slot;
  if(plan.lead) {
    if(slot >= plan.lead) {
      block = slot - plan.lead;
    } else if(slot < n_small) {
      block = n_main + slot;
    } else {   // an idle number between the small and the main tiles
      if(AMAX && args.absmax_out && threadIdx.x == 0) args.absmax_out[slot] = 0.0f;
      return;
    }
  }
  if(block < n_main) {
    int tn, tm;
    xcd_tile(plan.main_tiles_n, plan.main_tiles_m, block, tn, tm);
    gemm_pair_tiles<NT, AMAX>(args, tm * PairCfg::BM, tn * 2 * PairCfg::BN, lds, slot);
  } else if(block < n_main + n_bottom) {
    const int t = block - n_main;
    const int tn = t % plan.bottom_tiles_n, tm = t / plan.bottom_tiles_n;
    gemm_mfma32_tile<64, 128, 2, 2, 3, true, NT, false, AMAX>(args, plan.main_tiles_m * PairCfg::BM + tm * 64, tn * 128, lds, slot);
  } else {
    const int t = block - n_main - n_bottom;
    const int tm = t % plan.right_tiles_m, tn = t / plan.right_tiles_m;
    gemm_mfma32_tile<128, 64, 2, 2, 3, true, NT, false, AMAX>(args, tm * 128, plan.main_tiles_n * 2 * PairCfg::BN + tn * 64, lds, slot);
  }
}

}  // namespace marian_hip
