// Weight-streaming int8 GEMM for small M (decode shapes, M <= 128), optionally fused with the
// activation quantizer.
//
// The weights W^T [N x K] are read exactly once from HBM, straight into MFMA operand registers:
// lane l of a wave loads 16 consecutive K bytes of weight row n0 + l % 32, which is the row
// operand layout of v_mfma_i32_32x32x32_i8, so they need no LDS staging or transposition.  The
// small quantized activations are the column operand; a workgroup keeps them in LDS in operand
// order (within a fragment the 32 rows of a K chunk are XOR-permuted by a key of the chunk number,
// which spreads the quantizer's 4-byte writes over the LDS banks and keeps the fragment reads
// conflict free).  The 8 waves of a workgroup (4 for the smallest inputs: a wave then has its SIMD
// to itself and issues an instruction every 4 clocks instead of every 8) are arranged WN (different weight rows) x KW (different K
// ranges of the same rows); the KW partial sums are added through LDS (exact in any order).
//
// MODE kFusedAll: the workgroup reads the fp32 activations itself, takes their abs-max (every
// workgroup gets the same value: max is exact and order independent), quantizes them into LDS
// and so replaces a separate prepareA launch.  Workgroup 0 also writes the quantized activations
// and their quantMult to global memory, exactly what prepareA would have produced.
// MODE kFusedTiled: for activations too large for that.  A separate small kernel leaves per-
// workgroup abs-max values; this kernel reduces them, and quantizes its own 32 * MT32 rows chunk
// by chunk on the way into LDS (the workgroups of column 0 also write them out).
#pragma once

#include <type_traits>

#include "int8_common.h"
#include "quantize_kernels.h"

namespace marian_hip {

typedef int v16i_s __attribute__((ext_vector_type(16)));

constexpr int kFusedMaxElems = 32768;   // fp32 activations a workgroup holds in registers
constexpr int kPrequant = 0, kFusedAll = 1, kFusedTiled = 2;            // MODE

// The 32 rows of 16-byte chunk c16 of the activations are stored XOR-permuted by this key.  Any key
// leaves a fragment read (32 consecutive slots, permuted) free of bank conflicts; this one makes
// the quantizer's dword writes hit eight different slots (mod 8) for the eight quads that cover
// 32 consecutive chunks of one row, and for quads in neighbouring rows at the same chunk.
__device__ __forceinline__ int stream32_row_key(int c16) { return (c16 ^ (c16 >> 2)) & 7; }

// MT32: 32-row activation tiles per workgroup (blockIdx.y walks M in steps of 32 * MT32; the
// fused form needs all of M in one workgroup).  PW: 32-byte K sub-steps (weight loads in flight)
// per wave and chunk; a chunk is CS = PW * KW sub-steps, and its activations fill at most 64 KB
// of LDS.  The launcher picks the smallest PW that covers K in one chunk where there is one, so
// that no wave is left with sub-steps past the end of K.
template <int MT32, int WN, int KW, int PW_>
struct Stream32Cfg {
  static constexpr int kWaves = WN * KW;
  static constexpr int kThreads = kWaves * kWave;
  static_assert(kWaves == 8 || kWaves == 4, "eight waves, or four (one per SIMD) for the smallest inputs");
  static constexpr int kColsPerBlock = WN * 32;
  static constexpr int PW = PW_;
  static constexpr int CS = PW * KW;
  static constexpr int kStageBytes = MT32 * CS * kFragBytes;
  static constexpr int kReduceBytes = KW * WN * MT32 * 4 * kFragBytes;  // every wave's 32 * MT32 x 32 int32 tile
  static constexpr int kLdsBytes = kStageBytes > kReduceBytes ? kStageBytes : kReduceBytes;
  static_assert(PW >= 1 && PW <= 8 && kStageBytes <= 64 * 1024, "chunk size");
  static_assert(CS * MT32 * 64 % kThreads == 0, "stage must divide over the threads");
  static_assert(CS % 2 == 0, "a quad of lanes quantizes four 16-byte chunks of one row");
};

// Several weight matrices behind one activation tensor (kFusedTiled only): the grid's columns are
// the matrices' column blocks one after the other, and a workgroup takes weights, bias, output and
// width from the entry its block index falls into (block0[g] <= blockIdx.x < block0[g + 1]).
constexpr int kMaxGroups = 4;
struct GroupTable {
  const int8_t* Bq[kMaxGroups];
  const float* bias[kMaxGroups];
  void* out[kMaxGroups];
  int N[kMaxGroups];
  int block0[kMaxGroups + 1];
  int n;
};
struct NoGroups {};

// Dynamic LDS: one chunk (kStageBytes), for kFusedAll all of K (32 * MT32 * K bytes) if that is
// more; at least kReduceBytes.  partials: n_partials (1..2048) abs-max values (kFusedTiled only).
// NG (kFusedAll): 16-value groups per thread that are compiled in, 2 or 4; all but the last two are
// complete (the launcher picks NG = 2 for M * K <= 16384), so their loads, abs-max and
// quantization carry no range checks.
// ROWS: activation rows a workgroup multiplies, 32 * MT32 or (fused forms, MT32 = 1) 16: half the
// quantizing per workgroup and twice the workgroups, for calls that would otherwise leave most
// CUs idle.  With ROWS < M the kFusedAll form still takes the abs-max over all of A in every
// workgroup and quantizes only its own rows.
template <int MT32, int WN, int KW, int PW, int MODE, int NG = 4, int ROWS = 32 * MT32, typename GROUPS = NoGroups>
__global__ __launch_bounds__(WN * KW * kWave) void gemm_stream32_kernel(GemmArgs args,
                                                                        const float* A,
                                                                        int8_t* aq_out,
                                                                        const float* partials,
                                                                        int n_partials, GROUPS groups) {
  using Cfg = Stream32Cfg<MT32, WN, KW, PW>;
  constexpr bool GROUPED = std::is_same<GROUPS, GroupTable>::value;
  static_assert(!GROUPED || MODE == kFusedTiled, "several weight matrices: quantize-on-stage form only");
  int bx = blockIdx.x, gx = gridDim.x;   // column block within this workgroup's matrix, and how many it has
  if constexpr(GROUPED) {
    int g = 0;
#pragma unroll
    for(int i = 1; i < kMaxGroups; ++i)
      if(i < groups.n && bx >= groups.block0[i]) g = i;
    args.Bq = groups.Bq[g];
    args.bias = groups.bias[g];
    args.out = groups.out[g];
    args.N = args.n_out = groups.N[g];
    gx = groups.block0[g + 1] - groups.block0[g];
    bx -= groups.block0[g];
  }
  constexpr int kStream32Waves = Cfg::kWaves, kStream32Threads = Cfg::kThreads;
  constexpr bool TILED_ = MODE == kFusedTiled;
  constexpr int kFusedGroups = NG, kFullGroups = NG - 2;
  static_assert(NG == 2 || NG == 4, "groups per thread");
  static_assert(kFusedMaxElems == 4 * 16 * kWave * 8, "four groups per thread of eight waves hold the largest fused input");
  static_assert(!TILED_ || kAbsmaxSlots % Cfg::kThreads == 0, "the abs-max partials are split evenly over the threads");
  constexpr bool FUSED = MODE == kFusedAll;
  constexpr bool TILED = MODE == kFusedTiled;
  extern __shared__ __attribute__((aligned(16))) int8_t lds[];
  __shared__ float red[kStream32Waves];

  long long tp[6] = {0, 0, 0, 0, 0, 0}, wall0 = 0;
  if(MH_PROF(args)) {
    tp[0] = MH_CLOCK();
    wall0 = MH_WALL();
  }
  const int tid = threadIdx.x;
  const int wave = tid / kWave, lane = tid % kWave;
  const int wn = wave % WN, kw = wave / WN;
  const int li = lane % 32, lg = lane / 32;
  const int K = args.K, M = args.M;
  const int S = K / 32;                                   // K sub-steps
  const int n_chunks = (S + Cfg::CS - 1) / Cfg::CS;
  constexpr int R = ROWS;   // activation rows of this workgroup
  static_assert(R == MT32 * 32 || (R == 16 && MT32 == 1 && MODE != kPrequant && (FUSED || Cfg::CS % 16 == 0)),
                "half-height tiles");
  const int m_base = blockIdx.y * R;

  // Loads of a wave return in issue order and the compiler counts them: a value is waited for
  // with "all but the N youngest loads", and N can only count loads that are certain to have been
  // issued.  The order below follows from that: first the shortlist ids (one round trip, waited
  // for at once - they are addresses), then the activations, then the weights, last the bias
  // (needed last); the activation, weight and bias loads are unconditional (out-of-range indices
  // are clamped and the values replaced afterwards), so the activations are waited for with
  // exactly the weight and bias loads still in flight.

  // ---- weight row of this lane and where the bias of the four columns this lane will write
  //      sits (see the epilogue), both through the shortlist ids when there are any ----
  const int n0 = (bx * WN + wn) * 32;
  int wsrc = stream32_lane_column(n0, li, args.n_out);
  const int bias_n = min(n0 + 4 * (lane % 8), args.n_out - 4);   // n_out % 8 == 0: four valid columns
  uint32_t bias_at[4];
#pragma unroll
  for(int e = 0; e < 4; ++e) bias_at[e] = (uint32_t)(bias_n + e);
  if(args.idx) {
    if(args.bias) {
#pragma unroll
      for(int e = 0; e < 4; ++e) bias_at[e] = args.idx[bias_at[e]];
    }
    wsrc = (int)args.idx[wsrc];
  }
  // (pins the wait for the ids here, where nothing else is in flight; left to itself the compiler
  // computes the weight address, and waits, after the activation loads)
  asm volatile("" : "+v"(wsrc));
  const float bqm = tail_quant_mult(args.Bq, (size_t)K * (size_t)args.N);
  float aqm_pre = 0.0f;
  if(MODE == kPrequant) aqm_pre = tail_quant_mult(args.Aq, (size_t)M * (size_t)K);
  float amax = 0.0f;
  if(TILED) {   // a few (clamped) abs-max partials per thread cover all kAbsmaxSlots
    float pm[kAbsmaxSlots / kStream32Threads];
#pragma unroll
    for(int i = 0; i < kAbsmaxSlots / kStream32Threads; ++i)
      pm[i] = partials[min(tid + i * kStream32Threads, n_partials - 1)];
#pragma unroll
    for(int i = 0; i < kAbsmaxSlots / kStream32Threads; ++i) amax = fmaxf(amax, pm[i]);
  }
  // this lane's 16 bytes of K sub-step 0; a sub-step further is w_step bytes further for every column
  const int8_t* wrow = args.Bq + stream32_lane_offset(wsrc, lg);
  const size_t w_step = 32u * (size_t)args.N;
  __builtin_amdgcn_sched_barrier(0);

  // FUSED: the fp32 activations are requested before anything else - they are needed first, and
  // a wave's loads return in issue order, so behind the weight stream they would arrive last.
  // Four neighbouring lanes (a quad) own four consecutive groups of 16 values of one activation
  // row (K % 64 == 0 keeps them in one row); load e brings lane i of the quad the i-th four values
  // of group e, so a quad reads 64 contiguous bytes per load (one cache line per quad, the rate
  // the address unit works at) and, after quantization, holds dword i of four 16-byte LDS slots.
  // Quad number qi = j * threads / 4 + tid / 4 covers groups 4 * qi .. 4 * qi + 3; group g is row
  // g / (K/16), 16-byte chunk g % (K/16).
  v4f vals[FUSED ? kFusedGroups : 1][4];
  const int n16 = M * K / 16;   // groups; a multiple of four
  const int quad = tid / 4, qlane = tid % 4;
  const int wave_s = __builtin_amdgcn_readfirstlane(wave);   // (a scalar for the compiler)
  // does group set j reach into this thread's / this wave's range?  (complete sets: always)
  auto in_range = [&](int j) { return j < kFullGroups || 4 * (j * (kStream32Threads / 4) + quad) < n16; };
  if(FUSED) {
    // a quad's four groups are 256 consecutive bytes; group set j starts 32 KB after set j - 1
    const char* a_quad = reinterpret_cast<const char*>(A) + quad * 256 + qlane * 16;
#pragma unroll
    for(int j = 0; j < kFusedGroups; ++j) {
      if(j < kFullGroups) {
#pragma unroll
        for(int e = 0; e < 4; ++e)
          vals[j][e] = *reinterpret_cast<const v4f*>(a_quad + j * (kStream32Threads * 64) + e * 64);
      } else {
        // (a wave whose 64 groups are all out of range skips the loads; a thread past the end
        // reads a copy of the last groups, which is never looked at)
        const int g0 = min(4 * (j * (kStream32Threads / 4) + quad), n16 - 4);
        const char* a_part = reinterpret_cast<const char*>(A) + (size_t)g0 * 64 + qlane * 16;
#pragma unroll
        for(int e = 0; e < 4; ++e) {
          // (any value: never looked at.  Not zero - the compiler would share the register of an
          // existing zero constant with one component and then has to copy the loaded value into
          // it, waiting for the load right after issuing it)
          vals[j][e] = v4f{1.0f, 1.0f, 1.0f, 1.0f};
          if(j * kStream32Threads + wave_s * kWave < n16)
            vals[j][e] = *reinterpret_cast<const v4f*>(a_part + e * 64);
        }
      }
    }
  }

  // Where the quad's first group lies (two integer divisions: worked out here, while the loads
  // are in flight, not behind the abs-max where the quantization waits for them).
  const unsigned k16n = K / 16;   // 16-byte chunks per activation row (a multiple of four)
  unsigned row = 0, c16 = 0, drow = 0, dc16 = 0;
  if(FUSED) {
    row = 4 * quad / k16n;
    c16 = 4 * quad % k16n;
    drow = kStream32Threads / k16n;
    dc16 = kStream32Threads % k16n;
    asm volatile("" : "+v"(row), "+v"(c16));
  }

  float aqm = 0.0f;        // quantMult of the activations (fused modes)
  bool finite_t = false;   // kFusedTiled: the quantMult is finite
  // The multiplier of the epilogue (a division through double precision) is worked out as soon as
  // the quantMult of the activations is known, under the matrix instructions.
  float unquant = 0.0f;
  if(MODE == kPrequant) unquant = unquant_mult(aqm_pre, bqm, args.scale);
  // Otherwise a chunk of activations is fetched into registers (all loads in flight at once) and
  // then dropped into LDS, so the fetch of chunk c+1 overlaps the multiplication of chunk c.
  // Pre-quantized: thread slot (sub-step, m-tile, lane) in operand order.  kFusedTiled: fp32
  // source; group = row * 2 * CS + 16-byte chunk, a quad of lanes takes four consecutive groups
  // (a wave reads whole rows), quantizes them and finds the operand slots from there.
  constexpr int kStageVecs = Cfg::CS * R * 2 / kStream32Threads;
  v4i stage[TILED ? 1 : kStageVecs];
  v4f stagef[TILED ? kStageVecs : 1][4];
  auto stage_fetch = [&](int chunk) __attribute__((always_inline)) {
    const int s0 = chunk * Cfg::CS;
#pragma unroll
    for(int j = 0; j < kStageVecs; ++j) {
      const int slot = j * kStream32Threads + tid;
      if(TILED) {
        // quad slot / 4 takes chunks c16 .. c16 + 3 of row r, lane i of the quad the i-th four
        // values of each (64 contiguous bytes per quad and load, as in the fused form)
        const int g = (slot / 4) * 4, r = g / (2 * Cfg::CS), c16 = g % (2 * Cfg::CS);
        const int m = min(m_base + r, M - 1);
#pragma unroll
        for(int e = 0; e < 4; ++e) {
          const int s = min(s0 + (c16 + e) / 2, S - 1);
          stagef[j][e] = *reinterpret_cast<const v4f*>(A + (size_t)m * (size_t)K + s * 32 + (e % 2) * 16 + (slot % 4) * 4);
        }
      } else {
        const int l = slot % 64, f = slot / 64;
        const int mt = f % MT32, step = f / MT32;
        const int m = m_base + mt * 32 + (l % 32);
        const int s = s0 + step;
        stage[j] = load16(args.Aq + (size_t)min(m, M - 1) * (size_t)K + min(s, S - 1) * 32 + (l / 32) * 16);
      }
    }
  };
  auto stage_store = [&](int chunk) __attribute__((always_inline)) {
#pragma unroll
    for(int j = 0; j < kStageVecs; ++j) {
      const int slot = j * kStream32Threads + tid;
      if(TILED) {
        const int g = (slot / 4) * 4, r = g / (2 * Cfg::CS), c16 = g % (2 * Cfg::CS);
        const int m = m_base + r;
        uint32_t q[4];
        if(finite_t) {
#pragma unroll
          for(int e = 0; e < 4; ++e) q[e] = quantize_pack4_finite(stagef[j][e], aqm);
        } else {
#pragma unroll
          for(int e = 0; e < 4; ++e) q[e] = quantize_pack4(stagef[j][e], aqm);
        }
        const int slot0 = ((c16 / 2) * MT32 + r / 32) * 64, x = (r % 32) ^ stream32_row_key(c16);
#pragma unroll
        for(int e = 0; e < 4; ++e) {
          const int s = chunk * Cfg::CS + (c16 + e) / 2;
          const int sw = slot0 + (e / 2) * MT32 * 64 + (e % 2) * 32 + (x ^ e);
          *reinterpret_cast<uint32_t*>(lds + sw * 16 + (slot % 4) * 4) = q[e];
          if(aq_out && blockIdx.x == 0 && m < M && s < S)
            *reinterpret_cast<uint32_t*>(aq_out + (size_t)m * (size_t)K + s * 32 + (e % 2) * 16 + (slot % 4) * 4) = q[e];
        }
      } else {
        const int l = slot % 64, f = slot / 64;
        const int step = f / MT32;
        const int sw = (slot & ~31) | ((l % 32) ^ stream32_row_key(2 * step + l / 32));
        *reinterpret_cast<v4i*>(lds + sw * 16) = stage[j];   // (rows past M: a copy of row M - 1, never stored)
      }
    }
  };
  if(!FUSED) stage_fetch(0);   // ahead of the weights, like the fp32 activations above

  v4i w[Cfg::PW];
  const int kw_s = __builtin_amdgcn_readfirstlane(kw);   // (a scalar for the compiler)
  const int step0 = kw * Cfg::PW;                        // this wave's first sub-step within a chunk
  // weights of a chunk: PW sub-steps of the lane's column (a wave reads 1 KB of consecutive memory
  // per sub-step), one pointer and uniform offsets when the wave's sub-steps all lie within K,
  // clamped one by one otherwise
  auto load_weights = [&](int chunk, v4i (&dst)[Cfg::PW]) __attribute__((always_inline)) {
    if(stream32_chunk_is_whole(chunk, Cfg::CS, kw_s, Cfg::PW, S)) {
      const int8_t* wp = wrow + (size_t)(chunk * Cfg::CS + step0) * w_step;
#pragma unroll
      for(int p = 0; p < Cfg::PW; ++p) dst[p] = load16(wp + (size_t)p * w_step);
    } else {
#pragma unroll
      for(int p = 0; p < Cfg::PW; ++p) {
        const int s = chunk * Cfg::CS + step0 + p;
        dst[p] = load16(wrow + (size_t)stream32_clamped_substep(s, S) * w_step);
      }
    }
  };
  // sub-steps past the end of K multiply zero weights
  auto mask_weights = [&](int chunk) __attribute__((always_inline)) {
#pragma unroll
    for(int p = 0; p < Cfg::PW; ++p)
      if(chunk * Cfg::CS + kw * Cfg::PW + p >= S) w[p] = v4i{0, 0, 0, 0};
  };
  __builtin_amdgcn_sched_barrier(0);
  load_weights(0, w);   // in flight while the activations are prepared
  __builtin_amdgcn_sched_barrier(0);
  // (unconditional as well: without a bias the weights stand in - 4 * N readable bytes - and the
  // values are dropped in the epilogue)
  float bias_s[4];
  const float* bias_src = args.bias ? args.bias : reinterpret_cast<const float*>(args.Bq);
#pragma unroll
  for(int e = 0; e < 4; ++e) bias_s[e] = bias_src[bias_at[e]];
  __builtin_amdgcn_sched_barrier(0);

  // ---- activations into LDS, operand order: slot (sub-step, m-tile, lane) of 16 bytes holds
  //      Aq[mt*32 + lane%32][(s0+step)*32 + (lane/32)*16 .. +15]
  if(TILED) {
    amax = block_max(amax, red);
    aqm = quant_mult_from_maxabs(amax);
    unquant = unquant_mult(aqm, bqm, args.scale);
    finite_t = aqm < __builtin_inff();   // (see the fused form below)
    if(MH_PROF(args)) tp[1] = MH_CLOCK();
    if(aq_out && blockIdx.x == 0 && blockIdx.y == 0 && tid == 0)
      *reinterpret_cast<float*>(aq_out + (size_t)M * K) = aqm;
  }
  if(FUSED) {
    // whole A (M*K <= kFusedMaxElems floats) in registers: abs-max, then quantize into LDS
#pragma unroll
    for(int j = 0; j < kFusedGroups; ++j) {
      if(in_range(j)) {
#pragma unroll
        for(int e = 0; e < 4; ++e) amax = abs4max(vals[j][e], amax);
      }
    }
    // (activation rows between M and the end of the last 32-row tile stay whatever LDS holds: a
    // row only feeds its own output row, integer products cannot trap, and rows past M are never
    // stored)
    amax = block_max(amax, red);
    if(MH_PROF(args)) tp[1] = MH_CLOCK();
    aqm = quant_mult_from_maxabs(amax);
    unquant = unquant_mult(aqm, bqm, args.scale);
    // With a finite quantMult no product can leave [-127.0001, 127.0001]: finite values are at
    // most the abs-max in magnitude, and an infinite value makes the quantMult 0 and its product
    // NaN.  (An abs-max of zero, or one below 127 / FLT_MAX, gives an infinite quantMult, and then
    // infinite products, which the conversion of the CPU path turns into -127, not +127.)
    const bool finite = aqm < __builtin_inff();
    uint32_t q[kFusedGroups][4];
#pragma unroll
    for(int j = 0; j < kFusedGroups; ++j) {
      const unsigned rr = row - m_base;   // row within this workgroup's tile
      if(in_range(j) && rr < (unsigned)R) {
        if(finite) {
#pragma unroll
          for(int e = 0; e < 4; ++e) q[j][e] = quantize_pack4_finite(vals[j][e], aqm);
        } else {
#pragma unroll
          for(int e = 0; e < 4; ++e) q[j][e] = quantize_pack4(vals[j][e], aqm);
        }
        // slot of group e: chunk c16 + e, i.e. sub-step (c16 + e) / 2, half (c16 + e) % 2, and
        // the row permuted by the key of chunk c16 + e, which is the key of c16 (c16 % 4 == 0) ^ e
        const unsigned slot0 = ((c16 >> 1) * MT32 + (rr >> 5)) * 64, x = (rr & 31) ^ stream32_row_key(c16);
#pragma unroll
        for(int e = 0; e < 4; ++e) {
          const unsigned slot = slot0 + (e / 2) * MT32 * 64 + (e % 2) * 32 + (x ^ e);
          *reinterpret_cast<uint32_t*>(lds + slot * 16 + qlane * 4) = q[j][e];
        }
      }
      row += drow;
      c16 += dc16;
      if(c16 >= k16n) {
        c16 -= k16n;
        row += 1;
      }
    }
    if(aq_out && blockIdx.x == 0) {   // the quad's four groups are 64 consecutive bytes of Aq
#pragma unroll
      for(int j = 0; j < kFusedGroups; ++j) {
        const int g = 4 * (j * (kStream32Threads / 4) + quad);
        if(in_range(j) && (unsigned)(g / (int)k16n - m_base) < (unsigned)R) {
#pragma unroll
          for(int e = 0; e < 4; ++e)
            *reinterpret_cast<uint32_t*>(aq_out + (size_t)(g + e) * 16 + qlane * 4) = q[j][e];
        }
      }
    }
    if(aq_out && blockIdx.x == 0 && blockIdx.y == 0 && tid == 0)
      *reinterpret_cast<float*>(aq_out + (size_t)M * K) = aqm;
    __syncthreads();
  }
  if(!FUSED) {
    stage_store(0);
    __syncthreads();
  }

  if(MH_PROF(args)) tp[2] = MH_CLOCK();
  // The first chunk is peeled off the loop: its first product starts from a literal zero and its
  // fragment addresses are this wave's base plus constants (slot of sub-step step0 + p, half lg,
  // row li: the row key of chunk number 2 * (step0 + p) + lg is key(2 * step0) ^ key(2 * p) ^ lg,
  // the three parts occupy different bits).  In the fused form LDS holds every sub-step of K, so
  // later chunks address it by the global sub-step, clamped (sub-steps past the end of K multiply
  // zero weights; for the first chunk the allocation covers a whole chunk).
  v16i_s acc[MT32];
  v4i wnext[Cfg::PW];
  const int8_t* frag0 = lds + step0 * MT32 * kFragBytes + lg * 512;
  const int akey = li ^ lg ^ stream32_row_key(2 * step0);
  auto multiply_chunk = [&](int c, auto first_tag) __attribute__((always_inline)) {
    constexpr bool kFirst = decltype(first_tag)::value;
    const bool more = c + 1 < n_chunks;
    if(more) {
      if(!FUSED) stage_fetch(c + 1);
      load_weights(c + 1, wnext);
    }
    if((c + 1) * Cfg::CS > S) mask_weights(c);
#pragma unroll
    for(int p = 0; p < Cfg::PW; ++p) {
#pragma unroll
      for(int mt = 0; mt < MT32; ++mt) {
        v4i a;
        if(FUSED && !kFirst) {
          const int step = min(c * Cfg::CS + step0 + p, S - 1);
          a = *reinterpret_cast<const v4i*>(
              lds + (step * MT32 + mt) * kFragBytes + (lg * 32 + (li ^ stream32_row_key(2 * step + lg))) * 16);
        } else {
          a = *reinterpret_cast<const v4i*>(frag0 + (p * MT32 + mt) * kFragBytes +
                                            (akey ^ stream32_row_key(2 * p)) * 16);
        }
        if(kFirst && p == 0) {
          const v16i_s zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
          acc[mt] = __builtin_amdgcn_mfma_i32_32x32x32_i8(w[p], a, zero, 0, 0, 0);
        } else {
          acc[mt] = __builtin_amdgcn_mfma_i32_32x32x32_i8(w[p], a, acc[mt], 0, 0, 0);
        }
      }
    }
    if(more) {
      if(!FUSED) {
        __syncthreads();   // everyone is done reading chunk c
        stage_store(c + 1);
        __syncthreads();
      }
#pragma unroll
      for(int p = 0; p < Cfg::PW; ++p) w[p] = wnext[p];
    }
  };
  multiply_chunk(0, std::true_type());
  for(int c = 1; c < n_chunks; ++c) multiply_chunk(c, std::false_type());

  if(MH_PROF(args)) tp[3] = MH_CLOCK();
  // ---- every wave drops its 32 * MT32 x 32 tile of int32 partial sums into LDS as a row-major
  //      matrix [activation row][32 weight rows] (128 bytes per row; the eight 16-byte pieces of
  //      a row XOR-permuted by the row number, which keeps both sides free of bank conflicts),
  //      and finishes 1/KW of the rows of its column group: it adds the KW partial tiles (exact in
  //      any order) and stores whole 128-byte output rows, eight lanes per row.  Accumulator
  //      value v of tile mt in lane (li, lg) is activation row mt * 32 + li, weight row
  //      8 * (v / 4) + 4 * lg + v % 4, i.e. piece 2 * (v / 4) + lg of that row. ----
  constexpr int kTileBytes = R * 128;
  __syncthreads();   // every wave is done reading activations from LDS
  {
    int8_t* mine = lds + (size_t)(wn * KW + kw) * kTileBytes;
#pragma unroll
    for(int mt = 0; mt < MT32; ++mt)
#pragma unroll
      for(int q = 0; q < 4; ++q) {
        const int m = mt * 32 + li, piece = (2 * q + lg) ^ (li & 7);
        if(R < 32 && li >= R) continue;
        *reinterpret_cast<v4i*>(mine + m * 128 + piece * 16) =
            v4i{acc[mt][4 * q], acc[mt][4 * q + 1], acc[mt][4 * q + 2], acc[mt][4 * q + 3]};
      }
  }
  __syncthreads();

  if(MH_PROF(args)) tp[4] = MH_CLOCK();
  float omax = 0.0f;   // max |y| over what this wave stores
  {
    constexpr int kPieces = R * 8 / KW;        // 16-byte pieces this wave finishes (32 .. 1024)
    const bool has_bias = args.bias != nullptr;
    const int n = n0 + 4 * (lane % 8);
    const int8_t* tiles = lds + (size_t)(wn * KW) * kTileBytes;
    // Use the bias values once ahead of the stores, so that the compiler waits for their loads here
    // (they arrived long ago).  Otherwise it waits inside the loop, behind the branches, for all
    // vector memory operations before each use - and every store then waits for the one before.
#pragma unroll
    for(int e = 0; e < 4; ++e) asm volatile("" ::"v"(bias_s[e]));
#pragma unroll
    for(int it = 0; it < (kPieces + 63) / 64; ++it) {
      const int pc = it * 64 + lane;
      const int mrow = kw * (R / KW) + pc / 8;              // row within the workgroup's tile
      if(kPieces % 64 != 0 && pc >= kPieces) continue;
      const int8_t* src = tiles + mrow * 128 + (((lane % 8) ^ (mrow & 7)) * 16);
      v4i sum = *reinterpret_cast<const v4i*>(src);
#pragma unroll
      for(int t = 1; t < KW; ++t) sum += *reinterpret_cast<const v4i*>(src + t * kTileBytes);
      const int m = m_base + mrow;
      if(m >= M || n >= args.n_out) continue;
      const size_t off = (size_t)m * (size_t)args.n_out + (size_t)n;
      if(args.dump) {
        *reinterpret_cast<v4i*>(reinterpret_cast<int32_t*>(args.out) + off) = sum;
        continue;
      }
      // y = float(acc) * unquant (+ bias); relu: y > 0 ? y : 0; mul and add round separately
      float y[4];
#pragma unroll
      for(int e = 0; e < 4; ++e) {
        y[e] = (float)sum[e] * unquant;
        if(has_bias) y[e] = y[e] + bias_s[e];
        if(args.relu) y[e] = y[e] > 0.0f ? y[e] : 0.0f;
        omax = fmaxf(omax, fabsf(y[e]));
      }
      v4f* dst = reinterpret_cast<v4f*>(reinterpret_cast<float*>(args.out) + off);
      const v4f yv = v4f{y[0], y[1], y[2], y[3]};
      // (written out: behind a branch the compiler merges a non-temporal builtin store and a plain
      // one into one plain store)
      if(args.stream_out) asm volatile("global_store_dwordx4 %0, %1, off nt" : : "v"(dst), "v"(yv) : "memory");
      else *dst = yv;
    }
  }
  if(args.absmax_out && !args.dump) {
    // slot (workgroup, wave) takes this wave's maximum; workgroup 0 zeroes the slots nobody owns
    // (the launcher made sure that 8 slots per workgroup fit)
    const int block = blockIdx.y * gx + bx, used = gx * gridDim.y * kStream32Waves;
    omax = wave_max(omax);
    if(lane == 0) args.absmax_out[block * kStream32Waves + wave] = omax;
    if(block == 0)
      for(int sl = used + tid; sl < kAbsmaxSlots; sl += kStream32Threads) args.absmax_out[sl] = 0.0f;
  }
  if(MH_PROF(args) && tid == 0) {
    long long* p = MH_PROF(args) + ((size_t)blockIdx.y * gridDim.x + blockIdx.x) * 8;
    p[0] = tp[0]; p[1] = tp[1]; p[2] = tp[2]; p[3] = tp[3]; p[4] = tp[4]; p[5] = MH_CLOCK();
    p[6] = MH_WALL();
    p[7] = wall0;
  }
}

}  // namespace marian_hip
