// Weight-streaming int8 GEMM for small M (decode shapes, M <= 128), optionally fused with the
// activation quantizer.
//
// The weights W^T [N x K] are read exactly once from HBM, straight into MFMA operand registers:
// lane l of a wave loads 16 consecutive K bytes of weight row n0 + l % 32, which is the row
// operand layout of v_mfma_i32_32x32x32_i8, so they need no LDS staging or transposition.  The
// small quantized activations are the column operand; a workgroup keeps them in LDS in operand
// order (within a fragment the 32 rows of a K chunk are XOR-permuted by the chunk number, which
// spreads the quantizer's 4-byte writes over the LDS banks and keeps the fragment reads
// conflict free).  The 8 waves of a workgroup are arranged WN (different weight rows) x KW (different K
// ranges of the same rows); the KW partial sums are added through LDS (exact in any order).
//
// FUSED: the workgroup reads the fp32 activations itself, takes their abs-max (every workgroup
// gets the same value: max is exact and order independent), quantizes them into LDS and so
// replaces a separate prepareA launch.  Workgroup 0 also writes the quantized activations and
// their quantMult to global memory, exactly what prepareA would have produced.
#pragma once

#include "int8_common.h"
#include "quantize_kernels.h"

namespace marian_hip {

typedef int v16i_s __attribute__((ext_vector_type(16)));

constexpr int kStream32Waves = 8;
constexpr int kStream32Threads = kStream32Waves * kWave;
constexpr int kFusedMaxElems = 32768;   // fp32 activations a workgroup holds in registers
constexpr int kFusedGroups = kFusedMaxElems / 16 / kStream32Threads;   // 16-value groups per thread

// MT32: 32-row activation tiles per workgroup (blockIdx.y walks M in steps of 32 * MT32; the
// fused form needs all of M in one workgroup).  CS: 32-byte K sub-steps staged per chunk.
template <int MT32, int WN, int KW>
struct Stream32Cfg {
  static_assert(WN * KW == kStream32Waves, "eight waves");
  static constexpr int kColsPerBlock = WN * 32;
  // K sub-steps per chunk: activations of a chunk fill at most 64 KB of LDS, and each wave owns
  // at most 8 sub-steps (8 weight loads in flight) of a chunk
  static constexpr int kMaxChunkSteps = (64 * 1024) / (MT32 * kFragBytes) < 8 * KW
                                            ? (64 * 1024) / (MT32 * kFragBytes)
                                            : 8 * KW;
  static constexpr int PW = kMaxChunkSteps / KW;      // sub-steps per wave per chunk
  static constexpr int CS = PW * KW;
  static constexpr int kStageBytes = MT32 * CS * kFragBytes;
  static constexpr int kReduceBytes = (KW - 1) * WN * MT32 * 4 * kFragBytes;  // v16i per lane
  static constexpr int kLdsBytes = kStageBytes > kReduceBytes ? kStageBytes : kReduceBytes;
  static_assert(PW >= 1, "chunk too small");
};

// Dynamic LDS: FUSED holds all of K (32 * MT32 * K bytes); otherwise one chunk (kStageBytes);
// both at least kReduceBytes.
template <int MT32, int WN, int KW, bool FUSED>
__global__ __launch_bounds__(kStream32Threads) void gemm_stream32_kernel(GemmArgs args,
                                                                        const float* A,
                                                                        int8_t* aq_out) {
  using Cfg = Stream32Cfg<MT32, WN, KW>;
  extern __shared__ __attribute__((aligned(16))) int8_t lds[];
  __shared__ float red[kStream32Waves];

  long long tp[6] = {0, 0, 0, 0, 0, 0};
  if(args.prof) tp[0] = clock64();
  const int tid = threadIdx.x;
  const int wave = tid / kWave, lane = tid % kWave;
  const int wn = wave % WN, kw = wave / WN;
  const int li = lane % 32, lg = lane / 32;
  const int K = args.K, M = args.M;
  const int S = K / 32;                                   // K sub-steps
  const int n_chunks = (S + Cfg::CS - 1) / Cfg::CS;
  const int m_base = blockIdx.y * (MT32 * 32);            // activation rows of this workgroup

  // ---- weight row of this lane ----
  const int n0 = (blockIdx.x * WN + wn) * 32;
  int wsrc = 0;
  {
    const int n = n0 + li;
    if(n < args.n_out) wsrc = args.idx ? (int)args.idx[n] : n;
  }
  const int8_t* wrow = args.Bq + (size_t)wsrc * (size_t)K + lg * 16;

  // FUSED: the fp32 activations are requested before anything else - they are needed first, and
  // a wave's loads return in issue order, so behind the weight stream they would arrive last.
  // A thread owns groups of 16 consecutive values of one activation row (one 16-byte LDS slot
  // after quantization): group number gi = j * threads + tid is row gi / (K/16), chunk gi % (K/16).
  v4f vals[FUSED ? kFusedGroups : 1][4];
  float amax = 0.0f;
  const int n16 = M * K / 16;
  if(FUSED) {
    const v4f* a4 = reinterpret_cast<const v4f*>(A);
#pragma unroll
    for(int j = 0; j < kFusedGroups; ++j) {
      const int gi = j * kStream32Threads + tid;
#pragma unroll
      for(int e = 0; e < 4; ++e) {
        v4f v = {0.0f, 0.0f, 0.0f, 0.0f};
        if(gi < n16) v = a4[gi * 4 + e];
        vals[j][e] = v;
      }
    }
  }

  v4i w[Cfg::PW];
  auto load_weights = [&](int chunk) {
#pragma unroll
    for(int p = 0; p < Cfg::PW; ++p) {
      const int s = chunk * Cfg::CS + kw * Cfg::PW + p;
      v4i v = {0, 0, 0, 0};
      if(s < S) v = load16(wrow + s * 32);
      w[p] = v;
    }
  };
  load_weights(0);   // in flight while the activations are prepared

  // Everything else the epilogue needs from global memory is requested now as well, so that all
  // global latencies of this workgroup overlap: the weight quantMult, the bias of the lane's
  // columns n0 + 8q + 4*lg .. +3 (q = 0..3), through the shortlist ids when there are any.
  float bqm = 0.0f, aqm_pre = 0.0f;
  v4f bias_v[4];
#pragma unroll
  for(int q = 0; q < 4; ++q) bias_v[q] = v4f{0.0f, 0.0f, 0.0f, 0.0f};
  if(!args.dump) {
    bqm = tail_quant_mult(args.Bq, (size_t)K * (size_t)args.N);
    if(!FUSED) aqm_pre = tail_quant_mult(args.Aq, (size_t)M * (size_t)K);
    if(args.bias && kw == 0) {
#pragma unroll
      for(int q = 0; q < 4; ++q) {
        const int n = n0 + 8 * q + 4 * lg;
        if(n < args.n_out) {
          if(args.idx) {
            bias_v[q] = v4f{args.bias[args.idx[n]], args.bias[args.idx[n + 1]],
                            args.bias[args.idx[n + 2]], args.bias[args.idx[n + 3]]};
          } else {
            bias_v[q] = v4f{args.bias[n], args.bias[n + 1], args.bias[n + 2], args.bias[n + 3]};
          }
        }
      }
    }
  }

  // ---- activations into LDS, operand order: slot (sub-step, m-tile, lane) of 16 bytes holds
  //      Aq[mt*32 + lane%32][(s0+step)*32 + (lane/32)*16 .. +15]
  float aqm = 0.0f;
  if(FUSED) {
    // whole A (M*K <= kFusedMaxElems floats) in registers: abs-max, then quantize into LDS
#pragma unroll
    for(int j = 0; j < kFusedGroups; ++j)
#pragma unroll
      for(int e = 0; e < 4; ++e) amax = abs4max(vals[j][e], amax);
    // zero the rows between M and the next multiple of 32 (whole LDS stage, cheap)
    for(int i = tid; i < S * MT32 * 64; i += kStream32Threads)
      reinterpret_cast<v4i*>(lds)[i] = v4i{0, 0, 0, 0};
    amax = block_max(amax, red);   // its barriers also order the zero fill before the writes
    if(args.prof) tp[1] = clock64();
    aqm = quant_mult_from_maxabs(amax);
    // with a finite non-zero abs-max no product can leave [-127.0001, 127.0001]
    const bool finite = amax > 0.0f && amax < __builtin_inff();
    const int k16n = K / 16;   // 16-byte chunks per activation row
    int row = tid / k16n, c16 = tid % k16n;
    const int drow = kStream32Threads / k16n, dc16 = kStream32Threads % k16n;
#pragma unroll
    for(int j = 0; j < kFusedGroups; ++j) {
      const int gi = j * kStream32Threads + tid;
      if(gi < n16) {
        uint4 q;
        if(finite) {
          q.x = quantize_pack4_finite(vals[j][0], aqm);
          q.y = quantize_pack4_finite(vals[j][1], aqm);
          q.z = quantize_pack4_finite(vals[j][2], aqm);
          q.w = quantize_pack4_finite(vals[j][3], aqm);
        } else {
          q.x = quantize_pack4(vals[j][0], aqm);
          q.y = quantize_pack4(vals[j][1], aqm);
          q.z = quantize_pack4(vals[j][2], aqm);
          q.w = quantize_pack4(vals[j][3], aqm);
        }
        const int s = c16 / 2, g = c16 % 2;
        const int slot = (s * MT32 + row / 32) * 64 + g * 32 + ((row % 32) ^ (c16 & 7));
        *reinterpret_cast<uint4*>(lds + slot * 16) = q;
        if(aq_out && blockIdx.x == 0) *reinterpret_cast<uint4*>(aq_out + (size_t)row * K + c16 * 16) = q;
      }
      row += drow;
      c16 += dc16;
      if(c16 >= k16n) {
        c16 -= k16n;
        row += 1;
      }
    }
    if(aq_out && blockIdx.x == 0 && tid == 0)
      *reinterpret_cast<float*>(aq_out + (size_t)M * K) = aqm;
    __syncthreads();
  }
  // Pre-quantized activations: a chunk is fetched into registers (all loads in flight at once)
  // and then dropped into LDS, so the fetch of chunk c+1 overlaps the multiplication of chunk c.
  constexpr int kStageVecs = Cfg::CS * MT32 * 64 / kStream32Threads;
  v4i stage[kStageVecs];
  auto stage_fetch = [&](int chunk) {
    const int s0 = chunk * Cfg::CS;
#pragma unroll
    for(int j = 0; j < kStageVecs; ++j) {
      const int slot = j * kStream32Threads + tid;
      const int l = slot % 64, f = slot / 64;
      const int mt = f % MT32, step = f / MT32;
      const int m = m_base + mt * 32 + (l % 32);
      const int s = s0 + step;
      v4i v = {0, 0, 0, 0};
      if(m < M && s < S) v = load16(args.Aq + (size_t)m * (size_t)K + s * 32 + (l / 32) * 16);
      stage[j] = v;
    }
  };
  auto stage_store = [&]() {
#pragma unroll
    for(int j = 0; j < kStageVecs; ++j) {
      const int slot = j * kStream32Threads + tid;
      const int l = slot % 64, step = (slot / 64) / MT32;
      const int sw = (slot & ~31) | ((l % 32) ^ ((2 * step + l / 32) & 7));
      *reinterpret_cast<v4i*>(lds + sw * 16) = stage[j];
    }
  };
  if(!FUSED) {
    stage_fetch(0);
    stage_store();
    __syncthreads();
  }

  if(args.prof) tp[2] = clock64();
  v16i_s acc[MT32];
#pragma unroll
  for(int mt = 0; mt < MT32; ++mt)
#pragma unroll
    for(int v = 0; v < 16; ++v) acc[mt][v] = 0;

  v4i wnext[Cfg::PW];
  for(int c = 0; c < n_chunks; ++c) {
    const bool more = c + 1 < n_chunks;
    if(more) {
      if(!FUSED) stage_fetch(c + 1);
#pragma unroll
      for(int p = 0; p < Cfg::PW; ++p) {
        const int s = (c + 1) * Cfg::CS + kw * Cfg::PW + p;
        v4i v = {0, 0, 0, 0};
        if(s < S) v = load16(wrow + s * 32);
        wnext[p] = v;
      }
    }
#pragma unroll
    for(int p = 0; p < Cfg::PW; ++p) {
      // FUSED keeps every sub-step in LDS; otherwise LDS holds the current chunk only.  Sub-steps
      // past the end of K multiply zero weights; their LDS slot is clamped to a valid one.
      int step = kw * Cfg::PW + p;
      if(FUSED) step = min(c * Cfg::CS + step, S - 1);
#pragma unroll
      for(int mt = 0; mt < MT32; ++mt) {
        const v4i a = *reinterpret_cast<const v4i*>(
            lds + (step * MT32 + mt) * kFragBytes + (lg * 32 + (li ^ ((2 * step + lg) & 7))) * 16);
        acc[mt] = __builtin_amdgcn_mfma_i32_32x32x32_i8(w[p], a, acc[mt], 0, 0, 0);
      }
    }
    if(more) {
      if(!FUSED) {
        __syncthreads();   // everyone is done reading chunk c
        stage_store();
        __syncthreads();
      }
#pragma unroll
      for(int p = 0; p < Cfg::PW; ++p) w[p] = wnext[p];
    }
  }

  if(args.prof) tp[3] = clock64();
  // ---- add the KW partial sums into the kw == 0 waves ----
  if(KW > 1) {
    __syncthreads();
    v4i* redbuf = reinterpret_cast<v4i*>(lds);
    if(kw > 0) {
#pragma unroll
      for(int mt = 0; mt < MT32; ++mt)
#pragma unroll
        for(int q = 0; q < 4; ++q)
          redbuf[((((kw - 1) * WN + wn) * MT32 + mt) * 4 + q) * 64 + lane] =
              v4i{acc[mt][4 * q], acc[mt][4 * q + 1], acc[mt][4 * q + 2], acc[mt][4 * q + 3]};
    }
    __syncthreads();
    if(kw == 0) {
#pragma unroll 1   // one partial sum at a time keeps the register count down
      for(int r = 1; r < KW; ++r)
#pragma unroll
        for(int mt = 0; mt < MT32; ++mt)
#pragma unroll
          for(int q = 0; q < 4; ++q) {
            const v4i t = redbuf[((((r - 1) * WN + wn) * MT32 + mt) * 4 + q) * 64 + lane];
            acc[mt][4 * q] += t.x;
            acc[mt][4 * q + 1] += t.y;
            acc[mt][4 * q + 2] += t.z;
            acc[mt][4 * q + 3] += t.w;
          }
    }
  }

  // ---- epilogue: element v of lane (li, lg) is weight row 8*(v/4) + 4*lg + v%4 of the tile,
  //      activation row li ----
  if(args.prof) tp[4] = clock64();
  if(kw == 0) {
    const float unquant = unquant_mult(FUSED ? aqm : aqm_pre, bqm, args.scale);
    const bool has_bias = args.bias != nullptr;
#pragma unroll
    for(int mt = 0; mt < MT32; ++mt) {
      const int m = m_base + mt * 32 + li;
#pragma unroll
      for(int q = 0; q < 4; ++q) {
        const int n = n0 + 8 * q + 4 * lg;
        if(m >= M || n >= args.n_out) continue;
        const size_t off = (size_t)m * (size_t)args.n_out + (size_t)n;
        const v4i a4 = v4i{acc[mt][4 * q], acc[mt][4 * q + 1], acc[mt][4 * q + 2], acc[mt][4 * q + 3]};
        if(args.dump) {
          *reinterpret_cast<v4i*>(reinterpret_cast<int32_t*>(args.out) + off) = a4;
          continue;
        }
        // y = float(acc) * unquant (+ bias); relu: y > 0 ? y : 0; mul and add round separately
        v4f y;
        y.x = (float)a4.x * unquant;
        y.y = (float)a4.y * unquant;
        y.z = (float)a4.z * unquant;
        y.w = (float)a4.w * unquant;
        if(has_bias) {
          y.x = y.x + bias_v[q].x;
          y.y = y.y + bias_v[q].y;
          y.z = y.z + bias_v[q].z;
          y.w = y.w + bias_v[q].w;
        }
        if(args.relu) {
          y.x = y.x > 0.0f ? y.x : 0.0f;
          y.y = y.y > 0.0f ? y.y : 0.0f;
          y.z = y.z > 0.0f ? y.z : 0.0f;
          y.w = y.w > 0.0f ? y.w : 0.0f;
        }
        *reinterpret_cast<v4f*>(reinterpret_cast<float*>(args.out) + off) = y;
      }
    }
  }
  if(args.prof && tid == 0) {
    long long* p = args.prof + ((size_t)blockIdx.y * gridDim.x + blockIdx.x) * 8;
    p[0] = tp[0]; p[1] = tp[1]; p[2] = tp[2]; p[3] = tp[3]; p[4] = tp[4]; p[5] = clock64();
    p[6] = wall_clock64();
  }
}

}  // namespace marian_hip
