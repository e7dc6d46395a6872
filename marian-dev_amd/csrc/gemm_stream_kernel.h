// Weight-streaming int8 GEMM for small M (decode shapes, M <= 128).
//
// The weights W^T [N x K] are read exactly once from HBM, straight into MFMA operand
// registers: lane l of a wave loads 16 consecutive K bytes of weight row n0 + l % 16, which is
// already the 16x16x64 operand layout, so no LDS staging or transposition is needed for them.
// The (small) quantized activations are shared by all waves of a workgroup through LDS in
// operand order.  Waves of a workgroup are arranged WN (different weight rows) x KW (different
// K steps of the same rows, reduced through LDS at the end; the int32 sum is exact in any
// order).
#pragma once

#include "int8_common.h"

namespace marian_hip {

// MT: 16-row activation tiles (M <= 16*MT).  NT: 16-row weight tiles per wave.
// PF: K steps (64 bytes of K each) a wave has in flight per pipeline stage.
template <int MT, int NT, int WN, int KW, int PF>
struct StreamCfg {
  static constexpr int kThreads = WN * KW * kWave;
  static constexpr int kChunkSteps = PF * KW;                    // K steps staged per stage
  static constexpr int kStageBytes = MT * kChunkSteps * kFragBytes;
  static constexpr int kStageLoads = kStageBytes / (kThreads * 16);  // 16-byte loads per thread
  static constexpr int kReduceBytes = (KW - 1) * WN * NT * MT * kFragBytes;
  static constexpr int kLdsBytes =
      (2 * kStageBytes > kReduceBytes) ? 2 * kStageBytes : kReduceBytes;
  static constexpr int kColsPerBlock = WN * NT * 16;
  static_assert(kStageBytes % (kThreads * 16) == 0, "stage must divide evenly over threads");
};

template <int MT, int NT, int WN, int KW, int PF>
__global__ __launch_bounds__(WN * KW * kWave) void gemm_stream_kernel(GemmArgs args) {
  using Cfg = StreamCfg<MT, NT, WN, KW, PF>;
  extern __shared__ __attribute__((aligned(16))) int8_t lds[];

  const int tid = threadIdx.x;
  const int wave = tid / kWave, lane = tid % kWave;
  const int wn = wave % WN, kw = wave / WN;
  const int li = lane % 16, lg = lane / 16;
  const int K = args.K, M = args.M;
  const int KS = K / 64;
  const int n_chunks = (KS + Cfg::kChunkSteps - 1) / Cfg::kChunkSteps;

  // quantMult tails are requested first so that their latency overlaps the operand loads
  const Epilogue ep = make_epilogue(args);

  // weight rows of this lane
  const int n_base = (blockIdx.x * WN + wn) * NT * 16;
  const int8_t* wrow[NT];
  const size_t w_step = 64u * (size_t)args.N;   // bytes from one K step of 64 to the next, for every column
#pragma unroll
  for(int nt = 0; nt < NT; ++nt) {
    int n = n_base + nt * 16 + li;
    int src = 0;
    if(n < args.n_out) src = args.idx ? (int)args.idx[n] : n;
    // 16-byte chunk lg of K step 0: sub-step lg / 2, half lg % 2
    wrow[nt] = args.Bq + stream16_lane_offset(src, lg, args.N);
  }

  // activation staging: 16-byte slot t of a stage is (step, m-tile, lane) in operand order
  // slot = (step * MT + mt) * 64 + l ; source = Aq[(mt*16 + l%16) * K + (s0+step)*64 + (l/16)*16]
  v4i stage[Cfg::kStageLoads];
  auto load_stage = [&](int chunk) {
    const int s0 = chunk * Cfg::kChunkSteps;
#pragma unroll
    for(int j = 0; j < Cfg::kStageLoads; ++j) {
      int slot = j * Cfg::kThreads + tid;
      int l = slot % 64, f = slot / 64;
      int mt = f % MT, step = f / MT;
      int m = mt * 16 + (l % 16);
      int s = s0 + step;
      v4i v = {0, 0, 0, 0};
      if(m < M && s < KS) v = load16(args.Aq + (size_t)m * (size_t)K + s * 64 + (l / 16) * 16);
      stage[j] = v;
    }
  };
  auto store_stage = [&](int buf) {
#pragma unroll
    for(int j = 0; j < Cfg::kStageLoads; ++j) {
      int slot = j * Cfg::kThreads + tid;
      *reinterpret_cast<v4i*>(lds + buf * Cfg::kStageBytes + slot * 16) = stage[j];
    }
  };

  // weight pipeline: this wave's K steps of a chunk are s0 + p*KW + kw, p = 0..PF-1
  v4i wcur[PF][NT], wnext[PF][NT];
  auto load_weights = [&](int chunk, v4i (&w)[PF][NT]) {
    const int s0 = chunk * Cfg::kChunkSteps;
#pragma unroll
    for(int p = 0; p < PF; ++p) {
      int s = s0 + p * KW + kw;
#pragma unroll
      for(int nt = 0; nt < NT; ++nt) {
        v4i v = {0, 0, 0, 0};
        if(s < KS) v = load16(wrow[nt] + (size_t)s * w_step);
        w[p][nt] = v;
      }
    }
  };

  v4i acc[NT][MT];
#pragma unroll
  for(int nt = 0; nt < NT; ++nt)
#pragma unroll
    for(int mt = 0; mt < MT; ++mt) acc[nt][mt] = v4i{0, 0, 0, 0};

  load_weights(0, wcur);
  load_stage(0);
  store_stage(0);
  __syncthreads();

  for(int c = 0; c < n_chunks; ++c) {
    const bool more = (c + 1 < n_chunks);
    if(more) {
      load_weights(c + 1, wnext);
      load_stage(c + 1);
    }
    const int8_t* abuf = lds + (c & 1) * Cfg::kStageBytes;
#pragma unroll
    for(int p = 0; p < PF; ++p) {
      const int step = p * KW + kw;
#pragma unroll
      for(int mt = 0; mt < MT; ++mt) {
        v4i a = *reinterpret_cast<const v4i*>(abuf + (step * MT + mt) * kFragBytes + lane * 16);
#pragma unroll
        for(int nt = 0; nt < NT; ++nt) acc[nt][mt] = mfma_i8_16x16x64(wcur[p][nt], a, acc[nt][mt]);
      }
    }
    if(more) {
      store_stage((c + 1) & 1);
#pragma unroll
      for(int p = 0; p < PF; ++p)
#pragma unroll
        for(int nt = 0; nt < NT; ++nt) wcur[p][nt] = wnext[p][nt];
    }
    __syncthreads();
  }

  // reduce the KW partial sums (exact int32 adds) into the kw == 0 waves
  if(KW > 1) {
    v4i* red = reinterpret_cast<v4i*>(lds);
    if(kw > 0) {
#pragma unroll
      for(int nt = 0; nt < NT; ++nt)
#pragma unroll
        for(int mt = 0; mt < MT; ++mt)
          red[((((kw - 1) * WN + wn) * NT + nt) * MT + mt) * 64 + lane] = acc[nt][mt];
    }
    __syncthreads();
    if(kw == 0) {
#pragma unroll
      for(int q = 1; q < KW; ++q)
#pragma unroll
        for(int nt = 0; nt < NT; ++nt)
#pragma unroll
          for(int mt = 0; mt < MT; ++mt)
            acc[nt][mt] += red[((((q - 1) * WN + wn) * NT + nt) * MT + mt) * 64 + lane];
    }
  }

  if(kw == 0) {
#pragma unroll
    for(int nt = 0; nt < NT; ++nt)
#pragma unroll
      for(int mt = 0; mt < MT; ++mt)
        ep.store(acc[nt][mt], mt * 16 + li, n_base + nt * 16 + lg * 4);
  }
}

}  // namespace marian_hip
