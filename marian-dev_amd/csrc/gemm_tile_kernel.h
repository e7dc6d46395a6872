// LDS-tiled int8 MFMA GEMM for large M (encoder shapes, shortlisted output layer).
//
// A workgroup of 4 waves (2 along n x 2 along m) computes a BN x BM block of out^T; both
// operands are K-contiguous in memory (activations [M x K], weights W^T [N x K]), so a wave
// fetches a 16-row x 64-byte operand fragment with one 16-byte load per lane and drops it
// into LDS in lane order (conflict-free ds_write_b128 / ds_read_b128).  K advances in 64-byte
// steps with register-staged double buffering: global loads for step s+1 are in flight while
// step s is multiplied out of LDS.
#pragma once

#include "int8_common.h"

namespace marian_hip {

// WNT / WMT: 16x16 MFMA tiles per wave along n (weights) and m (activations).
template <int WNT, int WMT>
struct TileCfg {
  static constexpr int kThreads = 256;
  static constexpr int kWavesN = 2, kWavesM = 2;
  static constexpr int BN = kWavesN * WNT * 16;
  static constexpr int BM = kWavesM * WMT * 16;
  static constexpr int kFragsN = BN / 16, kFragsM = BM / 16;
  static constexpr int kFrags = kFragsN + kFragsM;     // fragments per K step
  static constexpr int kLoads = kFrags / 4;            // fragments fetched per wave per step
  static constexpr int kStepBytes = kFrags * kFragBytes;
  static constexpr int kLdsBytes = 2 * kStepBytes;
  static_assert(kFrags % 4 == 0, "fragments must divide over 4 waves");
};

// Maps the linear workgroup id to a tile so that workgroups that run on the same XCD (ids
// congruent mod 8 under round-robin dispatch) work on neighbouring tiles and share their
// operand panels in that XCD's L2.
__device__ __forceinline__ void tile_coords(int bid, int tiles_n, int tiles_m, int& tn, int& tm) {
  const int total = tiles_n * tiles_m;
  int t = bid;
  if(total % 8 == 0) {
    const int per_xcd = total / 8;
    t = (bid % 8) * per_xcd + bid / 8;
  }
  // walk m fastest inside bands of 8 n-tiles
  const int band = 8;
  const int band_tiles = band * tiles_m;
  const int b = t / band_tiles;
  const int r = t % band_tiles;
  const int bw = (tiles_n - b * band) < band ? (tiles_n - b * band) : band;
  tn = b * band + r % bw;
  tm = r / bw;
}

template <int WNT, int WMT>
__global__ __launch_bounds__(256) void gemm_tile_kernel(GemmArgs args, int tiles_n, int tiles_m) {
  using Cfg = TileCfg<WNT, WMT>;
  extern __shared__ __attribute__((aligned(16))) int8_t lds[];

  const int tid = threadIdx.x;
  const int wave = tid / kWave, lane = tid % kWave;
  const int wn = wave % 2, wm = wave / 2;
  const int li = lane % 16, lg = lane / 16;
  const int K = args.K, M = args.M;
  const int KS = K / 64;

  int tn, tm;
  tile_coords(blockIdx.x, tiles_n, tiles_m, tn, tm);
  const int n0 = tn * Cfg::BN, m0 = tm * Cfg::BM;

  // Fragments f = 0..kFragsN-1 are weight rows, the rest activation rows; wave w fetches
  // fragments w, w+4, ...  The row a lane fetches is fixed over K, so shortlist ids are
  // resolved once.
  const int8_t* src[Cfg::kLoads];
  bool valid[Cfg::kLoads];
#pragma unroll
  for(int j = 0; j < Cfg::kLoads; ++j) {
    int f = wave + 4 * j;
    if(f < Cfg::kFragsN) {
      int n = n0 + f * 16 + li;
      valid[j] = n < args.n_out;
      int row = valid[j] ? (args.idx ? (int)args.idx[n] : n) : 0;
      src[j] = args.Bq + (size_t)row * (size_t)K + lg * 16;
    } else {
      int m = m0 + (f - Cfg::kFragsN) * 16 + li;
      valid[j] = m < M;
      src[j] = args.Aq + (size_t)(valid[j] ? m : 0) * (size_t)K + lg * 16;
    }
  }

  v4i regs[Cfg::kLoads];
  auto fetch = [&](int s) {
#pragma unroll
    for(int j = 0; j < Cfg::kLoads; ++j) {
      v4i v = {0, 0, 0, 0};
      if(valid[j]) v = load16(src[j] + s * 64);
      regs[j] = v;
    }
  };
  auto stash = [&](int buf) {
#pragma unroll
    for(int j = 0; j < Cfg::kLoads; ++j) {
      int f = wave + 4 * j;
      *reinterpret_cast<v4i*>(lds + buf * Cfg::kStepBytes + f * kFragBytes + lane * 16) = regs[j];
    }
  };

  v4i acc[WNT][WMT];
#pragma unroll
  for(int a = 0; a < WNT; ++a)
#pragma unroll
    for(int b = 0; b < WMT; ++b) acc[a][b] = v4i{0, 0, 0, 0};

  fetch(0);
  stash(0);
  __syncthreads();

  for(int s = 0; s < KS; ++s) {
    const bool more = (s + 1 < KS);
    if(more) fetch(s + 1);
    const int8_t* buf = lds + (s & 1) * Cfg::kStepBytes;
    v4i wf[WNT], af[WMT];
#pragma unroll
    for(int a = 0; a < WNT; ++a)
      wf[a] = *reinterpret_cast<const v4i*>(buf + (wn * WNT + a) * kFragBytes + lane * 16);
#pragma unroll
    for(int b = 0; b < WMT; ++b)
      af[b] = *reinterpret_cast<const v4i*>(buf + (Cfg::kFragsN + wm * WMT + b) * kFragBytes +
                                            lane * 16);
#pragma unroll
    for(int a = 0; a < WNT; ++a)
#pragma unroll
      for(int b = 0; b < WMT; ++b) acc[a][b] = mfma_i8_16x16x64(wf[a], af[b], acc[a][b]);
    if(more) stash((s + 1) & 1);
    __syncthreads();
  }

  const Epilogue ep = make_epilogue(args);
#pragma unroll
  for(int a = 0; a < WNT; ++a)
#pragma unroll
    for(int b = 0; b < WMT; ++b)
      ep.store(acc[a][b], m0 + (wm * WMT + b) * 16 + li, n0 + (wn * WNT + a) * 16 + lg * 4);
}

}  // namespace marian_hip
