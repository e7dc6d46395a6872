// Machine-ceiling probes (tuning build only): what the memory system and the matrix cores deliver to
// kernels of this library's shapes when no arithmetic or no memory traffic is in the way.  The
// figures they give are the yardsticks the kernels' measured times are held against.
#pragma once

#include "gemm_mfma32_kernel.h"
#include "int8_common.h"

namespace marian_hip {

// Every thread reads its share of `read_bytes` (16 bytes per load, `U` loads in flight, grid
// stride), then - after all its loads have returned, like a kernel that needs its whole input
// before it can write - stores its share of `write_bytes`.  The stored value depends on what was
// read, so nothing is optimised away.  NT: non-temporal stores.
template <int U, bool NT>
__global__ __launch_bounds__(1024) void probe_stream_kernel(const v4i* __restrict__ src, size_t read_vecs,
                                                            v4i* __restrict__ dst, size_t write_vecs) {
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  v4i acc = {0, 0, 0, 0};
  for(; i + (U - 1) * stride < read_vecs; i += U * stride) {
    v4i v[U];
#pragma unroll
    for(int u = 0; u < U; ++u) v[u] = src[i + u * stride];
#pragma unroll
    for(int u = 0; u < U; ++u) acc ^= v[u];
  }
  for(; i < read_vecs; i += stride) acc ^= src[i];
  for(size_t o = (size_t)blockIdx.x * blockDim.x + threadIdx.x; o < write_vecs; o += stride) {
    if(NT) __builtin_nontemporal_store(acc, dst + o);
    else dst[o] = acc;
  }
}

// A wave issues `iters` rounds of eight independent v_mfma_i32_32x32x32_i8 on operands loaded from
// `data` (so that the multipliers see real bit patterns: the sustained clock depends on them).
// clocks[workgroup] = {shader clocks, 100 MHz reference clocks} of wave 0; sink keeps the results live.
__global__ __launch_bounds__(256) void probe_mfma_kernel(const v4i* __restrict__ data, int iters,
                                                         long long* __restrict__ clocks, int* __restrict__ sink) {
  typedef int v16 __attribute__((ext_vector_type(16)));
  const int lane = threadIdx.x % 64;
  const v4i a0 = data[lane], a1 = data[64 + lane], b0 = data[128 + lane], b1 = data[192 + lane];
  v16 acc[8];
#pragma unroll
  for(int t = 0; t < 8; ++t)
#pragma unroll
    for(int v = 0; v < 16; ++v) acc[t][v] = 0;
  __syncthreads();
  const long long c0 = clock64(), w0 = wall_clock64();
  for(int it = 0; it < iters; ++it) {
#pragma unroll
    for(int t = 0; t < 8; ++t)
      acc[t] = __builtin_amdgcn_mfma_i32_32x32x32_i8((t & 1) ? a1 : a0, (t & 2) ? b1 : b0, acc[t], 0, 0, 0);
  }
  const long long c1 = clock64(), w1 = wall_clock64();
  int s = 0;
#pragma unroll
  for(int t = 0; t < 8; ++t)
#pragma unroll
    for(int v = 0; v < 16; ++v) s ^= acc[t][v];
  if(s == 0x7fffffff) sink[0] = s;   // (practically never: keeps the accumulators live)
  if(threadIdx.x == 0) {
    clocks[2 * blockIdx.x] = c1 - c0;
    clocks[2 * blockIdx.x + 1] = w1 - w0;
  }
}

// One CU's LDS, vector L1 and matrix cores under a chosen instruction mix, without anything else in
// the way.  Every wave repeats `iters` times a body of 16 slots over which R conflict-free
// ds_read_b128 (1 KB per wave each), M v_mfma_i32_32x32x32_i8, D global_load_lds_dwordx4 (1 KB per
// wave from global memory straight into LDS) and G global_load_dwordx4 (1 KB per wave into
// registers) are spread evenly, in that fixed order (inline assembly and scheduling barriers).
// Global addresses walk over `span` bytes (a power of two) behind src, 1 KB per wave load, workgroup
// b starting b * stagger bytes in: a small span and stagger make the loads hit the vector L1 or the
// XCD's L2 (the workgroups follow each other over the same lines), a large span cut into one
// region per workgroup (stagger = span / workgroups) makes them stream from HBM.  Up to 12 LDS reads and
// 24 vector-memory loads of a wave are in flight.  clocks[2 * workgroup] = shader clocks,
// [2 * workgroup + 1] = 100 MHz reference clocks from the common start until the last wave has finished.
// SPLIT (eight waves): the first four waves, one per SIMD, issue only the LDS reads and the matrix
// instructions, the other four only the global loads - a wave that cannot issue a load because the
// vector memory path is full then does not hold up matrix instructions behind it.
template <int R, int M, int D, int G, bool SPLIT = false>
__global__ __launch_bounds__(M > 0 ? 512 : 1024) void probe_mix_kernel(const int8_t* __restrict__ src, unsigned span, unsigned stagger, int iters,
                                                         long long* __restrict__ clocks, int* __restrict__ sink) {
  extern __shared__ __attribute__((aligned(16))) int8_t lds[];   // 64 KB that are read + 64 KB that the DMA fills
  const unsigned lds_base = (unsigned)(size_t)lds;
  const int lane = threadIdx.x % kWave;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  const int waves = blockDim.x / kWave;
  const v4i a0 = reinterpret_cast<const v4i*>(src)[lane], a1 = reinterpret_cast<const v4i*>(src)[64 + lane];
  const v4i b0 = reinterpret_cast<const v4i*>(src)[128 + lane], b1 = reinterpret_cast<const v4i*>(src)[192 + lane];
  for(int i = threadIdx.x; i < 65536 / 16; i += blockDim.x)
    reinterpret_cast<v4i*>(lds)[i] = reinterpret_cast<const v4i*>(src)[i & 255];
  v16i acc[M > 0 ? 8 : 1];
#pragma unroll
  for(int t = 0; t < (M > 0 ? 8 : 1); ++t)
#pragma unroll
    for(int v = 0; v < 16; ++v) acc[t][v] = 0;
  const unsigned rd_addr = lds_base + (unsigned)((wave % 8) * 8192 + lane * 16);
  const unsigned voff = (unsigned)lane * 16u;
  const unsigned step = (unsigned)(SPLIT ? 4 : waves) * 1024u;
  unsigned goff = __builtin_amdgcn_readfirstlane(((unsigned)blockIdx.x * stagger + (unsigned)wave * 1024u) & (span - 1));
  unsigned dma_slot = (unsigned)wave;
  v4i rd = {0, 0, 0, 0}, gl = {0, 0, 0, 0};
  // (SPLIT: two loops behind one wave-uniform branch, so that neither has a branch per slot)
  auto run = [&](auto loads_c, auto computes_c) __attribute__((always_inline)) {
    constexpr bool loads = decltype(loads_c)::value, computes = decltype(computes_c)::value;
    for(int it = 0; it < iters; ++it) {
#pragma unroll
      for(int s = 0; s < 16; ++s) {
        if(loads && (s * D) / 16 != ((s + 1) * D) / 16) {
          global_load_lds16(src + goff, voff, lds_base + 65536u + (dma_slot & 63u) * 1024u);
          goff = (goff + step) & (span - 1);
          dma_slot += (unsigned)(SPLIT ? 4 : waves);
          wait_vmcnt<24>();
        }
        if(loads && (s * G) / 16 != ((s + 1) * G) / 16) {
          asm volatile("global_load_dwordx4 %0, %1, %2" : "=v"(gl) : "v"(voff), "s"(src + goff) : "memory");
          goff = (goff + step) & (span - 1);
          wait_vmcnt<24>();
        }
        if(computes && (s * R) / 16 != ((s + 1) * R) / 16) {
          asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(rd) : "v"(rd_addr), "n"((s % 8) * 1024) : "memory");
          __builtin_amdgcn_s_waitcnt(0xCC7F);   // lgkmcnt(12), nothing else
        }
        if(computes && (s * M) / 16 != ((s + 1) * M) / 16) {
          const int t = (s * M) / 16;
          acc[t] = __builtin_amdgcn_mfma_i32_32x32x32_i8((t & 1) ? a1 : a0, (t & 2) ? b1 : b0, acc[t], 0, 0, 0);
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  };
  __syncthreads();
  const long long c0 = clock64(), w0 = wall_clock64();
  if(!SPLIT) run(std::true_type(), std::true_type());
  else if(wave >= 4) run(std::true_type(), std::false_type());
  else run(std::false_type(), std::true_type());
  wait_vmcnt<0>();
  wait_lgkmcnt0();
  __syncthreads();   // the time of the slowest wave: waves that share a SIMD do not share it evenly
  const long long c1 = clock64(), w1 = wall_clock64();
  int x = rd.x ^ rd.w ^ gl.x ^ gl.w;
#pragma unroll
  for(int t = 0; t < (M > 0 ? 8 : 1); ++t)
#pragma unroll
    for(int v = 0; v < 16; ++v) x ^= acc[t][v];
  if(x == 0x7fffffff && iters < 0) sink[0] = x;   // (never: keeps the results live)
  if(threadIdx.x == 0) {
    clocks[2 * blockIdx.x] = c1 - c0;
    clocks[2 * blockIdx.x + 1] = w1 - w0;
  }
}

}  // namespace marian_hip
