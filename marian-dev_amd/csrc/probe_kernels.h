// Machine-ceiling probes (tuning build only): what the memory system and the matrix cores deliver to
// kernels of this library's shapes when no arithmetic or no memory traffic is in the way.  The
// figures they give are the yardsticks the kernels' measured times are held against.
#pragma once

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

}  // namespace marian_hip
