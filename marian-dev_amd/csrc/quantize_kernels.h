// abs-max + int8 quantize kernels (activation prepareA and offline weight prepareB).
#pragma once

#include "int8_common.h"
#include "quantize_common.h"

namespace marian_hip {

// Pass 1: per-workgroup abs-max of n floats (n % 4 == 0) -> partials[blockIdx.x].
__global__ __launch_bounds__(kQuantThreads) void absmax_partial_kernel(
    const float* __restrict__ x, size_t n4, float* __restrict__ partials) {
  __shared__ float red[kQuantThreads / kWave];
  const v4f* x4 = reinterpret_cast<const v4f*>(x);
  float m = 0.0f;
  size_t stride = (size_t)gridDim.x * blockDim.x;
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  // four independent loads in flight per thread
  for(; i + 3 * stride < n4; i += 4 * stride) {
    v4f a = x4[i], b = x4[i + stride], c = x4[i + 2 * stride], d = x4[i + 3 * stride];
    m = abs4max(a, m); m = abs4max(b, m); m = abs4max(c, m); m = abs4max(d, m);
  }
  for(; i < n4; i += stride) m = abs4max(x4[i], m);
  m = block_max(m, red);
  if(threadIdx.x == 0) partials[blockIdx.x] = m;
}

// Clears n floats (a kernel rather than a memset node, so callers may capture the call in a graph).
__global__ __launch_bounds__(kQuantThreads) void zero_floats_kernel(float* __restrict__ p, int n) {
  for(int i = blockIdx.x * blockDim.x + threadIdx.x; i < n; i += gridDim.x * blockDim.x) p[i] = 0.0f;
}

// Pass 2 of prepareA: reduce the partials, quantize 16 values per thread per step, block 0
// writes the quantMult tail at byte n.
__global__ __launch_bounds__(kQuantThreads) void quantize_a_kernel(
    const float* __restrict__ x, size_t n16, const float* __restrict__ partials, int n_partials,
    int8_t* __restrict__ out) {
  __shared__ float red[kQuantThreads / kWave];
  float m = 0.0f;
  for(int p = threadIdx.x; p < n_partials; p += blockDim.x) m = fmaxf(m, partials[p]);
  m = block_max(m, red);
  const float qm = quant_mult_from_maxabs(m);
  const v4f* x4 = reinterpret_cast<const v4f*>(x);
  uint4* o16 = reinterpret_cast<uint4*>(out);
  size_t stride = (size_t)gridDim.x * blockDim.x;
  for(size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n16; i += stride) {
    v4f a = x4[4 * i], b = x4[4 * i + 1], c = x4[4 * i + 2], d = x4[4 * i + 3];
    uint4 q;
    q.x = quantize_pack4(a, qm);
    q.y = quantize_pack4(b, qm);
    q.z = quantize_pack4(c, qm);
    q.w = quantize_pack4(d, qm);
    o16[i] = q;
  }
  if(blockIdx.x == 0 && threadIdx.x == 0) *reinterpret_cast<float*>(out + n16 * 16) = qm;
}

// Small activations: one workgroup computes abs-max and quantizes (one launch instead of two).
__global__ __launch_bounds__(kSingleBlockThreads) void prepare_a_single_block_kernel(
    const float* __restrict__ x, int n16, int8_t* __restrict__ out) {
  __shared__ float red[kSingleBlockThreads / kWave];
  const v4f* x4 = reinterpret_cast<const v4f*>(x);
  float m = 0.0f;
  // (eight loads in flight per thread; positions past the end are clamped - a repeated value does
  // not change a maximum)
  const int n4 = n16 * 4;
  for(int i = threadIdx.x; i < n4; i += 8 * kSingleBlockThreads) {
    v4f v[8];
#pragma unroll
    for(int u = 0; u < 8; ++u) v[u] = x4[min(i + u * kSingleBlockThreads, n4 - 1)];
#pragma unroll
    for(int u = 0; u < 8; ++u) m = abs4max(v[u], m);
  }
  m = block_max(m, red);
  const float qm = quant_mult_from_maxabs(m);
  uint4* o16 = reinterpret_cast<uint4*>(out);
  for(int i = threadIdx.x; i < n16; i += blockDim.x) {
    v4f a = x4[4 * i], b = x4[4 * i + 1], c = x4[4 * i + 2], d = x4[4 * i + 3];
    uint4 q;
    q.x = quantize_pack4(a, qm);
    q.y = quantize_pack4(b, qm);
    q.z = quantize_pack4(c, qm);
    q.w = quantize_pack4(d, qm);
    o16[i] = q;
  }
  if(threadIdx.x == 0) *reinterpret_cast<float*>(out + (size_t)n16 * 16) = qm;
}

// ---- prepareA in one pass over the input ----------------------------------------------------
// The two-pass form reads the fp32 input twice (abs-max, then quantize); at encoder sizes the
// second read costs as much as the first (67 MB: 14 us each, the memory-side cache does not help).
// Here the input stays in registers between the two steps: at most one workgroup of 1024 threads
// per CU, each thread holding SETS x 16 values, so 256 CUs hold up to 16.7 M values (4096 x 4096).
// In between, the workgroups exchange their abs-max through the workspace:
//   * every workgroup stores (tag, abs-max bits) into its arrival slot - one 8-byte store at device
//     scope, so tag and value arrive together;
//   * workgroup 0 polls all slots (one slot per thread), takes the maximum and publishes (tag, max)
//     to 16 mailboxes; the other workgroups poll one mailbox each (16 pollers per line);
//   * nothing but these 8-byte words is handed over, so no fence is needed.
// The tag is a host nonce plus a generation word that lives in the workspace and that workgroup 0
// advances at the end of every launch: words left by an earlier launch - or by an earlier replay of
// a recorded graph, which repeats the nonce - never match, whatever the workspace held before its
// first use.  Every wait is bounded: a workgroup that runs out of patience (the device was shared
// and not all workgroups were resident) takes the abs-max over the whole input itself - the
// result is the same - clears its slot, and the launch still ends.
template <int SETS>
__global__ __launch_bounds__(1024) void prepare_a_onepass_kernel(const float* __restrict__ x, unsigned n16,
                                                                 int8_t* __restrict__ out,
                                                                 unsigned long long* slots,
                                                                 unsigned long long* gen_word,
                                                                 unsigned long long* mailboxes,
                                                                 unsigned nonce, int spin_limit) {
  __shared__ float red[1024 / kWave];
  __shared__ float shared_max;
  __shared__ unsigned shared_tag;
  __shared__ __attribute__((aligned(16))) uint32_t turn[1024 * 4];   // 16 bytes per thread
  const int tid = threadIdx.x, quad = tid / 4, qlane = tid % 4;
  const int G = gridDim.x, g = blockIdx.x;
  // (one thread per workgroup asks for the generation: every access to the word is served by the
  // same memory channel, one after the other)
  unsigned gen = 0;
  if(tid == 0 && G > 1) gen = (unsigned)__hip_atomic_load(gen_word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  // set j of this workgroup: quads (g * SETS + j) * 256 .. + 255, a quad = four consecutive 16-value
  // groups (256 contiguous bytes); load e brings lane i of the quad the i-th four values of group e
  v4f vals[SETS][4];
  bool live[SETS];
  float m = 0.0f;
#pragma unroll
  for(int j = 0; j < SETS; ++j) {
    const unsigned q = (unsigned)(g * SETS + j) * 256u + (unsigned)quad;
    live[j] = 4u * q < n16;   // (n16 is a multiple of four: K % 64 == 0)
    const unsigned qc = live[j] ? q : 0u;
    const char* src = reinterpret_cast<const char*>(x) + (size_t)qc * 256 + qlane * 16;
#pragma unroll
    for(int e = 0; e < 4; ++e) vals[j][e] = *reinterpret_cast<const v4f*>(src + e * 64);
  }
#pragma unroll
  for(int j = 0; j < SETS; ++j)
    if(live[j]) {
#pragma unroll
      for(int e = 0; e < 4; ++e) m = abs4max(vals[j][e], m);
    }
  if(tid == 0) shared_tag = (nonce + gen) | 0x80000000u;   // never 0: a cleared word does not match
  m = block_max(m, red);   // (its barriers also publish shared_tag)
  const unsigned tag = shared_tag;

  // abs-max over all of x by this workgroup alone (the way out of a wait that ran out)
  auto scan_all = [&]() {
    const v4f* x4 = reinterpret_cast<const v4f*>(x);
    const size_t n4 = (size_t)n16 * 4;
    float mm = 0.0f;
    for(size_t i = tid; i < n4; i += 1024) mm = abs4max(x4[i], mm);
    return block_max(mm, red);
  };
  auto pack = [](unsigned t, float v) { return ((unsigned long long)t << 32) | (unsigned long long)__float_as_uint(v); };
  float amax = m;
  if(G > 1) {
    if(tid == 0) __hip_atomic_store(&slots[g * kOnePassStride], pack(tag, m), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    bool ok = true;
    if(g == 0) {
      float mine = 0.0f;
      if(tid < G) {
        ok = false;
        for(int spin = 0; spin < spin_limit; ++spin) {
          const unsigned long long w = __hip_atomic_load(&slots[tid * kOnePassStride], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          if((unsigned)(w >> 32) == tag) {
            mine = __uint_as_float((unsigned)w);
            ok = true;
            break;
          }
          __builtin_amdgcn_s_sleep(4);
        }
      }
      const bool all_ok = __syncthreads_and(ok ? 1 : 0) != 0;
      amax = all_ok ? block_max(mine, red) : scan_all();
      if(tid < kOnePassMailboxes)
        __hip_atomic_store(&mailboxes[tid * 32], pack(tag, amax), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      // the next launch (or replay) expects another tag; every workgroup of this launch has read
      // the generation by now, or will find its words unanswered and help itself
      if(tid == 0) {
        __hip_atomic_store(gen_word, (unsigned long long)(gen + 1u), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __hip_atomic_store(&slots[0], 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
    } else {
      if(tid == 0) {
        ok = false;
        const unsigned long long* box = &mailboxes[(g % kOnePassMailboxes) * 32];
        for(int spin = 0; spin < spin_limit; ++spin) {
          const unsigned long long w = __hip_atomic_load(box, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          if((unsigned)(w >> 32) == tag) {
            shared_max = __uint_as_float((unsigned)w);
            ok = true;
            break;
          }
          __builtin_amdgcn_s_sleep(8);
        }
        // answered or not, this launch is done with the slot
        __hip_atomic_store(&slots[g * kOnePassStride], 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
      const bool answered = __syncthreads_and(ok ? 1 : 0) != 0;
      amax = answered ? shared_max : scan_all();
    }
  }
  const float qm = quant_mult_from_maxabs(amax);
  const bool finite = qm < __builtin_inff();
#pragma unroll
  for(int j = 0; j < SETS; ++j) {
    if(!live[j]) continue;
    const unsigned q = (unsigned)(g * SETS + j) * 256u + (unsigned)quad;
    // Lane i of the quad holds dword i of the quad's four 16-byte outputs; through LDS (the four
    // lanes sit in one wave, whose LDS operations execute in order) it picks up the four dwords of
    // output i, so that a wave stores 1 KB of contiguous bytes, 16 per lane.
#pragma unroll
    for(int e = 0; e < 4; ++e)
      turn[(quad * 4 + e) * 4 + qlane] = finite ? quantize_pack4_finite(vals[j][e], qm) : quantize_pack4(vals[j][e], qm);
    const uint4 w = *reinterpret_cast<const uint4*>(&turn[(quad * 4 + qlane) * 4]);
    *reinterpret_cast<uint4*>(reinterpret_cast<char*>(out) + (size_t)q * 64 + qlane * 16) = w;
  }
  if(g == 0 && tid == 0) *reinterpret_cast<float*>(out + (size_t)n16 * 16) = qm;
}

// Quantization alone for large inputs whose abs-max is known (left in `partials` by the kernel that
// produced x): the memory access pattern of the one-pass kernel above - a quad of lanes reads 64
// contiguous bytes per load, four loads in flight per thread (eight while the next set is on its
// way), the packed bytes take a turn through LDS so that a wave stores 1 KB of contiguous output -
// without its exchange.  A set = 256 quads = 64 KB of input per workgroup and step.
__global__ __launch_bounds__(1024) void quantize_a_wide_kernel(const float* __restrict__ x, unsigned n16,
                                                               const float* __restrict__ partials, int n_partials,
                                                               int8_t* __restrict__ out) {
  __shared__ float red[1024 / kWave];
  __shared__ __attribute__((aligned(16))) uint32_t turn[1024 * 4];   // 16 bytes per thread
  const int tid = threadIdx.x, quad = tid / 4, qlane = tid % 4;
  const unsigned n_sets = (n16 / 4 + 255) / 256;
  auto load_set = [&](unsigned set, v4f (&v)[4]) {
    const unsigned q = set * 256u + (unsigned)quad;
    const unsigned qc = 4u * q < n16 ? q : 0u;   // (n16 is a multiple of four: whole quads)
    const char* src = reinterpret_cast<const char*>(x) + (size_t)qc * 256 + qlane * 16;
#pragma unroll
    for(int e = 0; e < 4; ++e) v[e] = *reinterpret_cast<const v4f*>(src + e * 64);
  };
  // the first loads are on their way while the partials are reduced
  unsigned set = blockIdx.x;
  v4f vals[4];
  if(set < n_sets) load_set(set, vals);
  float m = 0.0f;
  for(int p = tid; p < n_partials; p += 1024) m = fmaxf(m, partials[p]);
  m = block_max(m, red);
  const float qm = quant_mult_from_maxabs(m);
  const bool finite = qm < __builtin_inff();
  for(; set < n_sets; set += gridDim.x) {
    v4f cur[4];
#pragma unroll
    for(int e = 0; e < 4; ++e) cur[e] = vals[e];
    if(set + gridDim.x < n_sets) load_set(set + gridDim.x, vals);
    const unsigned q = set * 256u + (unsigned)quad;
    if(4u * q < n16) {
      // (the four lanes of a quad sit in one wave, whose LDS operations execute in order)
#pragma unroll
      for(int e = 0; e < 4; ++e)
        turn[(quad * 4 + e) * 4 + qlane] = finite ? quantize_pack4_finite(cur[e], qm) : quantize_pack4(cur[e], qm);
      const uint4 w = *reinterpret_cast<const uint4*>(&turn[(quad * 4 + qlane) * 4]);
      *reinterpret_cast<uint4*>(reinterpret_cast<char*>(out) + (size_t)q * 64 + qlane * 16) = w;
    }
  }
  if(blockIdx.x == 0 && tid == 0) *reinterpret_cast<float*>(out + (size_t)n16 * 16) = qm;
}

// Pass 2 of prepareB: W fp32 [K x N] -> K-blocked int8 payload of the quantized transpose + tail.
// A workgroup transposes a 64(k) x 64(n) tile through LDS: reads are coalesced along n, writes are
// 16-byte chunks of K values, the columns of a K sub-step side by side.
__global__ __launch_bounds__(256) void quantize_b_transpose_kernel(
    const float* __restrict__ W, int K, int N, const float* __restrict__ partials,
    int n_partials, int8_t* __restrict__ out) {
  __shared__ float red[256 / kWave];
  // [n][k / 4] as packed dwords, 17 dwords per row: the 64 lanes of a wave (consecutive n, one k
  // group) hit every bank twice, the minimum for 64 lanes on 32 banks
  __shared__ uint32_t tile[64][17];
  float m = 0.0f;
  for(int p = threadIdx.x; p < n_partials; p += blockDim.x) m = fmaxf(m, partials[p]);
  m = block_max(m, red);
  const float qm = quant_mult_from_maxabs(m);

  const int n0 = blockIdx.x * 64, k0 = blockIdx.y * 64;
  const int tn = threadIdx.x % 64, tk = threadIdx.x / 64;  // wave tk takes k rows 16*tk .. 16*tk+15
  const int n_in = n0 + tn;
#pragma unroll
  for(int g = 0; g < 4; ++g) {
    const int kk = tk * 16 + g * 4;   // four consecutive k of column n: one packed dword
    v4f v = v4f{0.0f, 0.0f, 0.0f, 0.0f};
    if(n_in < N) {   // (K % 64 == 0: the k rows of a tile are all inside)
      const float* w = W + (size_t)(k0 + kk) * N + n_in;
      v = v4f{w[0], w[(size_t)N], w[2 * (size_t)N], w[3 * (size_t)N]};
    }
    tile[tn][kk / 4] = quantize_pack4(v, qm);
  }
  __syncthreads();
  // 64 columns (n) x four 16-byte chunks (k): two neighbouring threads write the two halves of a
  // column's sub-step, a wave 32 columns of one sub-step (1 KB of consecutive memory)
  const int rn = (threadIdx.x / 2) % 64, ck = (threadIdx.x / 128) * 32 + (threadIdx.x % 2) * 16;
  int n = n0 + rn, k = k0 + ck;
  if(n < N && k < K) {  // K % 64 == 0, so a 16-byte run is inside or outside as a whole
    uint4 v;
    v.x = tile[rn][ck / 4]; v.y = tile[rn][ck / 4 + 1]; v.z = tile[rn][ck / 4 + 2]; v.w = tile[rn][ck / 4 + 3];
    *reinterpret_cast<uint4*>(out + b_chunk_offset(n, k / 16, N)) = v;
  }
  if(blockIdx.x == 0 && blockIdx.y == 0 && threadIdx.x == 0)
    *reinterpret_cast<float*>(out + (size_t)K * N) = qm;
}

// prepareBQuantizedTransposed: int8 W^T as plain rows [N x K] (the payload of a model file) -> the
// K-blocked layout.  One 16-byte chunk per thread, in output order (writes are consecutive).
__global__ __launch_bounds__(256) void retile_b_kernel(const int8_t* __restrict__ in, int K, int N,
                                                       int8_t* __restrict__ out) {
  const size_t chunks = (size_t)K * (size_t)N / 16;
  const size_t o = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if(o < chunks) {
    // chunk o of the output: sub-step o / (2 N), then column, half
    const int s = (int)(o / (2 * (size_t)N)), rem = (int)(o % (2 * (size_t)N));
    const int n = rem / 2, half = rem % 2;
    const uint4 v = *reinterpret_cast<const uint4*>(in + (size_t)n * K + (size_t)(2 * s + half) * 16);
    *reinterpret_cast<uint4*>(out + o * 16) = v;
  }
  if(o == 0) *reinterpret_cast<float*>(out + (size_t)K * N) = *reinterpret_cast<const float*>(in + (size_t)K * N);
}

}  // namespace marian_hip
