// Float32 operators between the int8 GEMMs of a transformer decode step: layer normalization
// (with the skip connection in front of it), softmax (with the attention mask in front of it),
// log-softmax, the 0213 transpose of the head split/join, and the batched attention products.
// Declarations and the reference code each entry point replaces: include/marian_hip_ops.h
//
// All of them are memory- or latency-bound at decode sizes (a few hundred KB per call), so the
// kernels are single-pass where the row fits in registers and use 64-lane wave reductions;
// nothing here needs LDS tiling or MFMA.
#include "../../include/marian_hip_ops.h"

#include <hip/hip_runtime.h>

#include <atomic>
#include <cmath>

#include "../../include/marian_hip_int8.h"
#include "abi_common.h"
#include "int8_common.h"
#include "nbest_plan.h"
#include "quantize_common.h"

using namespace marian_hip;

namespace {

constexpr int64_t kMaxElemsOps = 2147483647LL;

// Sum over each group of 16 consecutive lanes, left in all 16 of them (four DPP steps: the two
// lane swaps within a quad, then the mirror within half a row and within the row).
__device__ __forceinline__ float row16_sum(float v) {
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xB1, 0xF, 0xF, false));   // quad_perm [1,0,3,2]
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x4E, 0xF, 0xF, false));   // quad_perm [2,3,0,1]
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x141, 0xF, 0xF, false));  // row_half_mirror
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x140, 0xF, 0xF, false));  // row_mirror
  return v;
}
// Sum over the wave, the same value in all lanes: within the rows of 16 lanes, then across them
// with the two row-broadcast DPP steps (rows 1 and 3 take in the last lane of the row before them,
// then rows 2 and 3 the last lane of row 1), which leaves the total in lane 63, read from there as
// a scalar.  No step goes through the LDS crossbar (a lane exchange there costs ten times a DPP
// step).  All lanes of the wave must be active.
__device__ __forceinline__ float wave_sum(float v) {
  v = row16_sum(v);
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x142, 0xA, 0xF, false));   // row_bcast:15
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x143, 0xC, 0xF, false));   // row_bcast:31
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 63));
}
// Maximum over the wave, the same value in all lanes (`t > v ? t : v` at every step): the same
// steps.
__device__ __forceinline__ float wave_maxf(float v) {
  auto pick = [](float t, float v) { return t > v ? t : v; };
  v = pick(__builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xB1, 0xF, 0xF, false)), v);
  v = pick(__builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x4E, 0xF, 0xF, false)), v);
  v = pick(__builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x141, 0xF, 0xF, false)), v);
  v = pick(__builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x140, 0xF, 0xF, false)), v);
  v = pick(__builtin_bit_cast(float, __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, v), __builtin_bit_cast(int, v), 0x142, 0xA, 0xF, false)), v);   // row_bcast:15
  v = pick(__builtin_bit_cast(float, __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, v), __builtin_bit_cast(int, v), 0x143, 0xC, 0xF, false)), v);   // row_bcast:31
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 63));
}

// Reduction over the THREADS threads that share a row (64: one wave, no LDS; more: through LDS).
// red: one float per wave of the workgroup.
template <int THREADS, bool MAX>
__device__ __forceinline__ float row_reduce(float v, float* red) {
  v = MAX ? wave_maxf(v) : wave_sum(v);
  if(THREADS > 64) {
    const int wave = threadIdx.x / 64, lane = threadIdx.x % 64;
    __syncthreads();
    if(lane == 0) red[wave] = v;
    __syncthreads();
    float r = red[0];
#pragma unroll
    for(int w = 1; w < THREADS / 64; ++w) r = MAX ? (red[w] > r ? red[w] : r) : r + red[w];
    v = r;
  }
  return v;
}

// The same for a `red` that nothing has read or written since the last workgroup barrier (a
// fresh array per reduction): no barrier in front.
template <int THREADS, bool MAX>
__device__ __forceinline__ float row_reduce_fresh(float v, float* red) {
  v = MAX ? wave_maxf(v) : wave_sum(v);
  if(THREADS > 64) {
    const int wave = threadIdx.x / 64, lane = threadIdx.x % 64;
    if(lane == 0) red[wave] = v;
    __syncthreads();
    float r = red[0];
#pragma unroll
    for(int w = 1; w < THREADS / 64; ++w) r = MAX ? (red[w] > r ? red[w] : r) : r + red[w];
    v = r;
  }
  return v;
}

// ---------------------------------------------------------------- layer normalization
// One workgroup of 256 threads per row.  CACHE float4 vectors per thread hold the row in
// registers (cols <= 1024 * CACHE, cols % 4 == 0, 16-byte aligned rows); CACHE == 0 is the
// general form, which re-reads the row (it stays in L2).
template <int CACHE>
__global__ __launch_bounds__(256) void layer_norm_kernel(const float* in,
                                                         const float* __restrict__ add,
                                                         const float* __restrict__ gamma, int gamma_stride,
                                                         const float* __restrict__ beta, int beta_stride,
                                                         float* out, int cols, float eps,
                                                         float* __restrict__ absmax_out, int absmax_wrap) {
  __shared__ float red[4];
  float omax = 0.0f;   // max |y| over what this thread writes
  const size_t row = blockIdx.x;
  const float* x = in + row * cols;
  const float* a = add ? add + row * cols : nullptr;
  float* y = out + row * cols;
  const int tid = threadIdx.x;
  if(CACHE > 0) {
    const int cols4 = cols / 4;
    v4f v[CACHE > 0 ? CACHE : 1];
    // scale and shift are requested together with the row: read where they are used, behind the two
    // reductions, they would cost the kernel another memory round trip
    float gm[CACHE > 0 ? CACHE : 1][4], bt[CACHE > 0 ? CACHE : 1][4];
    float sum = 0.0f;
#pragma unroll
    for(int j = 0; j < CACHE; ++j) {
      const int i = j * 256 + tid;
      v[j] = v4f{0.0f, 0.0f, 0.0f, 0.0f};
      if(i < cols4) {
        v[j] = reinterpret_cast<const v4f*>(x)[i];
        v4f t = v4f{0.0f, 0.0f, 0.0f, 0.0f};
        if(a) t = reinterpret_cast<const v4f*>(a)[i];
#pragma unroll
        for(int e = 0; e < 4; ++e) {
          gm[j][e] = gamma[gamma_stride * (4 * i + e)];
          bt[j][e] = beta ? beta[beta_stride * (4 * i + e)] : 0.0f;
        }
        if(a) {
          v[j].x = v[j].x + t.x; v[j].y = v[j].y + t.y; v[j].z = v[j].z + t.z; v[j].w = v[j].w + t.w;
        }
        sum += (v[j].x + v[j].y) + (v[j].z + v[j].w);
      }
    }
    const float mean = row_reduce<256, false>(sum, red) / (float)cols;
    float sq = 0.0f;
#pragma unroll
    for(int j = 0; j < CACHE; ++j) {
      if(j * 256 + tid < cols4) {
        const float d0 = v[j].x - mean, d1 = v[j].y - mean, d2 = v[j].z - mean, d3 = v[j].w - mean;
        sq += (d0 * d0 + d1 * d1) + (d2 * d2 + d3 * d3);
      }
    }
    const float sigma = sqrtf(row_reduce<256, false>(sq, red) / (float)cols + eps);
#pragma unroll
    for(int j = 0; j < CACHE; ++j) {
      const int i = j * 256 + tid;
      if(i < cols4) {
        float r[4] = {v[j].x, v[j].y, v[j].z, v[j].w};
#pragma unroll
        for(int e = 0; e < 4; ++e) {
          float t = gm[j][e] * ((r[e] - mean) / sigma);
          if(beta) t = t + bt[j][e];
          r[e] = t;
          omax = fmaxf(omax, fabsf(t));
        }
        reinterpret_cast<v4f*>(y)[i] = v4f{r[0], r[1], r[2], r[3]};
      }
    }
  } else {
    float sum = 0.0f;
    for(int i = tid; i < cols; i += 256) sum += a ? x[i] + a[i] : x[i];
    const float mean = row_reduce<256, false>(sum, red) / (float)cols;
    float sq = 0.0f;
    for(int i = tid; i < cols; i += 256) {
      const float d = (a ? x[i] + a[i] : x[i]) - mean;
      sq += d * d;
    }
    const float sigma = sqrtf(row_reduce<256, false>(sq, red) / (float)cols + eps);
    for(int i = tid; i < cols; i += 256) {
      float t = gamma[gamma_stride * i] * (((a ? x[i] + a[i] : x[i]) - mean) / sigma);
      if(beta) t = t + beta[beta_stride * i];
      y[i] = t;
      omax = fmaxf(omax, fabsf(t));
    }
  }
  if(absmax_out) {   // slot `row`; workgroup 0 zeroes the slots past the last row
    omax = row_reduce<256, true>(omax, red);
    if(absmax_wrap) {
      // more rows than slots: the rows share the slots (cleared by the launcher) through an integer
      // maximum on the bits, which orders non-negative floats as the floats themselves
      if(tid == 0) atomicMax(reinterpret_cast<int*>(absmax_out) + (int)(row % kAbsmaxSlots), __float_as_int(omax));
    } else {
      if(tid == 0) absmax_out[row] = omax;
      if(row == 0)
        for(int sl = gridDim.x + tid; sl < kAbsmaxSlots; sl += 256) absmax_out[sl] = 0.0f;
    }
  }
}

// Rows of up to 1024 values: one wave per row and one row per workgroup, four float4 per lane.  The three reductions stay inside the wave, so the kernel has
// no workgroup barrier and no LDS traffic between its load and its store; scale and shift come as
// 16-byte loads (gamma_stride / beta_stride 1, 16-byte aligned) or as one broadcast value (0).
__global__ __launch_bounds__(64) void layer_norm_wave_kernel(const float* in, const float* __restrict__ add,
                                                             const float* __restrict__ gamma, int gamma_stride,
                                                             const float* __restrict__ beta, int beta_stride,
                                                             float* out, int cols, float eps,
                                                             float* __restrict__ absmax_out, int absmax_wrap) {
  constexpr int VPL = 4;
  const size_t row = blockIdx.x;
  const int lane = threadIdx.x, cols4 = cols / 4;
  const v4f* x = reinterpret_cast<const v4f*>(in + row * cols);
  const v4f* a = add ? reinterpret_cast<const v4f*>(add + row * cols) : nullptr;
  v4f* y = reinterpret_cast<v4f*>(out + row * cols);
  const v4f zero = v4f{0.0f, 0.0f, 0.0f, 0.0f};
  v4f v[VPL], t[VPL], gm[VPL], bt[VPL];
  // all loads at once, positions past the row clamped and dropped afterwards
#pragma unroll
  for(int j = 0; j < VPL; ++j) {
    const int i = min(j * 64 + lane, cols4 - 1);
    v[j] = x[i];
    t[j] = a ? a[i] : zero;
    if(gamma_stride) gm[j] = reinterpret_cast<const v4f*>(gamma)[i];
    if(beta && beta_stride) bt[j] = reinterpret_cast<const v4f*>(beta)[i];
  }
  if(!gamma_stride) {
    const float g0 = gamma[0];
#pragma unroll
    for(int j = 0; j < VPL; ++j) gm[j] = v4f{g0, g0, g0, g0};
  }
  if(!(beta && beta_stride)) {
    const float b0 = beta ? beta[0] : 0.0f;
#pragma unroll
    for(int j = 0; j < VPL; ++j) bt[j] = v4f{b0, b0, b0, b0};
  }
  float sum = 0.0f;
#pragma unroll
  for(int j = 0; j < VPL; ++j) {
    if(a) v[j] = v4f{v[j].x + t[j].x, v[j].y + t[j].y, v[j].z + t[j].z, v[j].w + t[j].w};
    if(j * 64 + lane < cols4) sum += (v[j].x + v[j].y) + (v[j].z + v[j].w);
  }
  const float mean = wave_sum(sum) / (float)cols;
  float sq = 0.0f;
#pragma unroll
  for(int j = 0; j < VPL; ++j) {
    if(j * 64 + lane < cols4) {
      const float d0 = v[j].x - mean, d1 = v[j].y - mean, d2 = v[j].z - mean, d3 = v[j].w - mean;
      sq += (d0 * d0 + d1 * d1) + (d2 * d2 + d3 * d3);
    }
  }
  const float sigma = sqrtf(wave_sum(sq) / (float)cols + eps);
  float omax = 0.0f;
#pragma unroll
  for(int j = 0; j < VPL; ++j) {
    const int i = j * 64 + lane;
    if(i < cols4) {
      float r[4] = {v[j].x, v[j].y, v[j].z, v[j].w};
      const float g[4] = {gm[j].x, gm[j].y, gm[j].z, gm[j].w}, b[4] = {bt[j].x, bt[j].y, bt[j].z, bt[j].w};
#pragma unroll
      for(int e = 0; e < 4; ++e) {
        float o = g[e] * ((r[e] - mean) / sigma);
        if(beta) o = o + b[e];
        r[e] = o;
        omax = fmaxf(omax, fabsf(o));
      }
      y[i] = v4f{r[0], r[1], r[2], r[3]};
    }
  }
  if(absmax_out) {   // slot `row`; the slots past the last row are zeroed by all workgroups together
    omax = wave_maxf(omax);
    if(absmax_wrap) {   // more rows than slots, see layer_norm_kernel
      if(lane == 0) atomicMax(reinterpret_cast<int*>(absmax_out) + (int)(row % kAbsmaxSlots), __float_as_int(omax));
    } else {
      if(lane == 0) absmax_out[row] = omax;
      for(int sl = (int)gridDim.x + (int)row * 64 + lane; sl < kAbsmaxSlots; sl += (int)gridDim.x * 64) absmax_out[sl] = 0.0f;
    }
  }
}

// ---------------------------------------------------------------- softmax / log-softmax
// THREADS threads per row, 256 / THREADS... rows per workgroup: 64 (a wave per row, four rows
// per workgroup: attention scores) or 1024 (vocabulary-size rows).  Three passes over the row:
// max, sum of exponentials, result; the row stays in L1/L2 between them.
template <int THREADS, bool LOG>
__global__ __launch_bounds__(THREADS < 256 ? 256 : THREADS) void softmax_kernel(
    const float* in, const float* __restrict__ mask, long long n_masks,
    long long rows_per_mask, float* out, long long rows, int cols) {
  __shared__ float red[THREADS > 64 ? THREADS / 64 : 1];
  constexpr int kRowsPerBlock = THREADS < 256 ? 256 / THREADS : 1;
  const long long row = (long long)blockIdx.x * kRowsPerBlock + (THREADS < 256 ? threadIdx.x / THREADS : 0);
  const int t = threadIdx.x % THREADS;
  if(THREADS <= 64 && row >= rows) return;   // whole waves leave; no workgroup barrier is used
  const float* x = in + (size_t)row * cols;
  const float* m = mask ? mask + (size_t)((row / rows_per_mask) % n_masks) * cols : nullptr;
  float* y = out + (size_t)row * cols;
  float mx = -__builtin_inff();
  for(int i = t; i < cols; i += THREADS) {
    const float v = m ? x[i] + m[i] : x[i];
    mx = v > mx ? v : mx;
  }
  mx = row_reduce<THREADS, true>(mx, red);
  float sum = 0.0f;
  for(int i = t; i < cols; i += THREADS) sum += expf((m ? x[i] + m[i] : x[i]) - mx);
  sum = row_reduce<THREADS, false>(sum, red);
  if(LOG) {
    const float log_sum = logf(sum);
    for(int i = t; i < cols; i += THREADS) y[i] = ((m ? x[i] + m[i] : x[i]) - mx) - log_sum;
  } else {
    for(int i = t; i < cols; i += THREADS) y[i] = expf((m ? x[i] + m[i] : x[i]) - mx) / sum;
  }
}

// Rows kept in registers (cols % 4 == 0, 16-byte aligned rows and mask), so that they are read
// once: 256 threads with four float4 each for rows up to 4096 values, 1024 threads with eight or
// sixteen for vocabulary-size rows (up to 32768 / 65536).  Same
// operations per element as softmax_kernel.
// softmax_wide_row leaves in v (vector j of thread t = elements 4 * (j * THREADS + t) .. + 3 of the
// row, where they exist): LOG: x - max, and returns log(sum of exp(x - max)); otherwise exp(x - max),
// and returns their sum.  red: 2 * THREADS / 64 floats that nothing else uses meanwhile (the wave
// maxima, then the wave sums: no barrier in front of either reduction).  after_max(max, wave maxima)
// runs between the two reductions, when the THREADS / 64 wave maxima are in red[0 ...]; they stay
// there.
struct NoAfterMax {
  __device__ void operator()(float, const float*) const {}
};
template <bool LOG, int THREADS, int VPT, typename AfterMax = NoAfterMax>
__device__ __forceinline__ float softmax_wide_row(const v4f* x, const v4f* mk, int cols4, v4f (&v)[VPT], float* red,
                                                  AfterMax after_max = AfterMax()) {
  const int t = threadIdx.x;
  float mx = -__builtin_inff();
  // (all loads at once, positions past the row clamped and dropped afterwards: a load behind a
  // range check is waited for inside its branch, one memory latency per load)
#pragma unroll
  for(int j = 0; j < VPT; ++j) v[j] = x[min(j * THREADS + t, cols4 - 1)];
  if(mk) {   // (wave-uniform: the whole row has a mask or none)
    v4f mv[VPT];
#pragma unroll
    for(int j = 0; j < VPT; ++j) mv[j] = mk[min(j * THREADS + t, cols4 - 1)];
#pragma unroll
    for(int j = 0; j < VPT; ++j) {
      v[j].x = v[j].x + mv[j].x; v[j].y = v[j].y + mv[j].y; v[j].z = v[j].z + mv[j].z; v[j].w = v[j].w + mv[j].w;
    }
  }
#pragma unroll
  for(int j = 0; j < VPT; ++j) {
    const int i = j * THREADS + t;
    if(i < cols4) {
      const float a = v[j].x > v[j].y ? v[j].x : v[j].y, b = v[j].z > v[j].w ? v[j].z : v[j].w;
      const float c = a > b ? a : b;
      mx = c > mx ? c : mx;
    }
  }
  mx = row_reduce_fresh<THREADS, true>(mx, red);
  after_max(mx, red);
  float sum = 0.0f;
#pragma unroll
  for(int j = 0; j < VPT; ++j) {
    if(j * THREADS + t < cols4) {
      if(LOG) {
        v[j].x = v[j].x - mx; v[j].y = v[j].y - mx; v[j].z = v[j].z - mx; v[j].w = v[j].w - mx;
        // (the exponentials only enter the logarithm of their sum: the hardware exp2 form, about
        // 1e-6 relative, moves log(sum) by 1e-6 absolute, and it is a fifth of the instructions of
        // this kernel's busiest loop)
        sum += (__expf(v[j].x) + __expf(v[j].y)) + (__expf(v[j].z) + __expf(v[j].w));
      } else {
        v[j].x = expf(v[j].x - mx); v[j].y = expf(v[j].y - mx);
        v[j].z = expf(v[j].z - mx); v[j].w = expf(v[j].w - mx);
        sum += (v[j].x + v[j].y) + (v[j].z + v[j].w);
      }
    }
  }
  sum = row_reduce_fresh<THREADS, false>(sum, red + THREADS / 64);
  return LOG ? logf(sum) : sum;
}

template <bool LOG, int THREADS, int VPT>
__global__ __launch_bounds__(THREADS) void softmax_wide_kernel(const float* in, const float* __restrict__ mask,
                                                                long long n_masks, long long rows_per_mask,
                                                                float* out, int cols) {
  __shared__ float red[2 * THREADS / 64];
  const size_t row = blockIdx.x;
  const v4f* x = reinterpret_cast<const v4f*>(in + row * cols);
  const v4f* mk = mask ? reinterpret_cast<const v4f*>(mask + (size_t)((row / rows_per_mask) % n_masks) * cols) : nullptr;
  v4f* y = reinterpret_cast<v4f*>(out + row * cols);
  const int cols4 = cols / 4, t = threadIdx.x;
  v4f v[VPT];
  const float s = softmax_wide_row<LOG, THREADS, VPT>(x, mk, cols4, v, red);   // log(sum) or sum
#pragma unroll
  for(int j = 0; j < VPT; ++j) {
    const int i = j * THREADS + t;
    if(i < cols4) {
      if(LOG) y[i] = v4f{v[j].x - s, v[j].y - s, v[j].z - s, v[j].w - s};
      else y[i] = v4f{v[j].x / s, v[j].y / s, v[j].z / s, v[j].w / s};
    }
  }
}

// ---------------------------------------------------------------- transpose 0213
// One element (VEC floats of the innermost dimension) per thread, indexed by the output.
template <int VEC>
__global__ __launch_bounds__(256) void transpose0213_kernel(const float* in,
                                                            float* __restrict__ out, long long total,
                                                            int d1, int d2, int d3v) {
  const long long stride = (long long)gridDim.x * 256;
  for(long long o = (long long)blockIdx.x * 256 + threadIdx.x; o < total; o += stride) {
    const int i3 = (int)(o % d3v);
    long long r = o / d3v;
    const int i1 = (int)(r % d1);
    r /= d1;
    const int i2 = (int)(r % d2);
    const long long i0 = r / d2;
    const long long src = ((i0 * d1 + i1) * d2 + i2) * d3v + i3;
    if(VEC == 4) reinterpret_cast<v4f*>(out)[o] = reinterpret_cast<const v4f*>(in)[src];
    else out[o] = in[src];
  }
}

// ---------------------------------------------------------------- batched product
// One wave per output row (batch i, row r): lanes walk the n columns, every lane runs over k.
// At decode sizes (m = 1, k or n = 64, a few thousand batch entries) a product is a matrix-vector
// product of a few KB; the operands of a wave stay in L1 while it walks k.
__global__ __launch_bounds__(256) void bdot_kernel(const float* __restrict__ A, const float* __restrict__ B,
                                                   float* __restrict__ C, long long batchA,
                                                   long long batchB, long long rows_total, int m, int n,
                                                   int k, int transA, int transB, float scalar) {
  const long long wr = (long long)blockIdx.x * 4 + threadIdx.x / 64;   // output row of this wave
  if(wr >= rows_total) return;
  const int lane = threadIdx.x % 64;
  const long long i = wr / m;
  const int r = (int)(wr % m);
  const float* a = A + (size_t)(i % batchA) * m * k;
  const float* b = B + (size_t)(i % batchB) * n * k;
  float* c = C + (size_t)wr * n;
  const int lda = transA ? m : k, ldb = transB ? k : n;
  for(int q = lane; q < n; q += 64) {
    float s = 0.0f;
    if(!transA && transB && (k % 4) == 0 && ((reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(b)) % 16) == 0) {
      const v4f* ar = reinterpret_cast<const v4f*>(a + (size_t)r * lda);
      const v4f* br = reinterpret_cast<const v4f*>(b + (size_t)q * ldb);
      for(int p = 0; p < k / 4; ++p) {
        const v4f av = ar[p], bv = br[p];
        s = fmaf(av.x, bv.x, s);
        s = fmaf(av.y, bv.y, s);
        s = fmaf(av.z, bv.z, s);
        s = fmaf(av.w, bv.w, s);
      }
    } else {
      for(int p = 0; p < k; ++p) {
        const float av = transA ? a[(size_t)p * lda + r] : a[(size_t)r * lda + p];
        const float bv = transB ? b[(size_t)q * ldb + p] : b[(size_t)p * ldb + q];
        s = fmaf(av, bv, s);
      }
    }
    c[q] = scalar * s;
  }
}

// The same products for matrices with many rows (encoder-size attention: m = n = 64 per head):
// a workgroup takes a 64 x 64 tile of one batch entry, K in chunks of 32 through LDS, a thread a
// 4 x 4 patch.  Every output is still summed over p = 0 .. k-1 in ascending order with one fma per
// term, so the result equals bdot_kernel's bit for bit.  A not transposed, k % 4 == 0 (TRANSB:
// B is [n x k]) or n % 4 == 0 (B is [k x n]), 16-byte aligned matrices.
template <bool TRANSB>
__global__ __launch_bounds__(256) void bdot_tile_kernel(const float* __restrict__ A, const float* __restrict__ B,
                                                        float* __restrict__ C, long long batchA,
                                                        long long batchB, int m, int n, int k, float scalar) {
  constexpr int KC = 32, LD = 64 + 4;
  __shared__ __attribute__((aligned(16))) float As[KC][LD];   // [p][row]
  __shared__ __attribute__((aligned(16))) float Bs[KC][LD];   // [p][col]
  const long long i = blockIdx.z;
  const float* a = A + (size_t)(i % batchA) * m * k;
  const float* b = B + (size_t)(i % batchB) * n * k;
  float* c = C + (size_t)i * m * n;
  const int r0 = blockIdx.y * 64, c0 = blockIdx.x * 64;
  const int tid = threadIdx.x, ty = tid / 16, tx = tid % 16;
  float acc[4][4];
#pragma unroll
  for(int y = 0; y < 4; ++y)
#pragma unroll
    for(int x = 0; x < 4; ++x) acc[y][x] = 0.0f;
  for(int p0 = 0; p0 < k; p0 += KC) {
    const int pc = min(KC, k - p0);   // a multiple of four
    __syncthreads();                  // the previous chunk has been read
    // rows of A (and of a transposed B): lane = row, so that the transposing LDS writes of a wave
    // fall into consecutive banks; four consecutive p per load
#pragma unroll
    for(int h = 0; h < 2; ++h) {
      const int idx = h * 256 + tid, row = idx % 64, p4 = idx / 64;   // p4 = 0 .. 7
      if(p4 * 4 < pc) {
        const v4f v = *reinterpret_cast<const v4f*>(a + (size_t)min(r0 + row, m - 1) * k + p0 + p4 * 4);
        As[p4 * 4][row] = v.x; As[p4 * 4 + 1][row] = v.y; As[p4 * 4 + 2][row] = v.z; As[p4 * 4 + 3][row] = v.w;
        if(TRANSB) {
          const v4f w = *reinterpret_cast<const v4f*>(b + (size_t)min(c0 + row, n - 1) * k + p0 + p4 * 4);
          Bs[p4 * 4][row] = w.x; Bs[p4 * 4 + 1][row] = w.y; Bs[p4 * 4 + 2][row] = w.z; Bs[p4 * 4 + 3][row] = w.w;
        }
      }
    }
    if(!TRANSB) {   // B is [k x n]: rows p, four consecutive columns per load
#pragma unroll
      for(int h = 0; h < 2; ++h) {
        const int idx = h * 256 + tid, col4 = idx % 16, p = idx / 16;   // p = 0 .. 31
        if(p < pc) {
          const int col = min(c0 + col4 * 4, n - 4);   // (n % 4 == 0; columns past n are never stored)
          *reinterpret_cast<v4f*>(&Bs[p][col4 * 4]) = *reinterpret_cast<const v4f*>(b + (size_t)(p0 + p) * n + col);
        }
      }
    }
    __syncthreads();
    for(int p = 0; p < pc; ++p) {
      const v4f av = *reinterpret_cast<const v4f*>(&As[p][ty * 4]);
      const v4f bv = *reinterpret_cast<const v4f*>(&Bs[p][tx * 4]);
      const float ar[4] = {av.x, av.y, av.z, av.w}, br[4] = {bv.x, bv.y, bv.z, bv.w};
#pragma unroll
      for(int y = 0; y < 4; ++y)
#pragma unroll
        for(int x = 0; x < 4; ++x) acc[y][x] = fmaf(ar[y], br[x], acc[y][x]);
    }
  }
#pragma unroll
  for(int y = 0; y < 4; ++y) {
    const int r = r0 + ty * 4 + y;
    if(r >= m) continue;
#pragma unroll
    for(int x = 0; x < 4; ++x) {
      const int q = c0 + tx * 4 + x;
      if(q < n) c[(size_t)r * n + q] = scalar * acc[y][x];
    }
  }
}

// ---------------------------------------------------------------- one-launch attention
// One wave per query row (entry i, row r): scores over the key positions (a lane per position,
// the query row and a key row are walked with the same fused multiply-adds, in the same order,
// as bdot_kernel walks them), softmax over them exactly as softmax_kernel<64> computes it, then
// the weighted sum of the value rows (a lane per output column, positions in ascending order,
// as bdot_kernel does).  The scores of a row live in LDS: `len` floats per wave.
// ANC (m == 1, dk == 64, one cache entry per query row, entry = hypothesis * heads + head): cached
// position p of hypothesis h is read from the entry of hypothesis anc[h * kv_cap + p] - the caches
// of a beam search stay where they were written and the table of ancestors says whose row a
// position of a hypothesis's history is; the newest position comes from k_new / v_new and goes into
// the hypothesis's own entry.
template <bool ANC>
__global__ __launch_bounds__(256) void attention_kernel(const float* __restrict__ Q, float* Kt, float* V,
                                                        const float* __restrict__ k_new,
                                                        const float* __restrict__ v_new,
                                                        const float* __restrict__ mask,
                                                        unsigned n_masks, unsigned rows_per_mask,
                                                        float* __restrict__ out, unsigned rows_total,
                                                        unsigned batchKV, int m, int len, int kv_cap, int dk,
                                                        float scale, float* __restrict__ absmax_out,
                                                        const uint32_t* __restrict__ anc, unsigned heads) {
  // kv_cap: positions a cache entry has room for (its stride, in rows of dk values); len of them are in use
  // (row counts are below 2^31, checked by the launcher: 32-bit divisions, a tenth of the
  // instructions of 64-bit ones, and this kernel is a chain of short phases)
  extern __shared__ __attribute__((aligned(16))) float att_lds[];
  const unsigned wr = blockIdx.x * 4 + threadIdx.x / 64;
  if(absmax_out && blockIdx.x == 0)   // slots past the last query row
    for(int sl = (int)rows_total + threadIdx.x; sl < kAbsmaxSlots; sl += 256) absmax_out[sl] = 0.0f;
  if(wr >= rows_total) return;   // whole waves leave; no workgroup barrier is used
  // per wave: the scores (rounded up to whole 16-byte units, so that the partial outputs behind
  // them are 16-byte aligned for the v4f stores), then 4 x 64 partial outputs
  const int len4 = (len + 3) & ~3;
  float* sc = att_lds + (threadIdx.x / 64) * (len4 + 256);
  float* part = sc + len4;
  const int lane = threadIdx.x % 64;
  // (no division in the usual cases: one position per entry, as many cache entries as entries)
  const unsigned i = m == 1 ? wr : wr / (unsigned)m;
  const unsigned entry = i < batchKV ? i : i % batchKV;
  const float* q = Q + (size_t)wr * dk;
  float* kb = Kt + (size_t)entry * kv_cap * dk;
  float* vb = V + (size_t)entry * kv_cap * dk;
  // Newest position (m == 1, one wave per cache entry): its key and value rows go into the cache
  // for the following steps; this step reads them from k_new / v_new directly.  Up to 64 values per
  // row they are requested here and stored at the end of the kernel (nothing in this call waits
  // for the copy, and a store right here would hold the wave for a memory round trip first).
  float k_app = 0.0f, v_app = 0.0f;
  const bool append_late = k_new && dk <= 64;
  if(append_late && lane < dk) {
    k_app = k_new[(size_t)wr * dk + lane];
    v_app = v_new[(size_t)wr * dk + lane];
  }
  if(k_new && !append_late) {
    for(int d = lane; d < dk; d += 64) {
      kb[(size_t)(len - 1) * dk + d] = k_new[(size_t)wr * dk + d];
      vb[(size_t)(len - 1) * dk + d] = v_new[(size_t)wr * dk + d];
    }
  }
  const float* k_last = k_new ? k_new + (size_t)wr * dk : kb + (size_t)(len - 1) * dk;
  const float* v_last = v_new ? v_new + (size_t)wr * dk : vb + (size_t)(len - 1) * dk;
  unsigned mask_row = 0;
  if(mask) {
    mask_row = rows_per_mask == 1 ? wr : wr / rows_per_mask;
    if(mask_row >= n_masks) mask_row %= n_masks;
  }
  const float* mk = mask ? mask + (size_t)mask_row * len : nullptr;
  const bool vec = (dk % 4) == 0 && ((reinterpret_cast<uintptr_t>(q) | reinterpret_cast<uintptr_t>(kb) |
                                     reinterpret_cast<uintptr_t>(k_last)) % 16) == 0;
  float mx = -__builtin_inff();
  float omax = 0.0f;   // max |out| of this query row
  const bool fast = vec && dk == 64 && ((reinterpret_cast<uintptr_t>(vb) | reinterpret_cast<uintptr_t>(v_last)) % 16) == 0;
  // The usual head size.  Sixteen lanes cover the 64 values of a key or value row with 16 bytes each
  // and the four groups of sixteen take four consecutive positions, so one load of the wave moves
  // 1 KB of contiguous cache.  Up to sixteen loads, 64 positions, are in flight at a time, and the
  // first 64 value rows are requested together with the first 64 key rows, so up to 64 positions
  // the call is one memory round trip.  Loads and products stop at the last group of four that
  // holds a position (the CU's address unit takes 16 clocks per load whether or not the row is a
  // duplicate, and eight waves share it).  The mask joins the scores afterwards, a lane per
  // position: one load for the first 64 positions, requested ahead of the key rows (inside the
  // score loop it was a dependent load per group of four).
  constexpr int kAttU = 16;
  v4f vr[kAttU];
  const int g = lane / 16, c = lane % 16;
  // Group of four positions U = (base + 4 u) / 4: this lane's position is 4 U + g, its row 4 U dk
  // floats behind the lane's first row; from group u_last on the lane's position is the last one
  // or past it, and it reads the last row (given separately: it may not be in the cache yet).
  const int u_last = (len + 2 - g) / 4;   // = ceil((len - 1 - g) / 4)
  auto load_rows = [&](const float* rows, const float* last, int base, v4f (&r)[kAttU]) __attribute__((always_inline)) {
    const float* first = rows + (size_t)g * dk + 4 * c;
    const float* last_c = last + 4 * c;
#pragma unroll
    for(int u = 0; u < kAttU; ++u) {
      if(base + 4 * u < len) {   // (the same for the whole wave)
        const int U = base / 4 + u;
        const float* p = U >= u_last ? last_c : first + (size_t)U * 4 * dk;
        r[u] = *reinterpret_cast<const v4f*>(p);
      } else if(base + 4 * (u & ~3) < len) {   // (read with its group of sixteen positions below)
        r[u] = v4f{0.0f, 0.0f, 0.0f, 0.0f};
      }
    }
  };
  // ANC: the entry a cached position is read from differs from position to position.  The lane's
  // (up to sixteen) ancestors of a batch of 64 positions are requested together, one round trip
  // ahead of the key and value rows.
  unsigned au[ANC ? kAttU : 1];
  const unsigned hyp = ANC ? wr / heads : 0u, head = ANC ? wr % heads : 0u;
  auto load_ancestors = [&](int base) __attribute__((always_inline)) {
    if(ANC) {
      const uint32_t* row = anc + (size_t)hyp * kv_cap;
      const unsigned n_hyp = rows_total / heads;
#pragma unroll
      for(int u = 0; u < kAttU; ++u)
        if(base + 4 * u < len) au[u] = min(row[min(base + 4 * u + g, len - 1)], n_hyp - 1u);
    }
  };
  auto load_rows_anc = [&](const float* tensor, const float* last, int base, v4f (&r)[kAttU]) __attribute__((always_inline)) {
    const float* last_c = last + 4 * c;
#pragma unroll
    for(int u = 0; u < kAttU; ++u) {
      if(base + 4 * u < len) {   // (the same for the whole wave)
        const int U = base / 4 + u;
        const float* p = U >= u_last ? last_c
                                     : tensor + ((size_t)(au[ANC ? u : 0] * heads + head) * kv_cap + (size_t)(4 * U + g)) * dk + 4 * c;
        r[u] = *reinterpret_cast<const v4f*>(p);
      } else if(base + 4 * (u & ~3) < len) {
        r[u] = v4f{0.0f, 0.0f, 0.0f, 0.0f};
      }
    }
  };
  auto load_k = [&](int base, v4f (&r)[kAttU]) __attribute__((always_inline)) {
    if(ANC) load_rows_anc(Kt, k_last, base, r);
    else load_rows(kb, k_last, base, r);
  };
  auto load_v = [&](int base, v4f (&r)[kAttU]) __attribute__((always_inline)) {
    if(ANC) load_rows_anc(V, v_last, base, r);
    else load_rows(vb, v_last, base, r);
  };
  if(fast) {
    float mk0 = 0.0f;
    if(mk) mk0 = mk[min(lane, len - 1)];
    const v4f q4 = reinterpret_cast<const v4f*>(q)[c];
    v4f kr[kAttU];
    load_ancestors(0);
    load_k(0, kr);
    load_v(0, vr);
    // (sixteen positions at a time without a branch between them: the four products and the four
    // exchange steps of a group of four positions depend on one another, and only independent
    // groups side by side keep the wave issuing; rows that were not loaded are zeros here and their
    // results are dropped)
    for(int base = 0;;) {
#pragma unroll
      for(int u0 = 0; u0 < kAttU; u0 += 4) {
        if(base + 4 * u0 < len) {
          float s[4];
#pragma unroll
          for(int u = u0; u < u0 + 4; ++u) {
            float t = q4.x * kr[u].x;
            t = fmaf(q4.y, kr[u].y, t);
            t = fmaf(q4.z, kr[u].z, t);
            s[u - u0] = fmaf(q4.w, kr[u].w, t);
          }
#pragma unroll
          for(int u = 0; u < 4; ++u) s[u] = row16_sum(s[u]);
#pragma unroll
          for(int u = u0; u < u0 + 4; ++u) {
            const int pos = base + 4 * u + g;
            if(c == 0 && pos < len) sc[pos] = scale * s[u - u0];
          }
        }
      }
      base += 4 * kAttU;
      if(base >= len) break;
      load_ancestors(base);
      load_k(base, kr);
    }
    for(int pos = lane; pos < len; pos += 64) {
      float z = sc[pos];
      if(mk) {
        z = z + (pos < 64 ? mk0 : mk[pos]);
        sc[pos] = z;
      }
      mx = fmaxf(mx, z);
    }
  }
  for(int pos = lane; pos < len && !fast; pos += 64) {
    float s = 0.0f;
    const float* krow = pos == len - 1 ? k_last : kb + (size_t)pos * dk;
    if(vec && dk == 64) {   // the usual head size: all sixteen loads of the key row in flight at once
      const v4f* ar = reinterpret_cast<const v4f*>(q);
      const v4f* br = reinterpret_cast<const v4f*>(krow);
      v4f kr[16];
#pragma unroll
      for(int p = 0; p < 16; ++p) kr[p] = br[p];
#pragma unroll
      for(int p = 0; p < 16; ++p) {
        const v4f av = ar[p];
        s = fmaf(av.x, kr[p].x, s);
        s = fmaf(av.y, kr[p].y, s);
        s = fmaf(av.z, kr[p].z, s);
        s = fmaf(av.w, kr[p].w, s);
      }
    } else if(vec) {
      const v4f* ar = reinterpret_cast<const v4f*>(q);
      const v4f* br = reinterpret_cast<const v4f*>(krow);
      for(int p = 0; p < dk / 4; ++p) {
        const v4f av = ar[p], bv = br[p];
        s = fmaf(av.x, bv.x, s);
        s = fmaf(av.y, bv.y, s);
        s = fmaf(av.z, bv.z, s);
        s = fmaf(av.w, bv.w, s);
      }
    } else {
      for(int p = 0; p < dk; ++p) s = fmaf(q[p], krow[p], s);
    }
    float z = scale * s;
    if(mk) z = z + mk[pos];
    sc[pos] = z;
    mx = z > mx ? z : mx;
  }
  mx = wave_maxf(mx);
  float sum = 0.0f;
  float e_first = 0.0f;   // exp of this lane's first position, kept for the division below
  for(int pos = lane; pos < len; pos += 64) {
    const float e = expf(sc[pos] - mx);
    if(pos == lane) e_first = e;
    sum += e;
  }
  sum = wave_sum(sum);
  for(int pos = lane; pos < len; pos += 64) sc[pos] = (pos == lane ? e_first : expf(sc[pos] - mx)) / sum;
  // (a wave's LDS writes are visible to its own later reads: same wave, program order)
  if(fast) {
    v4f o4 = v4f{0.0f, 0.0f, 0.0f, 0.0f};
    for(int base = 0; base < len; base += 4 * kAttU) {
      if(base > 0) {
        load_ancestors(base);
        load_v(base, vr);
      }
#pragma unroll
      for(int u0 = 0; u0 < kAttU; u0 += 4) {
        if(base + 4 * u0 < len) {
          // the four weights first (reads inside this wave's score area: a position past the row
          // reads a stale value there, which is replaced by zero)
          float w[4];
#pragma unroll
          for(int u = u0; u < u0 + 4; ++u) w[u - u0] = sc[min(base + 4 * u + g, len4 + 255)];
#pragma unroll
          for(int u = u0; u < u0 + 4; ++u) {
            const float wu = base + 4 * u + g < len ? w[u - u0] : 0.0f;
            o4.x = fmaf(wu, vr[u].x, o4.x);
            o4.y = fmaf(wu, vr[u].y, o4.y);
            o4.z = fmaf(wu, vr[u].z, o4.z);
            o4.w = fmaf(wu, vr[u].w, o4.w);
          }
        }
      }
    }
    reinterpret_cast<v4f*>(part)[g * 16 + c] = o4;   // partial sums of the positions g, g + 4, ...
    const float o = ((part[lane] + part[64 + lane]) + part[128 + lane]) + part[192 + lane];
    out[(size_t)wr * dk + lane] = o;
    omax = fabsf(o);
  }
  for(int d = lane; d < dk && !fast; d += 64) {
    float o = 0.0f;
    int pos = 0;
    for(; pos + 8 <= len; pos += 8) {   // eight value loads in flight, same summation order
      float vr[8];
#pragma unroll
      for(int u = 0; u < 8; ++u) vr[u] = pos + u == len - 1 ? v_last[d] : vb[(size_t)(pos + u) * dk + d];
#pragma unroll
      for(int u = 0; u < 8; ++u) o = fmaf(sc[pos + u], vr[u], o);
    }
    for(; pos < len; ++pos) o = fmaf(sc[pos], pos == len - 1 ? v_last[d] : vb[(size_t)pos * dk + d], o);
    out[(size_t)wr * dk + d] = 1.0f * o;
    omax = fmaxf(omax, fabsf(1.0f * o));
  }
  if(absmax_out) {   // slot = query row
    omax = wave_maxf(omax);
    if(lane == 0) absmax_out[wr] = omax;
  }
  if(append_late && lane < dk) {
    kb[(size_t)(len - 1) * dk + lane] = k_app;
    vb[(size_t)(len - 1) * dk + lane] = v_app;
  }
}

// ---------------------------------------------------------------- projection + attention in one launch
// The projections in front of an attention and the attention itself for one new target position
// (reference src/models/transformer.h:279-348: q = affine(input, Wq, bq), for self-attention also
// k, v = affine(input, Wk / Wv, ..), split into heads, then Attention()): a workgroup owns the 64
// columns of ONE head in every projection for R rows of the input, so it has everything that
// head's attention needs for its rows and runs it before it exits - one launch instead of two, and
// q (k, v) never travel through memory.
//   1. the abs-max of the input comes from the slots its producer left (or an abs-max launch);
//   2. the workgroup quantizes its R rows of the float32 input into LDS in matrix-operand order
//      (exactly the quantize-on-stage form of the decode GEMM: same quantizer, same layout); the
//      workgroups of head 0 also write them out, so the prepareA node's tensor still exists;
//   3. eight waves = 2 column tiles x 4 ranges of K; every wave requests its weights of all
//      projections at kernel start (up to 24 loads of 1 KB in flight), multiplies, and drops its
//      partial tiles into LDS;
//   4. the partial tiles are added (exact), dequantized with bias exactly like the GEMM epilogues
//      (two roundings) and kept in LDS as q[R][64] (k_new, v_new); k_new and v_new also go into
//      the caches at position len - 1, and all three into proj_out where a caller asks for them;
//   5. wave w runs the attention of row w: the code of attention_kernel's 64-wide path, operation
//      for operation, with q and the newest key/value row read from LDS.
// Where the caches are complete and shared - the encoder's keys and values, which every hypothesis
// of a sentence attends to (row m reads sentence m % sentences) - a workgroup takes hypotheses of
// the same one or two sentences instead of eight consecutive rows (ProjRowPlan in
// operand_addressing.h: as many hypotheses of a sentence as a workgroup has rows for, the rest in
// further workgroups; rows without a hypothesis idle), reads these sentences' keys and
// values once (asked for as soon as the abs-max is known, stored to LDS in step 4) and its waves
// take them from LDS: a quarter of the bytes through the CU's memory path with four hypotheses a
// sentence (60 positions: 60 KB instead of 240 KB per workgroup).
// Requirements (checked by the launcher): head size 64, K % 128 == 0, K <= 1024, len <= 512.
// Measured (transformer-big step, 128 rows, 16 heads): 13.5 us against 8.2 + 8.4 us for q, k, v and
// the self-attention over 21 positions, 13.9 against 5.3 + 8.4 us for Wq and the context attention over
// 60 positions with every wave reading its own keys and values; staging the shared ones takes the
// whole step from 0.437 to 0.425 ms.  Clocks read inside the kernel (weights and caches of 24
// layers in rotation, so that they come from HBM): the launch is bound by what a CU can fetch,
// about 15 bytes per clock when most of it misses L2 - the self-attention form's 310 KB per
// workgroup (192 KB of weights, 32 KB of input, 86 KB of keys and values) in 26 000 clocks, the
// context form's 156 KB (staged) in 17 700.  Tried and dropped, each without a gain in the step:
// asking for a row's keys and values at kernel start (loads into a scratch word of LDS, by the
// multiplying waves or by two more waves), or into registers once the abs-max is known in the
// self-attention form - the attention then waits less and the quantization more, for the same
// bytes; barriers that put every wave's small requests in front of any wave's large ones; the
// workgroups of a head starting at different sub-steps of K, so that they would not all miss L2 on
// the same lines of the weights at the same time (+5 us per step).
constexpr int kProjThreads = 512, kProjMaxK = 1024, kProjMaxLen = 512;
// keys and values shared by the rows of a workgroup are staged in LDS up to this many positions
constexpr int kProjStageLen = 96;
constexpr int kProjMaxLds = 160 * 1024 - 256;   // dynamic LDS of a workgroup (a few bytes are static)

struct ProjAttentionArgs {
  const float* A;           // [M, K] float32
  int8_t* aq_out;           // [M, K] int8 + quantMult tail
  const float* partials;    // abs-max slots of A
  int n_partials;
  const int8_t* Bq[3];      // prepared weights [K, heads * 64]
  const float* bias[3];     // or null
  float* proj_out[3];       // [M, heads * 64] or null: the projections themselves, for callers that want them
  int M, K, heads;
  float* k_cache;           // [batchKV, kv_cap, 64]
  float* v_cache;
  unsigned batchKV;
  int len, kv_cap;
  const float* mask;        // [n_masks, len] or null, one row per (query row / heads) % n_masks
  unsigned n_masks;
  float att_scale;
  float* out;               // [M * heads, 64]
  float* absmax_out;        // slots or null
  // Which input rows a workgroup takes (ProjRowPlan).  share_shift < 0: eight consecutive ones.
  // Otherwise the caches hold `share_nb` sentences that share_hyps hypotheses each attend to (row m
  // reads sentence m % share_nb), and a workgroup takes share_per of them for 1 << share_shift
  // neighbouring sentences, so that the waves that read the same keys and values sit on one CU.
  int share_shift, share_nb, share_hyps, share_per;
  // With it (and sentences two or one to a workgroup, len <= kProjStageLen): the keys and values of
  // the workgroup's sentences are read once, into LDS, and every hypothesis' wave takes them from there.
  int stage_kv;
};

// Entry g of one of the argument arrays, g differing between the threads: selected from the three
// values in scalar registers.  (Indexed by a thread-dependent g the compiler reads the entry from
// the kernel-argument memory with a vector load, and the wait for it - loads complete in order -
// is a wait for every load the thread has issued before: the weights.)
template <typename T>
__device__ __forceinline__ T pick3(const T (&a)[3], int g) {
  const T a0 = a[0], a1 = a[1], a2 = a[2];   // (values: a conditional between the elements themselves selects an address)
  return g == 0 ? a0 : (g == 1 ? a1 : a2);
}

// the row permutation of the staged activations (gemm_stream32_kernel.h: stream32_row_key)
__device__ __forceinline__ int proj_row_key(int c16) { return (c16 ^ (c16 >> 2)) & 7; }

// One query row of 64 values by one wave: attention_kernel's path for that head size (sixteen lanes
// cover a key or value row, four consecutive positions per load, up to 64 positions in flight), the
// same operations in the same order, so the result has the same bits.  q, k_last, v_last may lie
// in LDS.  sc: len4 floats of this wave, part: 256 floats behind them.  Returns |out| of this lane.
// LAST_IN_ROWS: k_last and v_last are row len - 1 of kb and vb (one address computation for all rows).
template <bool LAST_IN_ROWS = false>
__device__ __forceinline__ float attention_row64(const float* q, const float* kb, const float* vb, const float* k_last,
                                                 const float* v_last, const float* mk, float mk0, int len, float scale, float* sc,
                                                 float* part, float* out_row, int lane) {
  constexpr int kAttU = 16, dk = 64;
  const int len4 = (len + 3) & ~3;
  const int g = lane / 16, c = lane % 16;
  const int u_last = (len + 2 - g) / 4;
  auto load_rows = [&](const float* rows, const float* last, int base, v4f (&r)[kAttU]) __attribute__((always_inline)) {
    const float* first = rows + (size_t)g * dk + 4 * c;
    const float* last_c = last + 4 * c;
#pragma unroll
    for(int u = 0; u < kAttU; ++u) {
      if(base + 4 * u < len) {
        const int U = base / 4 + u;
        if constexpr(LAST_IN_ROWS) r[u] = *reinterpret_cast<const v4f*>(rows + (size_t)min(4 * U + g, len - 1) * dk + 4 * c);
        else if(U >= u_last) r[u] = *reinterpret_cast<const v4f*>(last_c);
        else r[u] = *reinterpret_cast<const v4f*>(first + (size_t)U * 4 * dk);
      } else if(base + 4 * (u & ~3) < len) {
        r[u] = v4f{0.0f, 0.0f, 0.0f, 0.0f};
      }
    }
  };
  const v4f q4 = reinterpret_cast<const v4f*>(q)[c];
  v4f kr[kAttU], vr[kAttU];
  load_rows(kb, k_last, 0, kr);
  load_rows(vb, v_last, 0, vr);
  for(int base = 0;;) {
#pragma unroll
    for(int u0 = 0; u0 < kAttU; u0 += 4) {
      if(base + 4 * u0 < len) {
        float s[4];
#pragma unroll
        for(int u = u0; u < u0 + 4; ++u) {
          float t = q4.x * kr[u].x;
          t = fmaf(q4.y, kr[u].y, t);
          t = fmaf(q4.z, kr[u].z, t);
          s[u - u0] = fmaf(q4.w, kr[u].w, t);
        }
#pragma unroll
        for(int u = 0; u < 4; ++u) s[u] = row16_sum(s[u]);
#pragma unroll
        for(int u = u0; u < u0 + 4; ++u) {
          const int pos = base + 4 * u + g;
          if(c == 0 && pos < len) sc[pos] = scale * s[u - u0];
        }
      }
    }
    base += 4 * kAttU;
    if(base >= len) break;
    load_rows(kb, k_last, base, kr);
  }
  float mx = -__builtin_inff();
  for(int pos = lane; pos < len; pos += 64) {
    float z = sc[pos];
    if(mk) {
      z = z + (pos < 64 ? mk0 : mk[pos]);
      sc[pos] = z;
    }
    mx = fmaxf(mx, z);
  }
  mx = wave_maxf(mx);
  float sum = 0.0f;
  float e_first = 0.0f;
  for(int pos = lane; pos < len; pos += 64) {
    const float e = expf(sc[pos] - mx);
    if(pos == lane) e_first = e;
    sum += e;
  }
  sum = wave_sum(sum);
  for(int pos = lane; pos < len; pos += 64) sc[pos] = (pos == lane ? e_first : expf(sc[pos] - mx)) / sum;
  v4f o4 = v4f{0.0f, 0.0f, 0.0f, 0.0f};
  for(int base = 0; base < len; base += 4 * kAttU) {
    if(base > 0) load_rows(vb, v_last, base, vr);
#pragma unroll
    for(int u0 = 0; u0 < kAttU; u0 += 4) {
      if(base + 4 * u0 < len) {
        float w[4];
#pragma unroll
        for(int u = u0; u < u0 + 4; ++u) w[u - u0] = sc[min(base + 4 * u + g, len4 + 255)];
#pragma unroll
        for(int u = u0; u < u0 + 4; ++u) {
          const float wu = base + 4 * u + g < len ? w[u - u0] : 0.0f;
          o4.x = fmaf(wu, vr[u].x, o4.x);
          o4.y = fmaf(wu, vr[u].y, o4.y);
          o4.z = fmaf(wu, vr[u].z, o4.z);
          o4.w = fmaf(wu, vr[u].w, o4.w);
        }
      }
    }
  }
  reinterpret_cast<v4f*>(part)[g * 16 + c] = o4;
  const float o = ((part[lane] + part[64 + lane]) + part[128 + lane]) + part[192 + lane];
  out_row[lane] = o;
  return fabsf(o);
}

// Attention over caches that several query rows share (the encoder's keys and values: query row
// r reads cache entry r % batchKV, so rows e, e + batchKV, e + 2 batchKV, .. - the hypotheses of a
// sentence, for one head - read the same entry).  Workgroup (e, y) takes rows e + (4 y + w) batchKV
// for its waves w = 0 .. 3, reads entry e's keys and values once (sixteen threads per position,
// PASSES passes of sixteen positions; positions past the end repeat the last one) into LDS, and each
// wave then runs attention_row64 on them: the operations of attention_kernel's 64-wide path in the
// same order, so the same bits, with a quarter (for four hypotheses) of the bytes through the
// CU's memory path and out of L2.  One position per query row, head size 64, len <= 16 * PASSES.
constexpr int kSharedAttLen = 96;
template <int PASSES>
__global__ __launch_bounds__(256) void attention_shared_kernel(const float* __restrict__ Q, const float* __restrict__ Kt,
                                                               const float* __restrict__ V, const float* __restrict__ mask,
                                                               unsigned n_masks, unsigned rows_per_mask,
                                                               float* __restrict__ out, unsigned rows_total,
                                                               unsigned batchKV, int len, int kv_cap, float scale,
                                                               float* __restrict__ absmax_out) {
  static_assert(PASSES * 16 <= kSharedAttLen, "sixteen positions per pass");
  extern __shared__ __attribute__((aligned(16))) float satt_lds[];
  const int tid = threadIdx.x, wave = tid / 64, lane = tid % 64;
  const unsigned entry = blockIdx.x;
  const unsigned wr = entry + (blockIdx.y * 4u + (unsigned)wave) * batchKV;
  const bool valid = wr < rows_total;
  if(absmax_out && blockIdx.x == 0 && blockIdx.y == 0)   // slots past the last query row
    for(int sl = (int)rows_total + tid; sl < kAbsmaxSlots; sl += 256) absmax_out[sl] = 0.0f;
  // everything is requested before anything is used: keys, values, the mask value of this lane
  v4f kst[PASSES], vst[PASSES];
  {
    const float* ksrc = Kt + (size_t)entry * kv_cap * 64 + (tid % 16) * 4;
    const float* vsrc = V + (size_t)entry * kv_cap * 64 + (tid % 16) * 4;
#pragma unroll
    for(int j = 0; j < PASSES; ++j) kst[j] = *reinterpret_cast<const v4f*>(ksrc + (size_t)min(tid / 16 + 16 * j, len - 1) * 64);
#pragma unroll
    for(int j = 0; j < PASSES; ++j) vst[j] = *reinterpret_cast<const v4f*>(vsrc + (size_t)min(tid / 16 + 16 * j, len - 1) * 64);
  }
  const float* mk = nullptr;
  if(mask && valid) {
    unsigned mask_row = rows_per_mask == 1 ? wr : wr / rows_per_mask;
    if(mask_row >= n_masks) mask_row %= n_masks;
    mk = mask + (size_t)mask_row * len;
  }
  const float mk0 = *(mk ? mk + min(lane, len - 1) : Q);   // (the latter not looked at)
  const int len4 = (len + 3) & ~3;
  float* ks = satt_lds;                       // [len][64]
  float* vs = ks + (size_t)len * 64;          // [len][64]
  float* sc = vs + (size_t)len * 64 + wave * (len4 + 256);   // per wave: scores + 256 partial outputs
#pragma unroll
  for(int j = 0; j < PASSES; ++j) {
    const int pos = tid / 16 + 16 * j;
    if(pos < len) {
      *reinterpret_cast<v4f*>(ks + (size_t)pos * 64 + (tid % 16) * 4) = kst[j];
      *reinterpret_cast<v4f*>(vs + (size_t)pos * 64 + (tid % 16) * 4) = vst[j];
    }
  }
  __syncthreads();
  if(valid) {   // (whole waves)
    float omax = attention_row64<true>(Q + (size_t)wr * 64, ks, vs, ks + (size_t)(len - 1) * 64, vs + (size_t)(len - 1) * 64, mk,
                                       mk0, len, scale, sc, sc + len4, out + (size_t)wr * 64, lane);
    if(absmax_out) {
      omax = wave_maxf(omax);
      if(lane == 0) absmax_out[wr] = omax;
    }
  }
}

// NPROJ: 3 (q, k_new, v_new: self-attention, the new key/value row is appended to the caches) or
// 1 (q only: attention over caches that are complete, e.g. the encoder's).  R: input rows per
// workgroup, 8 (a wave per row in the attention).
template <int NPROJ, int R, int SEGS, int PASSES>
__global__ __launch_bounds__(kProjThreads) void proj_attention_kernel(ProjAttentionArgs p) {
  static_assert(R == 8, "one wave per row in the attention");
  constexpr bool STAGED = SEGS > 0;
  static_assert(!STAGED || NPROJ == 1, "keys and values are shared only where the caches are complete");
  static_assert(SEGS == 0 || SEGS == 2 || SEGS == 4, "keys and values of one or two sentences");
  static_assert(PASSES * 32 <= kProjStageLen, "32 positions per pass");
  typedef int v16i_p __attribute__((ext_vector_type(16)));
  extern __shared__ __attribute__((aligned(16))) int8_t plds[];
  __shared__ float red[kProjThreads / 64];
  const int tid = threadIdx.x, wave = tid / 64, lane = tid % 64;
  const int wn = wave % 2, kw = wave / 2, li = lane % 32, lg = lane / 32;
  const int h = blockIdx.x;
  // input row r of this workgroup (rows past the end: M or more)
  const int sent_base = p.share_shift < 0 ? 0 : proj_first_sentence(p.share_shift, p.share_nb, (int)blockIdx.y);
  auto row_of = [&](int r) -> int { return proj_row_of(p.share_shift, p.share_nb, p.share_hyps, p.share_per, (int)blockIdx.y, r); };
  const int K = p.K, M = p.M, S = K / 32, PW = S / 4, N = p.heads * 64;
  int8_t* a_lds = plds;                                   // 32 rows x K bytes, operand order
  int8_t* part_lds = a_lds + 32 * K;                      // NPROJ x 2 x 4 partial tiles of R rows x 128 bytes
  float* proj_lds = reinterpret_cast<float*>(part_lds + NPROJ * 8 * R * 128);   // [NPROJ][R][64]
  float* att_lds = proj_lds + NPROJ * R * 64;             // per wave: scores + 256 partial outputs
  const int len4s = (p.len + 3) & ~3;
  float* kv_lds = att_lds + R * (len4s + 256);            // staged keys and values: [sentence][k, v][len][64]

  // ---- everything this workgroup will need is requested now, in the order of its use (a wave's
  //      loads complete in the order of their issue): abs-max slots, the input rows, weights, the
  //      mask value, the quantization multipliers of the weights, bias ----
  float pm[kAbsmaxSlots / kProjThreads];
#pragma unroll
  for(int i = 0; i < kAbsmaxSlots / kProjThreads; ++i) pm[i] = p.partials[min(tid + i * kProjThreads, p.n_partials - 1)];
  // a quad of lanes takes four consecutive 16-value groups of one row: 64 contiguous bytes per load
  const int grp = (tid / 4) * 4, qlane = tid % 4;
  const int r_in = grp / (2 * S), c16 = grp % (2 * S);
  const bool has_in = r_in < R;
  v4f in[4];
  {
    const int m = min(row_of(min(r_in, R - 1)), M - 1);
    const float* src = p.A + (size_t)m * (size_t)K + (size_t)c16 * 16 + qlane * 4;
#pragma unroll
    for(int e = 0; e < 4; ++e) in[e] = *reinterpret_cast<const v4f*>(src + e * 16);
  }
  v4i w[NPROJ][8];
  const int ncol = h * 64 + wn * 32 + li;
  // (asked for in the order the multiplication takes them: sub-step by sub-step, all projections)
#pragma unroll
  for(int pp = 0; pp < 8; ++pp) {
    const size_t at = stream32_lane_offset(ncol, lg) + (size_t)stream32_clamped_substep(kw * PW + pp, S) * 32u * (size_t)N;
#pragma unroll
    for(int g = 0; g < NPROJ; ++g) w[g][pp] = load16(p.Bq[g] + at);
  }
  // keys and values of the workgroup's sentences: sixteen threads per position, 32 positions per pass
  constexpr int kStageSegs = STAGED ? SEGS : 1, kStagePasses = STAGED ? PASSES : 1;
  v4f stage[kStageSegs][kStagePasses];
  // the mask value of this wave's row for position `lane`
  const int m_wave = row_of(min(wave, R - 1));
  const float* mk = nullptr;
  if(p.mask && m_wave < M) {
    unsigned mask_row = (unsigned)m_wave;
    if(mask_row >= p.n_masks) mask_row %= p.n_masks;
    mk = p.mask + (size_t)mask_row * p.len;
  }
  const float mk0 = *(mk ? mk + min(lane, p.len - 1) : p.partials);   // (the latter not looked at)
  float bqm[NPROJ];
#pragma unroll
  for(int g = 0; g < NPROJ; ++g) bqm[g] = tail_quant_mult(p.Bq[g], (size_t)K * (size_t)N);
  // the (up to two) pieces of four outputs this thread finishes in step 4, and their bias
  constexpr int kItems = NPROJ * 2 * R * 8;
  v4f bias4[2];
#pragma unroll
  for(int it = 0; it < 2; ++it) {
    const int item = min(it * kProjThreads + tid, kItems - 1);
    const int tg = item / (R * 8), pc = item % 8;
    const float* b = pick3(p.bias, tg / 2);
    // (no bias: sixteen bytes of the weights instead, not looked at)
    bias4[it] = *reinterpret_cast<const v4f*>(b ? b + h * 64 + (tg % 2) * 32 + pc * 4 : reinterpret_cast<const float*>(p.Bq[0]));
  }

  // ---- 1, 2: abs-max, quantize into LDS ----
  float amax = 0.0f;
#pragma unroll
  for(int i = 0; i < kAbsmaxSlots / kProjThreads; ++i) amax = fmaxf(amax, pm[i]);
  amax = block_max(amax, red);
  // The keys and values are asked for last - a wave's loads complete in the order of their issue,
  // and they are needed last - and only now: in front of the abs-max values they would delay them.
  // No branches around them (positions past the end repeat the last one; the number of loads is
  // the kernel's), so that the waits in front of the earlier loads' uses count exactly.
  if constexpr(STAGED) {
#pragma unroll
    for(int seg = 0; seg < SEGS; ++seg) {
      const unsigned entry = (unsigned)(sent_base + (seg >> 1)) * (unsigned)p.heads + (unsigned)h;
      const float* src = ((seg & 1) ? p.v_cache : p.k_cache) + (size_t)entry * p.kv_cap * 64 + (tid % 16) * 4;
#pragma unroll
      for(int j = 0; j < PASSES; ++j)
        stage[seg][j] = *reinterpret_cast<const v4f*>(src + (size_t)min(tid / 16 + 32 * j, p.len - 1) * 64);
    }
  }
  const float aqm = quant_mult_from_maxabs(amax);
  const bool finite = aqm < __builtin_inff();
  float unquant[NPROJ];
#pragma unroll
  for(int g = 0; g < NPROJ; ++g) unquant[g] = unquant_mult(aqm, bqm[g], 1.0f);
  if(has_in) {
    uint32_t q[4];
#pragma unroll
    for(int e = 0; e < 4; ++e) q[e] = finite ? quantize_pack4_finite(in[e], aqm) : quantize_pack4(in[e], aqm);
    const int slot0 = (c16 / 2) * 64, x = r_in ^ proj_row_key(c16);
    const int m = row_of(min(r_in, R - 1));
#pragma unroll
    for(int e = 0; e < 4; ++e) {
      const int sw = slot0 + (e / 2) * 64 + (e % 2) * 32 + (x ^ e);
      *reinterpret_cast<uint32_t*>(a_lds + sw * 16 + qlane * 4) = q[e];
      if(p.aq_out && h == 0 && m < M)
        *reinterpret_cast<uint32_t*>(p.aq_out + (size_t)m * (size_t)K + (size_t)(c16 + e) * 16 + qlane * 4) = q[e];
    }
  }
  if(p.aq_out && h == 0 && blockIdx.y == 0 && tid == 0) *reinterpret_cast<float*>(p.aq_out + (size_t)M * K) = aqm;
  __syncthreads();

  // ---- 3: multiply (rows R .. 31 of the operand are whatever LDS held: they only feed output rows
  //      that are never looked at) ----
  v16i_p acc[NPROJ];
#pragma unroll
  for(int g = 0; g < NPROJ; ++g)
#pragma unroll
    for(int v = 0; v < 16; ++v) acc[g][v] = 0;
#pragma unroll
  for(int pp = 0; pp < 8; ++pp) {
    if(pp < PW) {   // (the same for the whole workgroup)
      const int s = kw * PW + pp;
      const v4i a = *reinterpret_cast<const v4i*>(a_lds + s * 1024 + (lg * 32 + (li ^ proj_row_key(2 * s + lg))) * 16);
#pragma unroll
      for(int g = 0; g < NPROJ; ++g) acc[g] = __builtin_amdgcn_mfma_i32_32x32x32_i8(w[g][pp], a, acc[g], 0, 0, 0);
    }
  }
  // accumulator value v of lane (li, lg): input row li, column 8 * (v / 4) + 4 * lg + v % 4 of the
  // wave's 32; a tile row is 128 bytes, its eight 16-byte pieces XOR-permuted by the row number
  if(li < R) {
#pragma unroll
    for(int g = 0; g < NPROJ; ++g) {
      int8_t* mine = part_lds + ((g * 2 + wn) * 4 + kw) * (R * 128);
#pragma unroll
      for(int q = 0; q < 4; ++q)
        *reinterpret_cast<v4i*>(mine + li * 128 + (((2 * q + lg) ^ (li & 7)) * 16)) =
            v4i{acc[g][4 * q], acc[g][4 * q + 1], acc[g][4 * q + 2], acc[g][4 * q + 3]};
    }
  }
  __syncthreads();

  // ---- 4: add the four K ranges, dequantize, keep in LDS, append k_new / v_new to the caches ----
#pragma unroll
  for(int it = 0; it < 2; ++it) {
    const int item = it * kProjThreads + tid;
    if(item < kItems) {
      const int tg = item / (R * 8), r = (item / 8) % R, pc = item % 8;
      const int g = tg / 2, col = (tg % 2) * 32 + pc * 4;
      const int8_t* src = part_lds + (tg * 4) * (R * 128) + r * 128 + ((pc ^ (r & 7)) * 16);
      v4i sum = *reinterpret_cast<const v4i*>(src);
#pragma unroll
      for(int t = 1; t < 4; ++t) sum += *reinterpret_cast<const v4i*>(src + t * (R * 128));
      float uq = unquant[0];
      if constexpr(NPROJ == 3) uq = g == 0 ? unquant[0] : (g == 1 ? unquant[1] : unquant[2]);
      const bool has_bias = pick3(p.bias, g) != nullptr;
      const float b[4] = {bias4[it].x, bias4[it].y, bias4[it].z, bias4[it].w};
      float y[4];
#pragma unroll
      for(int e = 0; e < 4; ++e) {
        y[e] = (float)sum[e] * uq;
        if(has_bias) y[e] = y[e] + b[e];
      }
      const v4f yv = v4f{y[0], y[1], y[2], y[3]};
      *reinterpret_cast<v4f*>(proj_lds + (g * R + r) * 64 + col) = yv;
      const int m = row_of(r);
      if(m < M) {
        float* const po = pick3(p.proj_out, g);
        if(po) *reinterpret_cast<v4f*>(po + (size_t)m * (size_t)N + h * 64 + col) = yv;
        if(NPROJ == 3 && g > 0) {
          float* cache = g == 1 ? p.k_cache : p.v_cache;
          const size_t entry = (size_t)m * (size_t)p.heads + (size_t)h;
          *reinterpret_cast<v4f*>(cache + (entry * (size_t)p.kv_cap + (size_t)(p.len - 1)) * 64 + col) = yv;
        }
      }
    }
  }
  if constexpr(STAGED) {
#pragma unroll
    for(int seg = 0; seg < SEGS; ++seg) {
#pragma unroll
      for(int j = 0; j < PASSES; ++j) {
        const int pos = tid / 16 + 32 * j;
        if(pos < p.len) *reinterpret_cast<v4f*>(kv_lds + ((size_t)(seg * p.len + pos) * 64 + (tid % 16) * 4)) = stage[seg][j];
      }
    }
  }
  __syncthreads();

  // ---- 5: the attention of row `wave` ----
  const int rows_total = M * p.heads;
  if(p.absmax_out && blockIdx.x == 0 && blockIdx.y == 0)   // slots past the last query row
    for(int sl = rows_total + tid; sl < kAbsmaxSlots; sl += kProjThreads) p.absmax_out[sl] = 0.0f;
  const int m = m_wave;
  if(wave < R && m < M) {   // (whole waves)
    const unsigned wr = (unsigned)m * (unsigned)p.heads + (unsigned)h;
    const unsigned entry = wr < p.batchKV ? wr : wr % p.batchKV;
    const float* kb = p.k_cache + (size_t)entry * p.kv_cap * 64;
    const float* vb = p.v_cache + (size_t)entry * p.kv_cap * 64;
    const float* q = proj_lds + wave * 64;
    const float* k_last = NPROJ == 3 ? proj_lds + (R + wave) * 64 : kb + (size_t)(p.len - 1) * 64;
    const float* v_last = NPROJ == 3 ? proj_lds + (2 * R + wave) * 64 : vb + (size_t)(p.len - 1) * 64;
    const int len4 = (p.len + 3) & ~3;
    float* sc = att_lds + wave * (len4 + 256);
    float omax;
    if constexpr(STAGED) {
      const float* ks = kv_lds + (size_t)(2 * (wave & ((1 << p.share_shift) - 1))) * p.len * 64;
      const float* vs = ks + (size_t)p.len * 64;
      omax = attention_row64<true>(q, ks, vs, ks + (size_t)(p.len - 1) * 64, vs + (size_t)(p.len - 1) * 64, mk, mk0, p.len,
                             p.att_scale, sc, sc + len4, p.out + (size_t)wr * 64, lane);
    } else {
      omax = attention_row64(q, kb, vb, k_last, v_last, mk, mk0, p.len, p.att_scale, sc, sc + len4,
                             p.out + (size_t)wr * 64, lane);
    }
    if(p.absmax_out) {
      omax = wave_maxf(omax);
      if(lane == 0) p.absmax_out[wr] = omax;
    }
  }
}

// ---------------------------------------------------------------- n-best
// One workgroup of 1024 threads per row; a thread looks at every 1024th element (or group of
// four).  Scores are ordered by (value descending, index ascending).
//   1. every thread finds the largest of its scores, every wave the largest of its threads'; the
//      N-th largest of these 16 is a bound T: at least N elements of the row are >= T, so nothing
//      below T can be among the N best;
//   2. the row is read again (from cache) and the elements >= T - usually little more than N of
//      them - are collected in LDS with their positions;
//   3. the N best of the collected ones are found by rank (each candidate counts the candidates
//      before it), or drawn one at a time when there are more than 256.
// If more than 1024 elements pass the bound (large values concentrated in a few threads, or
// massive ties) every thread instead keeps the KEEP >= N best of its elements in registers and
// the draw pops them one by one.
constexpr int kNbestMax = 16;
constexpr long long kNbestMaxBatch = 4096;     // batch entries of the beam-major form
// Its counters, 256 bytes apart: atomics on one cache line are served one after the other
// (measured: the 256 arrivals of 32 entries on one line cost 7 us).
constexpr int kNbestCounterStride = 64;
constexpr size_t kNbestCounterBytes = kNbestMaxBatch * kNbestCounterStride * 4;

__device__ __forceinline__ bool nbest_before(float v, unsigned i, float w, unsigned j) {
  return v > w || (v == w && i < j);
}

struct NbestShared {
  float val[16];
  unsigned idx[16];
  int who[16];
  int winner;
  int count;
  float cand_val[1024];
  unsigned cand_idx[1024];
};

// Workgroup-wide best of one (value, index) per thread; every thread gets the result and the id of
// the thread that held it.
__device__ __forceinline__ void nbest_arg_best(float v, unsigned i, NbestShared& sh, float& gv, unsigned& gi,
                                               int& gw) {
  const int tid = threadIdx.x, lane = tid % 64, wave = tid / 64;
  float bv = v;
  unsigned bi = i;
  int bw = tid;
#pragma unroll
  for(int o = 32; o > 0; o >>= 1) {
    const float ov = __shfl_xor(bv, o, 64);
    const unsigned oi = (unsigned)__shfl_xor((int)bi, o, 64);
    const int ow = __shfl_xor(bw, o, 64);
    if(nbest_before(ov, oi, bv, bi)) {
      bv = ov; bi = oi; bw = ow;
    }
  }
  __syncthreads();   // the previous round's results have been read
  if(lane == 0) {
    sh.val[wave] = bv; sh.idx[wave] = bi; sh.who[wave] = bw;
  }
  __syncthreads();
  gv = sh.val[0]; gi = sh.idx[0]; gw = sh.who[0];
#pragma unroll
  for(int w = 1; w < 16; ++w)
    if(nbest_before(sh.val[w], sh.idx[w], gv, gi)) {
      gv = sh.val[w]; gi = sh.idx[w]; gw = sh.who[w];
    }
}

// One wave: the n best of `count` <= 64 (value, index) pairs, one per lane.
// A lane counts the pairs that come before its own; the lanes of rank < n call emit(rank, ...)
// themselves, and ranks that no pair fills (count < n) are emitted as (-inf, none) by lane 0.
template <typename Emit>
__device__ __forceinline__ void nbest_small_draw(const float* lv, const unsigned* li, int count, int n,
                                                 Emit emit) {
  const int lane = threadIdx.x % 64;
  const int e = min(lane, count - 1);
  const float v = lv[e];
  const unsigned ix = li[e];
  int rank = 0;
  for(int c = 0; c < count; ++c)   // (equal pairs - fillers (-inf, none) - rank in lane order)
    rank += (nbest_before(lv[c], li[c], v, ix) || (lv[c] == v && li[c] == ix && c < lane)) ? 1 : 0;
  if(lane < count && rank < n) emit(rank, v, ix);
  if(lane == 0)
    for(int r = count; r < n; ++r) emit(r, -__builtin_inff(), 0xFFFFFFFFu);
}

// Wave 0 only: draws the n best of the `count` <= 1024 (value, index) pairs in lv/li (LDS),
// sixteen per lane, without workgroup barriers.  emit(n, value, index) is called by lane 0.
template <typename Emit>
__device__ __forceinline__ void nbest_wave_draw(const float* lv, const unsigned* li, int count, int n,
                                                Emit emit) {
  const int lane = threadIdx.x % 64;
  const float ninf = -__builtin_inff();
  const unsigned none = 0xFFFFFFFFu;
  float v[16];
  unsigned ix[16];
#pragma unroll
  for(int j = 0; j < 16; ++j) {   // (clamped positions, dropped afterwards: all 32 loads in flight at once)
    const int e = min(j * 64 + lane, count - 1);
    v[j] = lv[e];
    ix[j] = li[e];
  }
#pragma unroll
  for(int j = 0; j < 16; ++j)
    if(j * 64 + lane >= count) {
      v[j] = ninf; ix[j] = none;
    }
  for(int r = 0; r < n; ++r) {
    float bv = v[0];
    unsigned bi = ix[0];
#pragma unroll
    for(int j = 1; j < 16; ++j)
      if(nbest_before(v[j], ix[j], bv, bi)) {
        bv = v[j]; bi = ix[j];
      }
    float gv = bv;
    unsigned gi = bi;
#pragma unroll
    for(int o = 32; o > 0; o >>= 1) {
      const float ov = __shfl_xor(gv, o, 64);
      const unsigned oi = (unsigned)__shfl_xor((int)gi, o, 64);
      if(nbest_before(ov, oi, gv, gi)) {
        gv = ov; gi = oi;
      }
    }
    if(lane == 0) emit(r, gv, gi);
    // the holder drops it (indices are unique, so at most one entry matches)
#pragma unroll
    for(int j = 0; j < 16; ++j)
      if(ix[j] == gi && gi != none) {
        v[j] = ninf; ix[j] = none;
      }
  }
}

// The N best of x[0 .. rowLen), by the whole workgroup (1024 threads).  emit(r, value, index) is
// called once for r = 0 .. N-1 (best first) by one thread each; index is the position within x.
// scan(f) calls f(value, index) for every element this thread owns (each element of the row is
// owned by exactly one thread of the workgroup; the order does not matter).
// The N-th largest of 16 values in LDS (equal values in index order), the same in every thread:
// lane l % 16 ranks value l % 16, the one of rank N - 1 is it (the cost does not grow with N).
__device__ __forceinline__ float nth_largest_of_16(const float* w16, int N) {
  const int c = threadIdx.x % 16;
  const float cvv = w16[c];
  int rank = 0;
#pragma unroll
  for(int w = 0; w < 16; ++w) rank += (w16[w] > cvv || (w16[w] == cvv && w < c)) ? 1 : 0;
  const unsigned long long holders = __ballot(rank == N - 1) & 0xFFFFull;
  return __shfl(cvv, __ffsll((long long)holders) - 1, 64);   // (ranks 0..15 are all taken: one holder)
}

// Steps 2 and 3: tv is a bound that at least N elements of the row reach (or -inf).
// count_is_zero: sh.count has been zero since a workgroup barrier that every thread has passed.
template <int KEEP, typename Scan, typename Emit>
__device__ __forceinline__ void nbest_from_bound(Scan scan, int N, NbestShared& sh, Emit emit, float tv,
                                                 bool count_is_zero) {
  const int tid = threadIdx.x;
  const float ninf = -__builtin_inff();
  const unsigned none = 0xFFFFFFFFu;

  // 2. collect what is >= the bound
  if(!count_is_zero) {
    if(tid == 0) sh.count = 0;
    __syncthreads();
  }
  scan([&](float v, unsigned i) {
    if(v >= tv) {
      const int slot = atomicAdd(&sh.count, 1);
      if(slot < 1024) {
        sh.cand_val[slot] = v; sh.cand_idx[slot] = i;
      }
    }
  });
  __syncthreads();
  const int count = sh.count;

  if(count <= 1024) {
    // 3. the N best of the collected elements, drawn by wave 0: up to 64, one per lane; more,
    //    sixteen per lane
    if(count <= 64) {
      if(tid < 64) nbest_small_draw(sh.cand_val, sh.cand_idx, count, N, emit);
    } else if(count <= 256) {
      // up to 256 (long lists): thread t ranks candidate t among all of them (distinct elements)
      if(tid < count) {
        const float v = sh.cand_val[tid];
        const unsigned ix = sh.cand_idx[tid];
        int rank = 0;
        for(int c = 0; c < count; ++c) rank += nbest_before(sh.cand_val[c], sh.cand_idx[c], v, ix) ? 1 : 0;
        if(rank < N) emit(rank, v, ix);
      }
    } else if(tid < 64) {
      nbest_wave_draw(sh.cand_val, sh.cand_idx, count, N, emit);
    }
    return;
  }

  // too many at or before the bound: per-thread sorted lists of the KEEP best, popped by the draw
  float val[KEEP];
  unsigned idx[KEEP];
#pragma unroll
  for(int j = 0; j < KEEP; ++j) {
    val[j] = ninf;
    idx[j] = none;
  }
  scan([&](float v, unsigned i) {
    if(nbest_before(v, i, val[KEEP - 1], idx[KEEP - 1])) {
      val[KEEP - 1] = v;
      idx[KEEP - 1] = i;
#pragma unroll
      for(int j = KEEP - 1; j > 0; --j) {
        if(nbest_before(val[j], idx[j], val[j - 1], idx[j - 1])) {
          const float sv = val[j]; val[j] = val[j - 1]; val[j - 1] = sv;
          const unsigned si = idx[j]; idx[j] = idx[j - 1]; idx[j - 1] = si;
        }
      }
    }
  });
  for(int n = 0; n < N; ++n) {
    float gv; unsigned gi; int who;
    nbest_arg_best(val[0], idx[0], sh, gv, gi, who);
    if(tid == 0) emit(n, gv, gi);
    if(tid == who) {   // pop the head
#pragma unroll
      for(int j = 0; j < KEEP - 1; ++j) {
        val[j] = val[j + 1];
        idx[j] = idx[j + 1];
      }
      val[KEEP - 1] = ninf;
      idx[KEEP - 1] = none;
    }
  }
}

template <int KEEP, typename Scan, typename Emit>
__device__ __forceinline__ void nbest_core(Scan scan, int N, NbestShared& sh, Emit emit) {
  const int tid = threadIdx.x;
  // 1. largest score of this thread, of its wave, and the N-th largest of the 16 wave maxima: the
  //    bound T.  The maxima belong to 16 distinct elements and N <= 16, so at least N elements of the
  //    row are >= T; for N = 16 and scores without structure some 50 are.  (A wave without elements
  //    contributes -inf; with fewer than N waves that hold elements the bound is -inf and
  //    everything passes.)
  float mv = -__builtin_inff();
  scan([&](float v, unsigned) { mv = fmaxf(mv, v); });
  const float wv = wave_maxf(mv);
  if(tid % 64 == 0) sh.val[tid / 64] = wv;
  __syncthreads();
  const float tv = nth_largest_of_16(sh.val, N);
  nbest_from_bound<KEEP>(scan, N, sh, emit, tv, false);
}

// The row in memory.  (Every scan keeps eight 16-byte loads in flight per thread; the last round
// reads clamped positions unconditionally and drops them afterwards, because loads behind a range
// check would be waited for one by one.)
template <int KEEP, typename Emit>
__device__ __forceinline__ void nbest_of_row(const float* __restrict__ x, long long rowLen, int N,
                                             NbestShared& sh, Emit emit) {
  const int tid = threadIdx.x;
  const bool vec = (rowLen % 4) == 0 && (reinterpret_cast<uintptr_t>(x) % 16) == 0;
  const long long n4 = rowLen / 4;
  auto scan = [&](auto f) __attribute__((always_inline)) {
    if(vec) {   // elements 4 * (t + 1024 * j) .. + 3
      const v4f* x4 = reinterpret_cast<const v4f*>(x);
      for(long long i = tid; i < n4; i += 8 * 1024) {
        v4f v[8];
#pragma unroll
        for(int u = 0; u < 8; ++u) v[u] = x4[min(i + u * 1024, n4 - 1)];
#pragma unroll
        for(int u = 0; u < 8; ++u) {
          if(i + u * 1024 >= n4) break;
          const unsigned b = (unsigned)(4 * (i + u * 1024));
          f(v[u].x, b); f(v[u].y, b + 1); f(v[u].z, b + 2); f(v[u].w, b + 3);
        }
      }
    } else {
      for(long long i = tid; i < rowLen; i += 16 * 1024) {
        float v[16];
#pragma unroll
        for(int u = 0; u < 16; ++u) v[u] = x[min(i + u * 1024, rowLen - 1)];
#pragma unroll
        for(int u = 0; u < 16; ++u)
          if(i + u * 1024 < rowLen) f(v[u], (unsigned)(i + u * 1024));
      }
    }
  };
  nbest_core<KEEP>(scan, N, sh, emit);
}

template <int KEEP>
__global__ __launch_bounds__(1024) void nbest_kernel(const float* __restrict__ scores, long long rowLen, int N,
                                                     float* __restrict__ outScores,
                                                     unsigned* __restrict__ outKeys) {
  __shared__ NbestShared sh;
  const long long row = blockIdx.x;
  nbest_of_row<KEEP>(scores + row * rowLen, rowLen, N, sh, [&](int r, float v, unsigned i) {
    outScores[row * N + r] = v;
    outKeys[row * N + r] = (unsigned)(row * rowLen) + i;
  });
}

// Hand-over of per-part candidates to the workgroup that finishes an entry last, without fences.
// What it relies on (gfx942/gfx950 memory model as the AMDGPU backend documents it): an agent-scope
// store or atomic bypasses the XCD-local L2 and is performed at the memory side, where all XCDs see
// it; a wave's vmcnt reaches zero only once each of its stores has been acknowledged from there; an
// agent-scope load reads from there too.  So: candidates stored (agent scope) -> vmcnt(0) in every
// wave -> workgroup barrier -> counter incremented; the workgroup that reads parts - 1 from the
// counter then loads (agent scope) candidates that are all in memory already.  FENCED makes the
// counter update an acquire-release operation instead (the compiler then adds the cache write-back /
// invalidate the language-level memory model asks for; ~8 us slower).  The tuning build holds both
// forms (marian_hip_nbest_set_fenced) and a GPU test compares them: if results ever differ, the
// hand-over is at fault and not the selection.  rowLen: length of an entry's whole row (keys are
// b * rowLen + position).
template <bool FENCED>
__device__ __forceinline__ void nbest_hand_over(NbestShared& sh, int* is_last, long long b, int parts, int N,
                                                long long rowLen, float* candVal, unsigned* candIdx,
                                                unsigned* counters, float* __restrict__ outScores,
                                                unsigned* __restrict__ outKeys) {
  constexpr int kCounterOrder = FENCED ? __ATOMIC_ACQ_REL : __ATOMIC_RELAXED;
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // every wave's stores have reached memory ...
  __syncthreads();
  if(threadIdx.x == 0)                               // ... before the count goes up
    *is_last = __hip_atomic_fetch_add(&counters[b * kNbestCounterStride], 1u, kCounterOrder,
                                      __HIP_MEMORY_SCOPE_AGENT) == (unsigned)(parts - 1);
  __syncthreads();
  if(!*is_last) return;
  // the entry's candidates (at most 1024 pairs), read past this XCD's caches, into LDS
  const int total = parts * N;
  for(int e = threadIdx.x; e < total; e += 1024) {
    sh.cand_val[e] = __hip_atomic_load(candVal + (size_t)b * total + e, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    sh.cand_idx[e] = __hip_atomic_load(candIdx + (size_t)b * total + e, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  __syncthreads();
  if(threadIdx.x < 64) {
    auto result = [&](int r, float v, unsigned i) {
      outScores[b * N + r] = v;
      outKeys[b * N + r] = (unsigned)(b * rowLen) + i;
    };
    if(total <= 64) nbest_small_draw(sh.cand_val, sh.cand_idx, total, N, result);
    else nbest_wave_draw(sh.cand_val, sh.cand_idx, total, N, result);
    if(threadIdx.x == 0)   // for the next call (every part of this entry has arrived: nobody else touches it)
      __hip_atomic_store(&counters[b * kNbestCounterStride], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
}

// Beam-major scores [beam, dimBatch, vocab]; the row of batch entry b is the beam's `beam` segments
// of `vocab` scores, element (k, v) at logical position k * vocab + v.  Workgroup (part, b) takes
// slice part % perSeg of segment part / perSeg and leaves the N best of it, with their logical
// positions, in cand*[(b * parts + part) * N ..]; a slice shorter than N fills up with
// (-inf, none), which sorts last.  The workgroup that finishes last for a batch entry (a counter per
// entry, zero between calls) draws the N best of all the entry's candidates.  No workgroup waits
// for another.
template <int KEEP, bool FENCED = false>
__global__ __launch_bounds__(1024) void nbest_part_kernel(const float* __restrict__ scores, long long dimBatch,
                                                          long long vocab, int perSeg, long long sliceLen,
                                                          int N, float* candVal, unsigned* candIdx,
                                                          unsigned* counters, float* __restrict__ outScores,
                                                          unsigned* __restrict__ outKeys) {
  __shared__ NbestShared sh;
  __shared__ int is_last;
  const int part = blockIdx.x, parts = gridDim.x;
  const long long b = blockIdx.y;
  const long long k = part / perSeg, v0 = (long long)(part % perSeg) * sliceLen;
  const long long len = min(sliceLen, vocab - v0);
  float* cv = candVal + ((size_t)b * parts + part) * N;
  unsigned* ci = candIdx + ((size_t)b * parts + part) * N;
  // Every path below publishes the candidates with stores that go through to memory
  // (device scope), so that whichever workgroup turns out to be the last can read them without a
  // cache write-back and invalidation around the counter (a fence pair costs ~8 us here).
  auto publish = [&](int r, float v, unsigned i) {
    __hip_atomic_store(cv + r, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __hip_atomic_store(ci + r, i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  };
  if(len < N) {   // (only a ragged last slice can be this short: one thread sorts it)
    if(threadIdx.x == 0) {
      const float* x = scores + ((size_t)k * dimBatch + b) * vocab + v0;
      float pv = __builtin_inff();
      long long pi = -1;
      for(int r = 0; r < N; ++r) {
        float bv = -__builtin_inff();
        long long bi = -1;
        for(long long c = 0; c < len; ++c) {
          const float v = x[c];
          const bool after_prev = r == 0 || v < pv || (v == pv && c > pi);
          if(after_prev && (bi < 0 || v > bv)) {
            bv = v; bi = c;
          }
        }
        publish(r, bi < 0 ? -__builtin_inff() : bv, bi < 0 ? 0xFFFFFFFFu : (unsigned)(k * vocab + v0 + bi));
        if(bi >= 0) { pv = bv; pi = bi; }
      }
    }
  } else {
    const unsigned base = (unsigned)(k * vocab + v0);
    nbest_of_row<KEEP>(scores + ((size_t)k * dimBatch + b) * vocab + v0, len, N, sh,
                       [&](int r, float v, unsigned i) { publish(r, v, base + i); });
  }
  nbest_hand_over<FENCED>(sh, &is_last, b, parts, N, (long long)(parts / perSeg) * vocab, candVal, candIdx, counters,
                  outScores, outKeys);
}

// Log-softmax of the rows of beam-major logits [beam, dimBatch, vocab] and the N best of every
// batch entry's beam * vocab log-probabilities in one launch: workgroup (k, b) keeps row (k, b) in
// registers (read once), computes the log-probabilities exactly as softmax_wide_kernel<true> does
// (optionally adds the row's path score and optionally writes them out), selects the N best of the
// row from the registers and leaves them as part k of entry b; the workgroup that finishes an
// entry last draws the N best of its beam * N candidates.
template <int VPT, int KEEP, bool FENCED = false>
__global__ __launch_bounds__(1024) void logsoftmax_nbest_kernel(const float* __restrict__ in,
                                                                const float* __restrict__ rowAdd,
                                                                float* __restrict__ lpOut, long long dimBatch,
                                                                int vocab, int N, float* candVal,
                                                                unsigned* candIdx, unsigned* counters,
                                                                float* __restrict__ outScores,
                                                                unsigned* __restrict__ outKeys) {
  __shared__ NbestShared sh;
  __shared__ int is_last;
  __shared__ float red[32];
  const int k = blockIdx.x, parts = gridDim.x, t = threadIdx.x;
  const long long b = blockIdx.y;
  const size_t row = (size_t)k * dimBatch + b;
  const int cols4 = vocab / 4;
  v4f v[VPT];
  if(t == 0) sh.count = 0;   // (the selection starts behind the barriers of the two reductions)
  // The selection's bound comes out of the softmax's own maximum: the N-th largest of the 16 wave
  // maxima of the logits (at least N logits reach it), taken through the same operations as every
  // element below, which are monotonic, so at least N scores reach the result.
  float bound_logit = -__builtin_inff(), row_max = 0.0f;
  const float log_sum = softmax_wide_row<true, 1024, VPT>(
      reinterpret_cast<const v4f*>(in + row * vocab), nullptr, cols4, v, red, [&](float mx, const float* wave_max) {
        row_max = mx;
        bound_logit = nth_largest_of_16(wave_max, N);
      });
  const float add = rowAdd ? rowAdd[row] : 0.0f;
  float tv = (bound_logit - row_max) - log_sum;
  if(rowAdd) tv = tv + add;
#pragma unroll
  for(int j = 0; j < VPT; ++j) {
    v[j] = v4f{v[j].x - log_sum, v[j].y - log_sum, v[j].z - log_sum, v[j].w - log_sum};
    if(lpOut && j * 1024 + t < cols4) reinterpret_cast<v4f*>(lpOut + row * vocab)[j * 1024 + t] = v[j];
    if(rowAdd) v[j] = v4f{v[j].x + add, v[j].y + add, v[j].z + add, v[j].w + add};
  }
  auto scan = [&](auto f) __attribute__((always_inline)) {
#pragma unroll
    for(int j = 0; j < VPT; ++j) {
      const int i4 = j * 1024 + t;
      if(i4 < cols4) {
        const unsigned e = 4u * (unsigned)i4;
        f(v[j].x, e); f(v[j].y, e + 1); f(v[j].z, e + 2); f(v[j].w, e + 3);
      }
    }
  };
  float* cv = candVal + ((size_t)b * parts + k) * N;
  unsigned* ci = candIdx + ((size_t)b * parts + k) * N;
  const unsigned base = (unsigned)k * (unsigned)vocab;
  nbest_from_bound<KEEP>(scan, N, sh, [&](int r, float val, unsigned i) {
    __hip_atomic_store(cv + r, val, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __hip_atomic_store(ci + r, base + i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }, tv, true);
  nbest_hand_over<FENCED>(sh, &is_last, b, parts, N, (long long)parts * vocab, candVal, candIdx, counters, outScores, outKeys);
}

// Fill: the 16-byte aligned middle of the range with 16-byte stores of the repeated pattern, the
// bytes before and after it one by one (byte i of the range holds byte i % elem_bytes of the
// pattern; the middle starts on an element boundary because the range does).
__global__ __launch_bounds__(256) void fill_kernel(unsigned char* __restrict__ p, long long bytes, long long head,
                                                   long long vecs, int elem_bytes, unsigned long long pattern) {
  const long long tid = (long long)blockIdx.x * blockDim.x + threadIdx.x, nthreads = (long long)gridDim.x * blockDim.x;
  unsigned long long rep = pattern;
  if(elem_bytes == 1) rep = (pattern & 0xFFull) * 0x0101010101010101ull;
  else if(elem_bytes == 2) rep = (pattern & 0xFFFFull) * 0x0001000100010001ull;
  else if(elem_bytes == 4) rep = (pattern & 0xFFFFFFFFull) * 0x0000000100000001ull;
  typedef unsigned long long v2u64 __attribute__((ext_vector_type(2)));
  v2u64* mid = reinterpret_cast<v2u64*>(p + head);
  for(long long i = tid; i < vecs; i += nthreads) mid[i] = v2u64{rep, rep};
  const long long tail0 = head + vecs * 16;
  for(long long i = tid; i < head + (bytes - tail0); i += nthreads) {
    const long long at = i < head ? i : tail0 + (i - head);
    p[at] = (unsigned char)(pattern >> (8 * (at % elem_bytes)));
  }
}

// ---------------------------------------------------------------- embedding step
// Workgroup (r, chunk) takes kEmbedChunk values of output row r: out[r, :] = scale * E[ids[r], :]
// (+ signal[(r / rows_per_signal) % n_signals, :]); rows of an embedding table are one chunk, the
// long rows of a decoder state (all cached positions of a hypothesis) many, so that such a gather
// fills the chip.  The product and the sum round separately.  An id at or past the table's end
// reads the table's last row.
constexpr int kEmbedChunk = 4096;
template <bool VEC>
__global__ __launch_bounds__(256) void embed_kernel(const float* __restrict__ E, const uint32_t* __restrict__ ids,
                                                    unsigned vocab, int dimEmb, float scale,
                                                    const float* __restrict__ signal, unsigned rows_per_signal,
                                                    unsigned n_signals, float* __restrict__ out,
                                                    float* __restrict__ absmax_out) {
  __shared__ float red[4];
  const unsigned row = blockIdx.x, chunk = blockIdx.y;
  const int tid = threadIdx.x;
  unsigned id = ids[row];
  id = id < vocab ? id : vocab - 1u;
  const int c0 = (int)chunk * kEmbedChunk, c1 = min(c0 + kEmbedChunk, dimEmb);
  const float* src = E + (size_t)id * dimEmb;
  const float* sg = signal ? signal + (size_t)((row / rows_per_signal) % n_signals) * dimEmb : nullptr;
  float* y = out + (size_t)row * dimEmb;
  float omax = 0.0f;
  if(VEC) {   // (four 16-byte loads per thread and operand, all requested before the first is used)
    constexpr int kV = kEmbedChunk / 4 / 256;
    const int last = c1 / 4 - 1;
    v4f e[kV], s[kV];
#pragma unroll
    for(int j = 0; j < kV; ++j) {
      const int i = min(c0 / 4 + j * 256 + tid, last);
      e[j] = reinterpret_cast<const v4f*>(src)[i];
      s[j] = sg ? reinterpret_cast<const v4f*>(sg)[i] : v4f{0.0f, 0.0f, 0.0f, 0.0f};
    }
#pragma unroll
    for(int j = 0; j < kV; ++j) {
      const int i = c0 / 4 + j * 256 + tid;
      if(i <= last) {
        v4f r = v4f{scale * e[j].x, scale * e[j].y, scale * e[j].z, scale * e[j].w};
        if(sg) r = v4f{r.x + s[j].x, r.y + s[j].y, r.z + s[j].z, r.w + s[j].w};
        omax = fmaxf(fmaxf(omax, fmaxf(fabsf(r.x), fabsf(r.y))), fmaxf(fabsf(r.z), fabsf(r.w)));
        reinterpret_cast<v4f*>(y)[i] = r;
      }
    }
  } else {
    for(int i = c0 + tid; i < c1; i += 256) {
      float r = scale * src[i];
      if(sg) r = r + sg[i];
      omax = fmaxf(omax, fabsf(r));
      y[i] = r;
    }
  }
  if(absmax_out) {   // a slot per workgroup; the first workgroup zeroes the slots past the last one
    const unsigned slot = row * gridDim.y + chunk, slots = gridDim.x * gridDim.y;
    omax = row_reduce<256, true>(omax, red);
    if(tid == 0) absmax_out[slot] = omax;
    if(slot == 0)
      for(int sl = (int)slots + tid; sl < kAbsmaxSlots; sl += 256) absmax_out[sl] = 0.0f;
  }
}

// The selection of decoder states whose entries are `segs` segments of seg_cap values of which the
// first seg_len are in use (cached positions of the heads of a hypothesis): workgroup (r * segs + s,
// chunk) copies kEmbedChunk values of segment s of entry ids[r]; what lies behind seg_len is neither
// read nor written.
template <bool VEC>
__global__ __launch_bounds__(256) void select_state_kernel(const float* __restrict__ in, const uint32_t* __restrict__ ids,
                                                           unsigned entries, unsigned segs, long long seg_cap,
                                                           int seg_len, float* __restrict__ out) {
  const unsigned row = blockIdx.x / segs, seg = blockIdx.x % segs, chunk = blockIdx.y;
  const int tid = threadIdx.x;
  unsigned id = ids[row];
  id = id < entries ? id : entries - 1u;
  const int c0 = (int)chunk * kEmbedChunk, c1 = min(c0 + kEmbedChunk, seg_len);
  const float* src = in + ((size_t)id * segs + seg) * (size_t)seg_cap;
  float* dst = out + ((size_t)row * segs + seg) * (size_t)seg_cap;
  if(VEC) {
    constexpr int kV = kEmbedChunk / 4 / 256;
    const int last = c1 / 4 - 1;
    v4f e[kV];
#pragma unroll
    for(int j = 0; j < kV; ++j) e[j] = reinterpret_cast<const v4f*>(src)[min(c0 / 4 + j * 256 + tid, last)];
#pragma unroll
    for(int j = 0; j < kV; ++j) {
      const int i = c0 / 4 + j * 256 + tid;
      if(i <= last) reinterpret_cast<v4f*>(dst)[i] = e[j];
    }
  } else {
    for(int i = c0 + tid; i < c1; i += 256) dst[i] = src[i];
  }
}

__global__ __launch_bounds__(256) void zero_words_kernel(unsigned* __restrict__ p, long long n) {
  for(long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (long long)gridDim.x * blockDim.x)
    p[i] = 0u;
}

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) % 16) == 0; }
inline bool aligned4(const void* p) { return (reinterpret_cast<uintptr_t>(p) % 4) == 0; }

#define MH_HIP(expr)                                      \
  do {                                                    \
    hipError_t e_ = (expr);                               \
    if(e_ != hipSuccess) return record_hip_error((int)e_); \
  } while(0)

// Which form of the n-best hand-over the launchers take: the shipped library has the unfenced one
// only; the tuning build holds both behind a process-wide switch.
#ifdef MARIAN_HIP_TUNING
std::atomic<int> g_nbest_fenced{0};
inline bool nbest_fenced() { return g_nbest_fenced.load(std::memory_order_relaxed) != 0; }
#else
constexpr bool nbest_fenced() { return false; }
#endif

}  // namespace

extern "C" {

#ifdef MARIAN_HIP_TUNING
int marian_hip_nbest_set_fenced(int on) { return g_nbest_fenced.exchange(on ? 1 : 0); }
#endif

int marian_hip_layer_norm(const float* in, const float* add, const float* gamma, int64_t gamma_cols,
                          const float* beta, int64_t beta_cols, float* out, int64_t rows,
                          int64_t cols, float eps, float* absmax_out, void* stream) {
  if(absmax_out && !aligned4(absmax_out)) return MARIAN_HIP_ERR_ALIGN;
  if(rows < 0 || cols <= 0) return MARIAN_HIP_ERR_SHAPE;
  if((gamma_cols != cols && gamma_cols != 1) || (beta && beta_cols != cols && beta_cols != 1))
    return MARIAN_HIP_ERR_SHAPE;
  if(rows == 0) return MARIAN_HIP_OK;
  if(!in || !gamma || !out) return MARIAN_HIP_ERR_NULL;
  if(rows * cols > kMaxElemsOps) return MARIAN_HIP_ERR_RANGE;
  if(!aligned4(in) || !aligned4(out) || !aligned4(gamma) || (add && !aligned4(add)) || (beta && !aligned4(beta)))
    return MARIAN_HIP_ERR_ALIGN;
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  const int gs = gamma_cols > 1 ? 1 : 0, bs = (beta && beta_cols > 1) ? 1 : 0;
  const bool vec = cols % 4 == 0 && aligned16(in) && aligned16(out) && (!add || aligned16(add));
  const bool wave_form = vec && cols <= 1024 && (gs == 0 || aligned16(gamma)) &&
                         (!beta || bs == 0 || aligned16(beta));
  // more rows than abs-max slots (an encoder's sentence batch): the rows share the slots, which are
  // cleared first (a kernel, so that the call may sit in a recorded graph)
  const int wrap = absmax_out && rows > kAbsmaxSlots ? 1 : 0;
  if(wrap) {
    hipLaunchKernelGGL(zero_words_kernel, dim3(kAbsmaxSlots / 256), dim3(256), 0, st, reinterpret_cast<unsigned*>(absmax_out),
                       (long long)kAbsmaxSlots);
    MH_HIP(hipGetLastError());
  }
  if(wave_form)
    hipLaunchKernelGGL(layer_norm_wave_kernel, dim3((unsigned)rows), dim3(64), 0, st, in, add, gamma, gs, beta, bs, out, (int)cols, eps, absmax_out, wrap);
  else if(vec && cols <= 1024)
    hipLaunchKernelGGL(layer_norm_kernel<1>, dim3((unsigned)rows), dim3(256), 0, st, in, add, gamma, gs, beta, bs, out, (int)cols, eps, absmax_out, wrap);
  else if(vec && cols <= 4096)
    hipLaunchKernelGGL(layer_norm_kernel<4>, dim3((unsigned)rows), dim3(256), 0, st, in, add, gamma, gs, beta, bs, out, (int)cols, eps, absmax_out, wrap);
  else if(vec && cols <= 8192)
    hipLaunchKernelGGL(layer_norm_kernel<8>, dim3((unsigned)rows), dim3(256), 0, st, in, add, gamma, gs, beta, bs, out, (int)cols, eps, absmax_out, wrap);
  else
    hipLaunchKernelGGL(layer_norm_kernel<0>, dim3((unsigned)rows), dim3(256), 0, st, in, add, gamma, gs, beta, bs, out, (int)cols, eps, absmax_out, wrap);
  MH_HIP(hipGetLastError());
  return MARIAN_HIP_OK;
}

int marian_hip_embed(const float* E, const uint32_t* ids, int64_t rows, int64_t vocab, int64_t dimEmb,
                     float scale, const float* signal, int64_t rows_per_signal, int64_t n_signals,
                     float* out, float* absmax_out, void* stream) {
  if(rows < 0 || vocab <= 0 || dimEmb <= 0) return MARIAN_HIP_ERR_SHAPE;
  const int64_t chunks = (dimEmb + kEmbedChunk - 1) / kEmbedChunk;
  if(absmax_out && rows * chunks > kAbsmaxSlots) return MARIAN_HIP_ERR_RANGE;
  if(absmax_out && !aligned4(absmax_out)) return MARIAN_HIP_ERR_ALIGN;
  if(signal && (rows_per_signal <= 0 || n_signals <= 0)) return MARIAN_HIP_ERR_SHAPE;
  if(rows == 0) return MARIAN_HIP_OK;
  if(!E || !ids || !out) return MARIAN_HIP_ERR_NULL;
  if(chunks > 65535 || rows * dimEmb > kMaxElemsOps || vocab > 0xFFFFFFFFLL || rows_per_signal > 0x7FFFFFFFLL ||
     n_signals > 0x7FFFFFFFLL || (signal && n_signals * dimEmb > kMaxElemsOps))
    return MARIAN_HIP_ERR_RANGE;
  if(!aligned4(E) || !aligned4(ids) || !aligned4(out) || (signal && !aligned4(signal))) return MARIAN_HIP_ERR_ALIGN;
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  const bool vec = dimEmb % 4 == 0 && aligned16(E) && aligned16(out) && (!signal || aligned16(signal));
  const unsigned rps = signal ? (unsigned)rows_per_signal : 1u, ns = signal ? (unsigned)n_signals : 1u;
  if(vec)
    hipLaunchKernelGGL(embed_kernel<true>, dim3((unsigned)rows, (unsigned)chunks), dim3(256), 0, st, E, ids,
                       (unsigned)vocab, (int)dimEmb, scale, signal, rps, ns, out, absmax_out);
  else
    hipLaunchKernelGGL(embed_kernel<false>, dim3((unsigned)rows, (unsigned)chunks), dim3(256), 0, st, E, ids,
                       (unsigned)vocab, (int)dimEmb, scale, signal, rps, ns, out, absmax_out);
  MH_HIP(hipGetLastError());
  return MARIAN_HIP_OK;
}

int marian_hip_select_state(const float* state, const uint32_t* ids, int64_t rows, int64_t entries,
                            int64_t segments, int64_t seg_capacity, int64_t seg_len, float* out, void* stream) {
  if(rows < 0 || entries <= 0 || segments <= 0 || seg_capacity <= 0 || seg_len < 0 || seg_len > seg_capacity)
    return MARIAN_HIP_ERR_SHAPE;
  if(rows == 0 || seg_len == 0) return MARIAN_HIP_OK;
  if(!state || !ids || !out) return MARIAN_HIP_ERR_NULL;
  const int64_t chunks = (seg_len + kEmbedChunk - 1) / kEmbedChunk;
  if(entries > 0xFFFFFFFFLL || segments > 65535 || rows > kMaxElemsOps / segments || chunks > 65535 ||
     seg_len > kMaxElemsOps ||
     entries * segments > kMaxElemsOps / seg_capacity || rows * segments > kMaxElemsOps / seg_capacity)
    return MARIAN_HIP_ERR_RANGE;
  if(!aligned4(state) || !aligned4(ids) || !aligned4(out)) return MARIAN_HIP_ERR_ALIGN;
  // not in place: an entry may be read after the row of the same number has been written
  const uintptr_t a0 = reinterpret_cast<uintptr_t>(state), a1 = a0 + (uintptr_t)(entries * segments * seg_capacity) * 4;
  const uintptr_t b0 = reinterpret_cast<uintptr_t>(out), b1 = b0 + (uintptr_t)(rows * segments * seg_capacity) * 4;
  if(a0 < b1 && b0 < a1) return MARIAN_HIP_ERR_ALIAS;
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  const bool vec = seg_len % 4 == 0 && seg_capacity % 4 == 0 && aligned16(state) && aligned16(out);
  const dim3 grid((unsigned)(rows * segments), (unsigned)chunks);
  if(vec)
    hipLaunchKernelGGL(select_state_kernel<true>, grid, dim3(256), 0, st, state, ids, (unsigned)entries, (unsigned)segments,
                       (long long)seg_capacity, (int)seg_len, out);
  else
    hipLaunchKernelGGL(select_state_kernel<false>, grid, dim3(256), 0, st, state, ids, (unsigned)entries, (unsigned)segments,
                       (long long)seg_capacity, (int)seg_len, out);
  MH_HIP(hipGetLastError());
  return MARIAN_HIP_OK;
}

int marian_hip_sinusoidal_position_embeddings(float* host_out, int64_t dimWords, int64_t dimEmb, int64_t start) {
  if(dimWords < 0 || dimEmb < 4) return MARIAN_HIP_ERR_SHAPE;   // (one timescale: the increment divides by zero)
  if(dimWords == 0) return MARIAN_HIP_OK;
  if(!host_out) return MARIAN_HIP_ERR_NULL;
  if(dimWords * dimEmb > kMaxElemsOps || start < 0 || start + dimWords > 0x7FFFFFFFLL) return MARIAN_HIP_ERR_RANGE;
  const float numTimescales = (float)dimEmb / 2;
  const int half = (int)numTimescales;
  const float logTimescaleIncrement = std::log(10000.f) / (numTimescales - 1.f);
  for(int64_t j = 0; j < dimWords; ++j) {
    const int position = (int)(j + start);
    float* row = host_out + j * dimEmb;
    for(int i = 0; i < (int)dimEmb; ++i) {
      const float v = (float)position * std::exp((float)(i % half) * -logTimescaleIncrement);
      row[i] = i < half ? std::sin(v) : std::cos(v);
    }
  }
  return MARIAN_HIP_OK;
}

static int softmax_common(const float* in, const float* mask, int64_t n_masks, int64_t rows_per_mask,
                          float* out, int64_t rows, int64_t cols, bool log, void* stream) {
  if(rows < 0 || cols <= 0) return MARIAN_HIP_ERR_SHAPE;
  if(mask && (n_masks <= 0 || rows_per_mask <= 0)) return MARIAN_HIP_ERR_SHAPE;
  if(rows == 0) return MARIAN_HIP_OK;
  if(!in || !out) return MARIAN_HIP_ERR_NULL;
  if(rows * cols > kMaxElemsOps) return MARIAN_HIP_ERR_RANGE;
  if(!aligned4(in) || !aligned4(out) || (mask && !aligned4(mask))) return MARIAN_HIP_ERR_ALIGN;
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  if(!mask) { n_masks = 1; rows_per_mask = 1; }
  // rows of more than 256 values that fit the registers of one workgroup: read once (a wave per row
  // walks a 1024-value row in 16 dependent steps per pass: 10 us for 128 rows against 4)
  const bool wide_ok = cols % 4 == 0 && cols <= 65536 && aligned16(in) && aligned16(out) && (!mask || aligned16(mask));
  if(cols <= 2048 && !(wide_ok && cols > 256)) {
    const unsigned blocks = (unsigned)((rows + 3) / 4);
    if(log) hipLaunchKernelGGL((softmax_kernel<64, true>), dim3(blocks), dim3(256), 0, st, in, mask, (long long)n_masks, (long long)rows_per_mask, out, (long long)rows, (int)cols);
    else hipLaunchKernelGGL((softmax_kernel<64, false>), dim3(blocks), dim3(256), 0, st, in, mask, (long long)n_masks, (long long)rows_per_mask, out, (long long)rows, (int)cols);
  } else if(wide_ok && cols <= 4096) {
    if(log) hipLaunchKernelGGL((softmax_wide_kernel<true, 256, 4>), dim3((unsigned)rows), dim3(256), 0, st, in, mask, (long long)n_masks, (long long)rows_per_mask, out, (int)cols);
    else hipLaunchKernelGGL((softmax_wide_kernel<false, 256, 4>), dim3((unsigned)rows), dim3(256), 0, st, in, mask, (long long)n_masks, (long long)rows_per_mask, out, (int)cols);
  } else if(wide_ok && cols <= 32768) {
    if(log) hipLaunchKernelGGL((softmax_wide_kernel<true, 1024, 8>), dim3((unsigned)rows), dim3(1024), 0, st, in, mask, (long long)n_masks, (long long)rows_per_mask, out, (int)cols);
    else hipLaunchKernelGGL((softmax_wide_kernel<false, 1024, 8>), dim3((unsigned)rows), dim3(1024), 0, st, in, mask, (long long)n_masks, (long long)rows_per_mask, out, (int)cols);
  } else if(wide_ok) {
    if(log) hipLaunchKernelGGL((softmax_wide_kernel<true, 1024, 16>), dim3((unsigned)rows), dim3(1024), 0, st, in, mask, (long long)n_masks, (long long)rows_per_mask, out, (int)cols);
    else hipLaunchKernelGGL((softmax_wide_kernel<false, 1024, 16>), dim3((unsigned)rows), dim3(1024), 0, st, in, mask, (long long)n_masks, (long long)rows_per_mask, out, (int)cols);
  } else {
    if(log) hipLaunchKernelGGL((softmax_kernel<1024, true>), dim3((unsigned)rows), dim3(1024), 0, st, in, mask, (long long)n_masks, (long long)rows_per_mask, out, (long long)rows, (int)cols);
    else hipLaunchKernelGGL((softmax_kernel<1024, false>), dim3((unsigned)rows), dim3(1024), 0, st, in, mask, (long long)n_masks, (long long)rows_per_mask, out, (long long)rows, (int)cols);
  }
  MH_HIP(hipGetLastError());
  return MARIAN_HIP_OK;
}

int marian_hip_softmax(const float* in, const float* mask, int64_t n_masks, int64_t rows_per_mask,
                       float* out, int64_t rows, int64_t cols, void* stream) {
  return softmax_common(in, mask, n_masks, rows_per_mask, out, rows, cols, false, stream);
}

int marian_hip_logsoftmax(const float* in, float* out, int64_t rows, int64_t cols, void* stream) {
  return softmax_common(in, nullptr, 1, 1, out, rows, cols, true, stream);
}

int marian_hip_transpose0213(const float* in, float* out, int64_t d0, int64_t d1, int64_t d2,
                             int64_t d3, void* stream) {
  if(d0 < 0 || d1 <= 0 || d2 <= 0 || d3 <= 0) return MARIAN_HIP_ERR_SHAPE;
  if(d0 == 0) return MARIAN_HIP_OK;
  if(!in || !out) return MARIAN_HIP_ERR_NULL;
  if(in == out) return MARIAN_HIP_ERR_SHAPE;
  if(d0 * d1 * d2 * d3 > kMaxElemsOps) return MARIAN_HIP_ERR_RANGE;
  if(!aligned4(in) || !aligned4(out)) return MARIAN_HIP_ERR_ALIGN;
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  const bool vec = d3 % 4 == 0 && aligned16(in) && aligned16(out);
  const long long total = d0 * d1 * d2 * (vec ? d3 / 4 : d3);
  long long blocks = (total + 255) / 256;
  if(blocks > 8192) blocks = 8192;
  if(vec) hipLaunchKernelGGL(transpose0213_kernel<4>, dim3((unsigned)blocks), dim3(256), 0, st, in, out, total, (int)d1, (int)d2, (int)(d3 / 4));
  else hipLaunchKernelGGL(transpose0213_kernel<1>, dim3((unsigned)blocks), dim3(256), 0, st, in, out, total, (int)d1, (int)d2, (int)d3);
  MH_HIP(hipGetLastError());
  return MARIAN_HIP_OK;
}

int marian_hip_bdot_legacy(const float* A, const float* B, float* C, int64_t batchA, int64_t batchB,
                           int64_t m, int64_t n, int64_t k, int transA, int transB, float scalar,
                           void* stream) {
  if(batchA < 0 || batchB < 0 || m <= 0 || n <= 0 || k <= 0) return MARIAN_HIP_ERR_SHAPE;
  if(batchA == 0 || batchB == 0) return MARIAN_HIP_OK;
  if(!A || !B || !C) return MARIAN_HIP_ERR_NULL;
  const int64_t batchC = batchA > batchB ? batchA : batchB;
  if(batchA * m * k > kMaxElemsOps || batchB * n * k > kMaxElemsOps || batchC * m * n > kMaxElemsOps)
    return MARIAN_HIP_ERR_RANGE;
  if(!aligned4(A) || !aligned4(B) || !aligned4(C)) return MARIAN_HIP_ERR_ALIGN;
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  const long long rows_total = batchC * m;
  const bool tile_ok = !transA && m >= 8 && batchC <= 65535 && aligned16(A) && aligned16(B) &&
                       (transB ? k % 4 == 0 : (k % 4 == 0 && n % 4 == 0));
  if(tile_ok) {
    const dim3 grid((unsigned)((n + 63) / 64), (unsigned)((m + 63) / 64), (unsigned)batchC);
    if(transB)
      hipLaunchKernelGGL(bdot_tile_kernel<true>, grid, dim3(256), 0, st, A, B, C, (long long)batchA,
                         (long long)batchB, (int)m, (int)n, (int)k, scalar);
    else
      hipLaunchKernelGGL(bdot_tile_kernel<false>, grid, dim3(256), 0, st, A, B, C, (long long)batchA,
                         (long long)batchB, (int)m, (int)n, (int)k, scalar);
    MH_HIP(hipGetLastError());
    return MARIAN_HIP_OK;
  }
  hipLaunchKernelGGL(bdot_kernel, dim3((unsigned)((rows_total + 3) / 4)), dim3(256), 0, st, A, B, C,
                     (long long)batchA, (long long)batchB, rows_total, (int)m, (int)n, (int)k,
                     transA ? 1 : 0, transB ? 1 : 0, scalar);
  MH_HIP(hipGetLastError());
  return MARIAN_HIP_OK;
}

int marian_hip_attention(const float* q, float* k, float* v, const float* mask, int64_t n_masks,
                         int64_t rows_per_mask, float* out, int64_t batchQ, int64_t batchKV,
                         int64_t m, int64_t len, int64_t dk, float scale, float* absmax_out,
                         const float* k_new, const float* v_new, void* stream) {
  return marian_hip_attention_cached(q, k, v, mask, n_masks, rows_per_mask, out, batchQ, batchKV, m, len, len, dk,
                                     scale, absmax_out, k_new, v_new, stream);
}

static int attention_impl(const float* q, float* k, float* v, const float* mask, int64_t n_masks,
                          int64_t rows_per_mask, float* out, int64_t batchQ, int64_t batchKV, int64_t m,
                          int64_t len, int64_t kv_capacity, int64_t dk, float scale, float* absmax_out,
                          const float* k_new, const float* v_new, const uint32_t* ancestors, int64_t heads,
                          void* stream);

int marian_hip_attention_cached(const float* q, float* k, float* v, const float* mask, int64_t n_masks,
                                int64_t rows_per_mask, float* out, int64_t batchQ, int64_t batchKV,
                                int64_t m, int64_t len, int64_t kv_capacity, int64_t dk, float scale,
                                float* absmax_out, const float* k_new, const float* v_new, void* stream) {
  return attention_impl(q, k, v, mask, n_masks, rows_per_mask, out, batchQ, batchKV, m, len, kv_capacity, dk, scale,
                        absmax_out, k_new, v_new, nullptr, 1, stream);
}

int marian_hip_attention_ancestors(const float* q, float* k, float* v, float* out, int64_t n_hyp, int64_t heads,
                                   int64_t len, int64_t kv_capacity, int64_t dk, float scale, float* absmax_out,
                                   const float* k_new, const float* v_new, const uint32_t* ancestors,
                                   void* stream) {
  if(n_hyp < 0 || heads <= 0 || dk != 64) return MARIAN_HIP_ERR_SHAPE;
  if(n_hyp == 0) return MARIAN_HIP_OK;
  if(!ancestors || !k_new || !v_new) return MARIAN_HIP_ERR_NULL;
  if(n_hyp > kMaxElemsOps / heads) return MARIAN_HIP_ERR_RANGE;
  if(!aligned4(ancestors)) return MARIAN_HIP_ERR_ALIGN;
  if(q && k && v && (!aligned16(q) || !aligned16(k) || !aligned16(v) || !aligned16(k_new) || !aligned16(v_new)))
    return MARIAN_HIP_ERR_ALIGN;
  return attention_impl(q, k, v, nullptr, 0, 0, out, n_hyp * heads, n_hyp * heads, 1, len, kv_capacity, dk, scale,
                        absmax_out, k_new, v_new, ancestors, heads, stream);
}

// next[h, p] = prev[parents[h], p] for the len_prev positions cached so far, next[h, len_prev] = h:
// the position the coming step appends lies in the hypothesis's own entry.
__global__ __launch_bounds__(256) void ancestors_advance_kernel(const uint32_t* __restrict__ prev,
                                                                const uint32_t* __restrict__ parents, unsigned n_hyp,
                                                                unsigned kv_cap, unsigned len_prev,
                                                                uint32_t* __restrict__ next) {
  const unsigned i = blockIdx.x * 256 + threadIdx.x;
  if(i >= n_hyp * (len_prev + 1)) return;
  const unsigned h = i / (len_prev + 1), p = i % (len_prev + 1);
  const unsigned from = min(parents[h], n_hyp - 1u);
  next[(size_t)h * kv_cap + p] = p < len_prev ? prev[(size_t)from * kv_cap + p] : h;
}

int marian_hip_ancestors_advance(const uint32_t* prev, const uint32_t* parents, int64_t n_hyp, int64_t kv_capacity,
                                 int64_t len_prev, uint32_t* next, void* stream) {
  if(n_hyp < 0 || kv_capacity <= 0 || len_prev < 0 || len_prev >= kv_capacity) return MARIAN_HIP_ERR_SHAPE;
  if(n_hyp == 0) return MARIAN_HIP_OK;
  if(!prev || !parents || !next) return MARIAN_HIP_ERR_NULL;
  if(n_hyp > kMaxElemsOps / kv_capacity) return MARIAN_HIP_ERR_RANGE;
  if(!aligned4(prev) || !aligned4(parents) || !aligned4(next)) return MARIAN_HIP_ERR_ALIGN;
  const uintptr_t a0 = reinterpret_cast<uintptr_t>(prev), b0 = reinterpret_cast<uintptr_t>(next);
  const uintptr_t bytes = (uintptr_t)(n_hyp * kv_capacity) * 4;
  if(a0 < b0 + bytes && b0 < a0 + bytes) return MARIAN_HIP_ERR_ALIAS;   // (a row may be read after the row of the same number has been written)
  const int64_t n = n_hyp * (len_prev + 1);
  hipLaunchKernelGGL(ancestors_advance_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0,
                     reinterpret_cast<hipStream_t>(stream), prev, parents, (unsigned)n_hyp, (unsigned)kv_capacity,
                     (unsigned)len_prev, next);
  MH_HIP(hipGetLastError());
  return MARIAN_HIP_OK;
}

static int attention_impl(const float* q, float* k, float* v, const float* mask, int64_t n_masks,
                          int64_t rows_per_mask, float* out, int64_t batchQ, int64_t batchKV, int64_t m,
                          int64_t len, int64_t kv_capacity, int64_t dk, float scale, float* absmax_out,
                          const float* k_new, const float* v_new, const uint32_t* ancestors, int64_t heads,
                          void* stream) {
  if((k_new != nullptr) != (v_new != nullptr)) return MARIAN_HIP_ERR_NULL;
  if(kv_capacity < len) return MARIAN_HIP_ERR_SHAPE;
  if(k_new && (m != 1 || batchKV != batchQ)) return MARIAN_HIP_ERR_SHAPE;
  if(k_new && (!aligned4(k_new) || !aligned4(v_new))) return MARIAN_HIP_ERR_ALIGN;
  if(absmax_out && batchQ * m > kAbsmaxSlots) return MARIAN_HIP_ERR_RANGE;
  if(absmax_out && !aligned4(absmax_out)) return MARIAN_HIP_ERR_ALIGN;
  if(batchQ < 0 || batchKV <= 0 || m <= 0 || len <= 0 || dk <= 0) return MARIAN_HIP_ERR_SHAPE;
  if(mask && (n_masks <= 0 || rows_per_mask <= 0)) return MARIAN_HIP_ERR_SHAPE;
  if(mask && (n_masks > 2147483647LL || rows_per_mask > 2147483647LL)) return MARIAN_HIP_ERR_RANGE;
  if(len > 4096) return MARIAN_HIP_ERR_RANGE;
  if(batchQ == 0) return MARIAN_HIP_OK;
  if(!q || !k || !v || !out) return MARIAN_HIP_ERR_NULL;
  if(kv_capacity > kMaxElemsOps || batchQ * m * dk > kMaxElemsOps || batchKV * kv_capacity * dk > kMaxElemsOps)
    return MARIAN_HIP_ERR_RANGE;
  if(!aligned4(q) || !aligned4(k) || !aligned4(v) || !aligned4(out) || (mask && !aligned4(mask)))
    return MARIAN_HIP_ERR_ALIGN;
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  if(!mask) { n_masks = 1; rows_per_mask = 1; }
  const long long rows_total = batchQ * m;
  const size_t lds = (size_t)4 * (size_t)(((len + 3) & ~(int64_t)3) + 256) * sizeof(float);   // per wave: scores (whole 16-byte units) + partial outputs
  {   // the kernel's dynamic LDS limit, raised once per device (one bit per device)
    static std::atomic<uint64_t> lds_done{0};
    int dev = 0;
    MH_HIP(hipGetDevice(&dev));
    if(dev < 0 || dev >= 64) return MARIAN_HIP_ERR_RANGE;
    if(!(lds_done.load(std::memory_order_acquire) & (1ull << dev))) {
      MH_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(attention_kernel<false>),
                                 hipFuncAttributeMaxDynamicSharedMemorySize, 72 * 1024));
      MH_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(attention_kernel<true>),
                                 hipFuncAttributeMaxDynamicSharedMemorySize, 72 * 1024));
      lds_done.fetch_or(1ull << dev, std::memory_order_release);
    }
  }
  // Complete caches that several query rows share, head size 64, one position per row, everything
  // aligned for 16-byte loads: the rows of a cache entry in one workgroup, the entry read once.
  if(!ancestors && !k_new && dk == 64 && m == 1 && len <= kSharedAttLen && batchKV < rows_total && rows_total % batchKV == 0 &&
     rows_total / batchKV <= 4 * 65535 && aligned16(q) && aligned16(k) && aligned16(v) && aligned16(out)) {
    const long long hyps = rows_total / batchKV;
    const dim3 grid((unsigned)batchKV, (unsigned)((hyps + 3) / 4));
    const size_t slds = (size_t)2 * (size_t)len * 256 + lds;
#define MH_SATT(PASSES) \
    hipLaunchKernelGGL(attention_shared_kernel<PASSES>, grid, dim3(256), slds, st, q, k, v, mask, (unsigned)n_masks, \
                       (unsigned)rows_per_mask, out, (unsigned)rows_total, (unsigned)batchKV, (int)len, (int)kv_capacity, \
                       scale, absmax_out)
    if(len <= 32) MH_SATT(2);
    else if(len <= 64) MH_SATT(4);
    else MH_SATT(6);
#undef MH_SATT
    MH_HIP(hipGetLastError());
    return MARIAN_HIP_OK;
  }
  if(ancestors)
    hipLaunchKernelGGL(attention_kernel<true>, dim3((unsigned)((rows_total + 3) / 4)), dim3(256), lds, st, q, k, v,
                       k_new, v_new, mask, (unsigned)n_masks, (unsigned)rows_per_mask, out, (unsigned)rows_total,
                       (unsigned)batchKV, (int)m, (int)len, (int)kv_capacity, (int)dk, scale, absmax_out, ancestors,
                       (unsigned)heads);
  else
    hipLaunchKernelGGL(attention_kernel<false>, dim3((unsigned)((rows_total + 3) / 4)), dim3(256), lds, st, q, k, v,
                       k_new, v_new, mask, (unsigned)n_masks, (unsigned)rows_per_mask, out, (unsigned)rows_total,
                       (unsigned)batchKV, (int)m, (int)len, (int)kv_capacity, (int)dk, scale, absmax_out, ancestors,
                       1u);
  MH_HIP(hipGetLastError());
  return MARIAN_HIP_OK;
}

int marian_hip_int8_proj_attention(const float* A, int8_t* Aq, int64_t n_proj, const int8_t* const* Bq,
                                   const float* const* bias, float* const* proj_out, int64_t M, int64_t K,
                                   int64_t heads, float* k_cache, float* v_cache, int64_t batchKV, int64_t len,
                                   int64_t kv_capacity, const float* mask, int64_t n_masks, float att_scale,
                                   float* out, const float* absmax_in, float* absmax_out, void* workspace,
                                   size_t workspace_bytes, void* stream) {
  if(n_proj != 1 && n_proj != 3) return MARIAN_HIP_ERR_SHAPE;
  if(M < 0 || K <= 0 || heads <= 0 || (K % 128) != 0 || K > kProjMaxK) return MARIAN_HIP_ERR_SHAPE;
  if(len <= 0 || len > kProjMaxLen || kv_capacity < len || batchKV <= 0) return MARIAN_HIP_ERR_SHAPE;
  if(mask && n_masks <= 0) return MARIAN_HIP_ERR_SHAPE;
  if(M == 0) return MARIAN_HIP_OK;
  if(!A || !Aq || !Bq || !k_cache || !v_cache || !out) return MARIAN_HIP_ERR_NULL;
  if(M * heads > kMaxElemsOps / 64 || batchKV * kv_capacity > kMaxElemsOps / 64 || M * K > kMaxElemsOps ||
     K * heads * 64 > kMaxElemsOps || n_masks > 2147483647LL)
    return MARIAN_HIP_ERR_RANGE;
  // the self-attention form appends to the caches: every query row needs an entry of its own
  if(n_proj == 3 && batchKV != M * heads) return MARIAN_HIP_ERR_SHAPE;
  if(absmax_out && M * heads > kAbsmaxSlots) return MARIAN_HIP_ERR_RANGE;
  if(!aligned16(A) || !aligned16(Aq) || !aligned16(k_cache) || !aligned16(v_cache) || !aligned16(out))
    return MARIAN_HIP_ERR_ALIGN;
  if((mask && !aligned4(mask)) || (absmax_in && !aligned4(absmax_in)) || (absmax_out && !aligned4(absmax_out)))
    return MARIAN_HIP_ERR_ALIGN;
  ProjAttentionArgs p;
  for(int g = 0; g < 3; ++g) {
    p.Bq[g] = nullptr; p.bias[g] = nullptr; p.proj_out[g] = nullptr;
  }
  for(int64_t g = 0; g < n_proj; ++g) {
    if(!Bq[g]) return MARIAN_HIP_ERR_NULL;
    p.Bq[g] = Bq[g];
    p.bias[g] = bias ? bias[g] : nullptr;
    p.proj_out[g] = proj_out ? proj_out[g] : nullptr;
    if(!aligned16(p.Bq[g]) || (p.bias[g] && !aligned16(p.bias[g])) || (p.proj_out[g] && !aligned16(p.proj_out[g])))
      return MARIAN_HIP_ERR_ALIGN;
  }
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  p.A = A; p.aq_out = Aq;
  if(absmax_in) {
    p.partials = absmax_in;
    p.n_partials = kAbsmaxSlots;
  } else {   // nobody left the abs-max of the input: a launch for it
    if(!workspace) return MARIAN_HIP_ERR_NULL;
    if(workspace_bytes < kWorkspaceBytes) return MARIAN_HIP_ERR_WORKSPACE;
    if(!aligned4(workspace)) return MARIAN_HIP_ERR_ALIGN;
    float* partials = reinterpret_cast<float*>(workspace);
    int n_partials = 0;
    const int pst = launch_absmax_partials(A, (size_t)M * (size_t)K, partials, &n_partials, stream);
    if(pst != MARIAN_HIP_OK) return pst;
    p.partials = partials;
    p.n_partials = n_partials;
  }
  p.M = (int)M; p.K = (int)K; p.heads = (int)heads;
  p.k_cache = k_cache; p.v_cache = v_cache; p.batchKV = (unsigned)batchKV;
  p.len = (int)len; p.kv_cap = (int)kv_capacity;
  p.mask = mask; p.n_masks = mask ? (unsigned)n_masks : 1u;
  p.att_scale = att_scale; p.out = out; p.absmax_out = absmax_out;
  constexpr int R = 8;
  const int len4 = ((int)len + 3) & ~3;
  size_t lds = (size_t)32 * (size_t)K + (size_t)n_proj * 8 * R * 128 + (size_t)n_proj * R * 64 * 4 +
               (size_t)R * (size_t)(len4 + 256) * 4;
  {   // the kernels' dynamic LDS limit, raised once per device (one bit per device)
    static std::atomic<uint64_t> lds_done{0};
    int dev = 0;
    MH_HIP(hipGetDevice(&dev));
    if(dev < 0 || dev >= 64) return MARIAN_HIP_ERR_RANGE;
    if(!(lds_done.load(std::memory_order_acquire) & (1ull << dev))) {
      const void* staged[] = {
          reinterpret_cast<const void*>(proj_attention_kernel<1, R, 2, 1>), reinterpret_cast<const void*>(proj_attention_kernel<1, R, 2, 2>),
          reinterpret_cast<const void*>(proj_attention_kernel<1, R, 2, 3>), reinterpret_cast<const void*>(proj_attention_kernel<1, R, 4, 1>),
          reinterpret_cast<const void*>(proj_attention_kernel<1, R, 4, 2>), reinterpret_cast<const void*>(proj_attention_kernel<1, R, 4, 3>)};
      for(const void* f : staged) MH_HIP(hipFuncSetAttribute(f, hipFuncAttributeMaxDynamicSharedMemorySize, kProjMaxLds));
      MH_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(proj_attention_kernel<1, R, 0, 0>),
                                 hipFuncAttributeMaxDynamicSharedMemorySize, 96 * 1024));
      MH_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(proj_attention_kernel<3, R, 0, 0>),
                                 hipFuncAttributeMaxDynamicSharedMemorySize, 96 * 1024));
      lds_done.fetch_or(1ull << dev, std::memory_order_release);
    }
  }
  const ProjRowPlan plan = proj_row_plan(n_proj, M, heads, batchKV, len, kProjStageLen, lds, (size_t)kProjMaxLds);
  p.share_shift = plan.shift;
  p.share_nb = plan.sentences;
  p.share_hyps = plan.hyps;
  p.share_per = plan.per_wg;
  p.stage_kv = plan.stage;
  if(plan.blocks_y > 65535) return MARIAN_HIP_ERR_RANGE;
  if(plan.stage) lds += (size_t)(2 << plan.shift) * (size_t)len * 256;
  const dim3 grid((unsigned)heads, (unsigned)plan.blocks_y);
#define MH_PA(NP, SEGS, PASSES) \
  hipLaunchKernelGGL((proj_attention_kernel<NP, R, SEGS, PASSES>), grid, dim3(kProjThreads), lds, st, p)
  if(n_proj == 3) MH_PA(3, 0, 0);
  else if(!p.stage_kv) MH_PA(1, 0, 0);
  else {
    const int passes = ((int)len + 31) / 32;   // 1 .. 3
    if(p.share_shift == 0) {   // one sentence per workgroup
      if(passes == 1) MH_PA(1, 2, 1);
      else if(passes == 2) MH_PA(1, 2, 2);
      else MH_PA(1, 2, 3);
    } else {
      if(passes == 1) MH_PA(1, 4, 1);
      else if(passes == 2) MH_PA(1, 4, 2);
      else MH_PA(1, 4, 3);
    }
  }
#undef MH_PA
  MH_HIP(hipGetLastError());
  return MARIAN_HIP_OK;
}

int marian_hip_nbest(const float* scores, int64_t dimBatch, int64_t rowLen, int64_t N,
                     float* outScores, uint32_t* outKeys, void* stream) {
  if(dimBatch < 0 || rowLen <= 0 || N <= 0 || N > kNbestMax || N > rowLen) return MARIAN_HIP_ERR_SHAPE;
  if(dimBatch == 0) return MARIAN_HIP_OK;
  if(!scores || !outScores || !outKeys) return MARIAN_HIP_ERR_NULL;
  if(dimBatch * rowLen > 4294967295LL) return MARIAN_HIP_ERR_RANGE;   // keys are uint32
  if(!aligned4(scores) || !aligned4(outScores) || !aligned4(outKeys)) return MARIAN_HIP_ERR_ALIGN;
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  if(N <= 4)
    hipLaunchKernelGGL(nbest_kernel<4>, dim3((unsigned)dimBatch), dim3(1024), 0, st, scores, (long long)rowLen, (int)N, outScores, outKeys);
  else if(N <= 8)
    hipLaunchKernelGGL(nbest_kernel<8>, dim3((unsigned)dimBatch), dim3(1024), 0, st, scores, (long long)rowLen, (int)N, outScores, outKeys);
  else
    hipLaunchKernelGGL(nbest_kernel<16>, dim3((unsigned)dimBatch), dim3(1024), 0, st, scores, (long long)rowLen, (int)N, outScores, outKeys);
  MH_HIP(hipGetLastError());
  return MARIAN_HIP_OK;
}

int marian_hip_fill(void* begin, int64_t count, int elem_bytes, uint64_t pattern, void* stream) {
  if(count < 0 || (elem_bytes != 1 && elem_bytes != 2 && elem_bytes != 4 && elem_bytes != 8))
    return MARIAN_HIP_ERR_SHAPE;
  if(count == 0) return MARIAN_HIP_OK;
  if(!begin) return MARIAN_HIP_ERR_NULL;
  if(reinterpret_cast<uintptr_t>(begin) % (uintptr_t)elem_bytes != 0) return MARIAN_HIP_ERR_ALIGN;
  if(count > (int64_t)(0x7FFFFFFFFFFFFFFFll / 8)) return MARIAN_HIP_ERR_RANGE;
  const long long bytes = (long long)count * elem_bytes;
  long long head = (long long)((16 - reinterpret_cast<uintptr_t>(begin) % 16) % 16);
  if(head > bytes) head = bytes;
  const long long vecs = (bytes - head) / 16;
  long long blocks = (vecs + 255) / 256;
  if(blocks < 1) blocks = 1;
  if(blocks > 4096) blocks = 4096;
  hipLaunchKernelGGL(fill_kernel, dim3((unsigned)blocks), dim3(256), 0, reinterpret_cast<hipStream_t>(stream),
                     reinterpret_cast<unsigned char*>(begin), bytes, head, vecs, elem_bytes,
                     (unsigned long long)pattern);
  MH_HIP(hipGetLastError());
  return MARIAN_HIP_OK;
}

size_t marian_hip_nbest_beams_workspace_bytes(int64_t beam, int64_t dimBatch, int64_t vocab, int64_t N) {
  if(beam <= 0 || dimBatch <= 0 || vocab <= 0 || N <= 0 || N > kNbestMax) return 0;
  const NbestPlan plan = nbest_plan(beam, dimBatch, vocab, N);
  return kNbestCounterBytes + (size_t)dimBatch * plan.parts * N * 8;
}

int marian_hip_nbest_beams_workspace_init(void* workspace, size_t workspace_bytes, void* stream) {
  if(workspace_bytes == 0) return MARIAN_HIP_OK;
  if(!workspace) return MARIAN_HIP_ERR_NULL;
  if(!aligned4(workspace)) return MARIAN_HIP_ERR_ALIGN;
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  const long long words = (long long)(workspace_bytes / 4);
  const unsigned blocks = (unsigned)((words + 255) / 256 < 1024 ? (words + 255) / 256 : 1024);
  if(words > 0)
    hipLaunchKernelGGL(zero_words_kernel, dim3(blocks), dim3(256), 0, st, reinterpret_cast<unsigned*>(workspace), words);
  MH_HIP(hipGetLastError());
  return MARIAN_HIP_OK;
}

int marian_hip_nbest_beams(const float* scores, int64_t beam, int64_t dimBatch, int64_t vocab, int64_t N,
                           float* outScores, uint32_t* outKeys, void* workspace, size_t workspace_bytes,
                           void* stream) {
  if(beam <= 0 || dimBatch < 0 || vocab <= 0 || N <= 0 || N > kNbestMax || N > beam * vocab)
    return MARIAN_HIP_ERR_SHAPE;
  if(beam * N > 1024) return MARIAN_HIP_ERR_SHAPE;
  if(dimBatch == 0) return MARIAN_HIP_OK;
  if(!scores || !outScores || !outKeys || !workspace) return MARIAN_HIP_ERR_NULL;
  if(dimBatch * beam * vocab > 4294967295LL || dimBatch > kNbestMaxBatch) return MARIAN_HIP_ERR_RANGE;   // keys are uint32
  if(!aligned4(scores) || !aligned4(outScores) || !aligned4(outKeys) || !aligned4(workspace))
    return MARIAN_HIP_ERR_ALIGN;
  const NbestPlan plan = nbest_plan(beam, dimBatch, vocab, N);
  const size_t entries = (size_t)dimBatch * plan.parts * N;
  if(workspace_bytes < kNbestCounterBytes + entries * 8) return MARIAN_HIP_ERR_WORKSPACE;
  // layout: the counters (one per batch entry, zero between calls) in a region of fixed size, so
  // that no call's candidates ever land on another call's counters; then candidate scores and
  // candidate positions
  unsigned* counters = reinterpret_cast<unsigned*>(workspace);
  float* candVal = reinterpret_cast<float*>(counters + kNbestMaxBatch * kNbestCounterStride);
  unsigned* candIdx = reinterpret_cast<unsigned*>(candVal + entries);
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  const dim3 grid((unsigned)plan.parts, (unsigned)dimBatch);
#define MH_NBP(KEEP, FENCED)                                                                                   \
  hipLaunchKernelGGL((nbest_part_kernel<KEEP, FENCED>), grid, dim3(1024), 0, st, scores, (long long)dimBatch, \
                     (long long)vocab, plan.perSeg, plan.sliceLen, (int)N, candVal, candIdx, counters,         \
                     outScores, outKeys)
  if(nbest_fenced()) {
#ifdef MARIAN_HIP_TUNING
    if(N <= 4) MH_NBP(4, true);
    else if(N <= 8) MH_NBP(8, true);
    else MH_NBP(16, true);
#endif
  } else {
    if(N <= 4) MH_NBP(4, false);
    else if(N <= 8) MH_NBP(8, false);
    else MH_NBP(16, false);
  }
#undef MH_NBP
  MH_HIP(hipGetLastError());
  return MARIAN_HIP_OK;
}

int marian_hip_logsoftmax_nbest_beams(const float* logits, const float* rowAdd, float* logProbs, int64_t beam,
                                      int64_t dimBatch, int64_t vocab, int64_t N, float* outScores,
                                      uint32_t* outKeys, void* workspace, size_t workspace_bytes, void* stream) {
  if(beam <= 0 || dimBatch < 0 || vocab <= 0 || N <= 0 || N > kNbestMax || N > vocab) return MARIAN_HIP_ERR_SHAPE;
  // (a row in the registers of one workgroup, and the sizes for which marian_hip_logsoftmax takes the
  // same row computation, softmax_wide_kernel<true, 1024, 8>: the results are to be the same bits)
  if(beam * N > 1024 || (vocab % 4) != 0 || vocab <= 4096 || vocab > 32768) return MARIAN_HIP_ERR_SHAPE;
  if(dimBatch == 0) return MARIAN_HIP_OK;
  if(!logits || !outScores || !outKeys || !workspace) return MARIAN_HIP_ERR_NULL;
  if(dimBatch * beam * vocab > 4294967295LL || dimBatch > kNbestMaxBatch) return MARIAN_HIP_ERR_RANGE;   // keys are uint32
  if(!aligned16(logits) || (logProbs && !aligned16(logProbs)) || (rowAdd && !aligned4(rowAdd)) ||
     !aligned4(outScores) || !aligned4(outKeys) || !aligned4(workspace))
    return MARIAN_HIP_ERR_ALIGN;
  const size_t entries = (size_t)dimBatch * beam * N;
  if(workspace_bytes < kNbestCounterBytes + entries * 8) return MARIAN_HIP_ERR_WORKSPACE;
  // (the layout of marian_hip_nbest_beams with one part per beam entry)
  unsigned* counters = reinterpret_cast<unsigned*>(workspace);
  float* candVal = reinterpret_cast<float*>(counters + kNbestMaxBatch * kNbestCounterStride);
  unsigned* candIdx = reinterpret_cast<unsigned*>(candVal + entries);
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  const dim3 grid((unsigned)beam, (unsigned)dimBatch);
#define MH_LSNB(VPT, KEEP, FENCED)                                                                                   \
  hipLaunchKernelGGL((logsoftmax_nbest_kernel<VPT, KEEP, FENCED>), grid, dim3(1024), 0, st, logits, rowAdd, logProbs, \
                     (long long)dimBatch, (int)vocab, (int)N, candVal, candIdx, counters, outScores, outKeys)
  if(nbest_fenced()) {
#ifdef MARIAN_HIP_TUNING
    if(N <= 4) MH_LSNB(8, 4, true);
    else if(N <= 8) MH_LSNB(8, 8, true);
    else MH_LSNB(8, 16, true);
#endif
  } else {
    if(N <= 4) MH_LSNB(8, 4, false);
    else if(N <= 8) MH_LSNB(8, 8, false);
    else MH_LSNB(8, 16, false);
  }
#undef MH_LSNB
  MH_HIP(hipGetLastError());
  return MARIAN_HIP_OK;
}

}  // extern "C"
