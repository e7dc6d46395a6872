// The 16-bit intgemm path (Type::intgemm16): quantizers, a dot2-based GEMM and its C ABI.
// Declarations and the reference call sites each entry point replaces: include/marian_hip_int16.h
#include "../../include/marian_hip_int16.h"

#include <hip/hip_runtime.h>

#include "../../include/marian_hip_int8.h"
#include "abi_common.h"
#include "int8_common.h"

using namespace marian_hip;

namespace {

typedef short v2s __attribute__((ext_vector_type(2)));

constexpr int64_t kMaxElems16 = 2147483647LL;
constexpr float kQuantMult16 = 1024.0f;   // reference src/tensors/cpu/integer_common.h:174-175

#define MH_HIP(expr)                                       \
  do {                                                     \
    hipError_t e_ = (expr);                                \
    if(e_ != hipSuccess) return record_hip_error((int)e_); \
  } while(0)

inline bool aligned(const void* p, size_t a) { return (reinterpret_cast<uintptr_t>(p) % a) == 0; }

// q = saturate_int16(rne(fl32(x * qm))); a product that is NaN or not below 2^31 gives -32768
// (x86 cvtps2dq "integer indefinite" INT_MIN, then packssdw); products at or below -2^31 saturate
// to -32768 anyway.  med3 returns the smallest operand when one is NaN.
__device__ __forceinline__ int quantize16_one(float x, float qm) {
  const float v = x * qm;
  const float c = __builtin_amdgcn_fmed3f(v, -32768.0f, 32767.0f);
  return (int)__builtin_rintf(v >= 2147483648.0f ? -32768.0f : c);
}
__device__ __forceinline__ uint32_t quantize16_pair(float x0, float x1, float qm) {
  return ((uint32_t)quantize16_one(x0, qm) & 0xFFFFu) | ((uint32_t)quantize16_one(x1, qm) << 16);
}

// prepareA: elementwise, eight values (two 16-byte loads, one 16-byte store) per thread and step
__global__ __launch_bounds__(256) void quantize16_a_kernel(const float* __restrict__ x, size_t n8,
                                                           int16_t* __restrict__ out) {
  const v4f* x4 = reinterpret_cast<const v4f*>(x);
  uint4* o = reinterpret_cast<uint4*>(out);
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  for(size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n8; i += stride) {
    const v4f a = x4[2 * i], b = x4[2 * i + 1];
    uint4 q;
    q.x = quantize16_pair(a.x, a.y, kQuantMult16);
    q.y = quantize16_pair(a.z, a.w, kQuantMult16);
    q.z = quantize16_pair(b.x, b.y, kQuantMult16);
    q.w = quantize16_pair(b.z, b.w, kQuantMult16);
    o[i] = q;
  }
  if(blockIdx.x == 0 && threadIdx.x == 0) *reinterpret_cast<float*>(out + n8 * 8) = kQuantMult16;
}

// prepareB: W fp32 [K x N] -> payload int16 [N x K].  A workgroup transposes a 32(k) x 64(n) tile
// through LDS: reads coalesced along n, writes 16-byte runs along k (K % 32 == 0).
__global__ __launch_bounds__(256) void quantize16_b_transpose_kernel(const float* __restrict__ W, int K, int N,
                                                                      int16_t* __restrict__ out) {
  __shared__ uint32_t tile[64][17];   // [n][k / 2] packed pairs, 17 dwords per row
  const int n0 = blockIdx.x * 64, k0 = blockIdx.y * 32;
  const int tn = threadIdx.x % 64, tk = threadIdx.x / 64;   // wave tk takes k rows 8*tk .. 8*tk+7
  const int n_in = n0 + tn;
#pragma unroll
  for(int g = 0; g < 4; ++g) {
    const int kk = tk * 8 + g * 2;
    float w0 = 0.0f, w1 = 0.0f;
    if(n_in < N) {
      w0 = W[(size_t)(k0 + kk) * N + n_in];
      w1 = W[(size_t)(k0 + kk + 1) * N + n_in];
    }
    tile[tn][kk / 2] = quantize16_pair(w0, w1, kQuantMult16);
  }
  __syncthreads();
  // 64 rows (n) x 64 bytes (32 k): 4 threads per row, 16 bytes each
  const int rn = threadIdx.x / 4, c4 = (threadIdx.x % 4) * 4;
  const int n = n0 + rn;
  if(n < N) {
    uint4 v;
    v.x = tile[rn][c4]; v.y = tile[rn][c4 + 1]; v.z = tile[rn][c4 + 2]; v.w = tile[rn][c4 + 3];
    *reinterpret_cast<uint4*>(out + (size_t)n * K + k0 + c4 * 2) = v;
  }
  if(blockIdx.x == 0 && blockIdx.y == 0 && threadIdx.x == 0)
    *reinterpret_cast<float*>(out + (size_t)K * N) = kQuantMult16;
}

// C[m, n] = sum_k A[m, k] * B[n, k] over int16 operands, both K-contiguous.  A workgroup of 256
// threads owns a 64 x 64 tile of the output and walks K in blocks of 64 values (128 bytes per row)
// staged in LDS as packed pairs, 33 dwords per row (conflict-free for the strided reads); thread
// (ty, tx) accumulates the 4 x 4 outputs of rows ty + 16 i, columns tx + 16 j with v_dot2_i32_i16:
// two products and the accumulator, summed mod 2^32.
template <bool DUMP>
__global__ __launch_bounds__(256) void gemm16_kernel(const int16_t* __restrict__ Aq, const int16_t* __restrict__ Bq,
                                                     const float* __restrict__ bias, void* __restrict__ out,
                                                     int M, int K, int N, float scale, int relu) {
  __shared__ uint32_t As[64][33], Bs[64][33];
  const int tid = threadIdx.x, tx = tid % 16, ty = tid / 16;
  const int m0 = blockIdx.y * 64, n0 = blockIdx.x * 64;
  int acc[4][4];
#pragma unroll
  for(int i = 0; i < 4; ++i)
#pragma unroll
    for(int j = 0; j < 4; ++j) acc[i][j] = 0;
  // staging: 64 rows x 128 bytes per operand = 512 pieces of 16 bytes, two per thread and operand
  const int lr = tid / 8, lc = (tid % 8) * 4;   // row (and row + 32), first dword of the piece
  for(int kb = 0; kb < K; kb += 64) {
    const int kv = (K - kb) >= 64 ? 64 : (K - kb);   // K % 32 == 0: a last block of 32 values
    uint4 ra[2], rb[2];
#pragma unroll
    for(int h = 0; h < 2; ++h) {
      const int r = lr + 32 * h;
      const int am = min(m0 + r, M - 1), bn = min(n0 + r, N - 1);   // rows past the edge: copies, never stored
      const bool in_k = lc * 2 < kv;
      ra[h] = in_k ? *reinterpret_cast<const uint4*>(Aq + (size_t)am * K + kb + lc * 2) : uint4{0, 0, 0, 0};
      rb[h] = in_k ? *reinterpret_cast<const uint4*>(Bq + (size_t)bn * K + kb + lc * 2) : uint4{0, 0, 0, 0};
    }
    __syncthreads();   // the previous block has been read
#pragma unroll
    for(int h = 0; h < 2; ++h) {
      const int r = lr + 32 * h;
      As[r][lc] = ra[h].x; As[r][lc + 1] = ra[h].y; As[r][lc + 2] = ra[h].z; As[r][lc + 3] = ra[h].w;
      Bs[r][lc] = rb[h].x; Bs[r][lc + 1] = rb[h].y; Bs[r][lc + 2] = rb[h].z; Bs[r][lc + 3] = rb[h].w;
    }
    __syncthreads();
#pragma unroll 8
    for(int kk = 0; kk < 32; ++kk) {
      uint32_t a[4], b[4];
#pragma unroll
      for(int i = 0; i < 4; ++i) a[i] = As[ty + 16 * i][kk];
#pragma unroll
      for(int j = 0; j < 4; ++j) b[j] = Bs[tx + 16 * j][kk];
#pragma unroll
      for(int i = 0; i < 4; ++i)
#pragma unroll
        for(int j = 0; j < 4; ++j)
          acc[i][j] = __builtin_amdgcn_sdot2(__builtin_bit_cast(v2s, a[i]), __builtin_bit_cast(v2s, b[j]), acc[i][j], false);
    }
  }
  float unquant = 0.0f;
  if(!DUMP) {
    const float aqm = *reinterpret_cast<const float*>(Aq + (size_t)M * K);
    const float bqm = *reinterpret_cast<const float*>(Bq + (size_t)K * N);
    unquant = unquant_mult(aqm, bqm, scale);
  }
#pragma unroll
  for(int i = 0; i < 4; ++i) {
    const int m = m0 + ty + 16 * i;
    if(m >= M) continue;
#pragma unroll
    for(int j = 0; j < 4; ++j) {
      const int n = n0 + tx + 16 * j;
      if(n >= N) continue;
      const size_t off = (size_t)m * N + n;
      if(DUMP) {
        reinterpret_cast<int32_t*>(out)[off] = acc[i][j];
      } else {
        // y = float(acc) * unquant (+ bias); relu: y > 0 ? y : 0; multiply and add round separately
        float y = (float)acc[i][j] * unquant;
        if(bias) y = y + bias[n];
        if(relu) y = y > 0.0f ? y : 0.0f;
        reinterpret_cast<float*>(out)[off] = y;
      }
    }
  }
}

int check16(const void* Aq, const void* Bq, const void* out, const float* bias, int64_t M, int64_t K, int64_t N) {
  if(M < 0 || K <= 0 || N < 0 || (K % 32) != 0 || (N % 8) != 0) return MARIAN_HIP_ERR_SHAPE;
  if(M == 0 || N == 0) return MARIAN_HIP_OK;
  if(!Aq || !Bq || !out) return MARIAN_HIP_ERR_NULL;
  if(M * K > kMaxElems16 || K * N > kMaxElems16 || M * N > kMaxElems16) return MARIAN_HIP_ERR_RANGE;
  if(!aligned(Aq, 16) || !aligned(Bq, 16) || !aligned(out, 16) || (bias && !aligned(bias, 4))) return MARIAN_HIP_ERR_ALIGN;
  return MARIAN_HIP_OK;
}

template <bool DUMP>
int run16(const int16_t* Aq, const int16_t* Bq, const float* bias, void* out, int64_t M, int64_t K, int64_t N,
          float scale, int relu, void* stream) {
  int st = check16(Aq, Bq, out, bias, M, K, N);
  if(st != MARIAN_HIP_OK) return st;
  if(M == 0 || N == 0) return MARIAN_HIP_OK;
  const dim3 grid((unsigned)((N + 63) / 64), (unsigned)((M + 63) / 64));
  if(grid.y > 65535) return MARIAN_HIP_ERR_RANGE;
  hipLaunchKernelGGL(gemm16_kernel<DUMP>, grid, dim3(256), 0, reinterpret_cast<hipStream_t>(stream), Aq, Bq, bias, out,
                     (int)M, (int)K, (int)N, scale, relu ? 1 : 0);
  MH_HIP(hipGetLastError());
  return MARIAN_HIP_OK;
}

}  // namespace

extern "C" {

int marian_hip_int16_prepare_a(const float* A, int16_t* Aq, int64_t M, int64_t K, void* stream) {
  if(M < 0 || K <= 0 || (K % 32) != 0) return MARIAN_HIP_ERR_SHAPE;
  if(M == 0) return MARIAN_HIP_OK;
  if(!A || !Aq) return MARIAN_HIP_ERR_NULL;
  if(M * K > kMaxElems16) return MARIAN_HIP_ERR_RANGE;
  if(!aligned(A, 16) || !aligned(Aq, 16)) return MARIAN_HIP_ERR_ALIGN;
  const size_t n8 = (size_t)M * (size_t)K / 8;
  size_t blocks = (n8 + 255) / 256;
  if(blocks > 4096) blocks = 4096;
  hipLaunchKernelGGL(quantize16_a_kernel, dim3((unsigned)blocks), dim3(256), 0, reinterpret_cast<hipStream_t>(stream), A, n8, Aq);
  MH_HIP(hipGetLastError());
  return MARIAN_HIP_OK;
}

int marian_hip_int16_prepare_b(const float* W, int16_t* Bq, int64_t K, int64_t N, void* stream) {
  if(K <= 0 || N <= 0 || (K % 32) != 0 || (N % 8) != 0) return MARIAN_HIP_ERR_SHAPE;
  if(!W || !Bq) return MARIAN_HIP_ERR_NULL;
  if(K * N > kMaxElems16) return MARIAN_HIP_ERR_RANGE;
  if(!aligned(W, 4) || !aligned(Bq, 16)) return MARIAN_HIP_ERR_ALIGN;
  const dim3 grid((unsigned)((N + 63) / 64), (unsigned)(K / 32));
  if(grid.y > 65535) return MARIAN_HIP_ERR_RANGE;
  hipLaunchKernelGGL(quantize16_b_transpose_kernel, grid, dim3(256), 0, reinterpret_cast<hipStream_t>(stream), W, (int)K, (int)N, Bq);
  MH_HIP(hipGetLastError());
  return MARIAN_HIP_OK;
}

int marian_hip_int16_prepare_b_quantized_transposed(const int16_t* in, int16_t* out, int64_t K, int64_t N, void* stream) {
  if(!in || !out) return MARIAN_HIP_ERR_NULL;
  if(K <= 0 || N <= 0 || (K % 32) != 0 || (N % 8) != 0) return MARIAN_HIP_ERR_SHAPE;
  if(K * N > 2147483647LL) return MARIAN_HIP_ERR_RANGE;
  if(in == out) return MARIAN_HIP_OK;   // the two orders are the same for 16-bit tensors: nothing to do in place
  // a copy between buffers that overlap only in part has no defined result
  const uintptr_t a0 = reinterpret_cast<uintptr_t>(in), b0 = reinterpret_cast<uintptr_t>(out);
  const uintptr_t bytes = 2 * (uintptr_t)K * (uintptr_t)N + sizeof(float);
  if(a0 < b0 + bytes && b0 < a0 + bytes) return MARIAN_HIP_ERR_ALIAS;
  MH_HIP(hipMemcpyAsync(out, in, 2 * (size_t)K * (size_t)N + sizeof(float), hipMemcpyDeviceToDevice,
                        reinterpret_cast<hipStream_t>(stream)));
  return MARIAN_HIP_OK;
}

int marian_hip_int16_affine(const int16_t* Aq, const int16_t* Bq, const float* bias, float* out, int64_t M, int64_t K,
                            int64_t N, float scale, int relu, void* stream) {
  return run16<false>(Aq, Bq, bias, out, M, K, N, scale, relu, stream);
}

int marian_hip_int16_multiply_i32(const int16_t* Aq, const int16_t* Bq, int32_t* acc, int64_t M, int64_t K, int64_t N,
                                  void* stream) {
  return run16<true>(Aq, Bq, nullptr, acc, M, K, N, 1.0f, 0, stream);
}

}  // extern "C"
