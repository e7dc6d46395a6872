// Shared device helpers for the gfx950 int8 affine kernels.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "operand_addressing.h"

namespace marian_hip {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef float v4f __attribute__((ext_vector_type(4)));

constexpr int kWave = 64;        // CDNA wavefront
constexpr int kFragBytes = 1024; // one MFMA 16x16x64 i8 operand: 64 lanes x 16 bytes

// D[i][j] += sum_k A[i][k] * B[j][k] over 64 values of k.  Lane l supplies 16 consecutive
// bytes of row (l % 16) of each operand, taken at byte offset (l / 16) * 16 of the 64-byte
// K slab; both operands use the same lane->k assignment, so the sum is independent of how the
// hardware orders k internally.  Lane l receives D[4 * (l / 16) + r][l % 16] in element r.
__device__ __forceinline__ v4i mfma_i8_16x16x64(v4i a, v4i b, v4i c) {
  return __builtin_amdgcn_mfma_i32_16x16x64_i8(a, b, c, 0, 0, 0);
}

__device__ __forceinline__ v4i load16(const int8_t* p) {
  return *reinterpret_cast<const v4i*>(p);
}

// (the prepared weight order and every operand offset of the kernels: operand_addressing.h)

// quantMult stored behind `elements` int8 values (reference
// src/tensors/cpu/integer_common.h:101-106).
__device__ __forceinline__ float tail_quant_mult(const int8_t* q, size_t elements) {
  return *reinterpret_cast<const float*>(q + elements);
}

// unquant_mult of reference src/tensors/cpu/intgemm_interface.h:69-70: fl32(1/fl32(a*b)) then
// * scale.  The reciprocal goes through double so it is the correctly rounded fp32 quotient.
__device__ __forceinline__ float unquant_mult(float aqm, float bqm, float scale) {
  float prod = aqm * bqm;
  float inv = (float)(1.0 / (double)prod);
  return inv * scale;
}

// Epilogue for the four accumulators a lane owns: rows n .. n+3 of one activation row m.
//   y = float(acc) * unquant (+ bias) ; relu: y > 0 ? y : 0
// mul and add stay separate roundings like the CPU callbacks (compiled with
// -ffp-contract=off).  n is a multiple of 4 and n_out a multiple of 8, so the four values are
// either all inside or all outside the output.
struct Epilogue {
  float unquant;
  const float* bias;     // may be null
  const uint32_t* idx;   // shortlist ids or null; bias is gathered through it
  int relu;
  int dump;              // store raw int32 accumulators instead
  void* out;             // float* or int32_t*
  int M;
  int n_out;             // columns of the output matrix (N, or shortlist length)

  __device__ __forceinline__ void store(v4i acc, int m, int n) const {
    if(m >= M || n >= n_out) return;
    size_t off = (size_t)m * (size_t)n_out + (size_t)n;
    if(dump) {
      *reinterpret_cast<v4i*>(reinterpret_cast<int32_t*>(out) + off) = acc;
      return;
    }
    v4f y;
    y.x = (float)acc.x * unquant;
    y.y = (float)acc.y * unquant;
    y.z = (float)acc.z * unquant;
    y.w = (float)acc.w * unquant;
    if(bias) {
      if(idx) {
        y.x = y.x + bias[idx[n + 0]];
        y.y = y.y + bias[idx[n + 1]];
        y.z = y.z + bias[idx[n + 2]];
        y.w = y.w + bias[idx[n + 3]];
      } else {
        y.x = y.x + bias[n + 0];
        y.y = y.y + bias[n + 1];
        y.z = y.z + bias[n + 2];
        y.w = y.w + bias[n + 3];
      }
    }
    if(relu) {
      y.x = y.x > 0.0f ? y.x : 0.0f;
      y.y = y.y > 0.0f ? y.y : 0.0f;
      y.z = y.z > 0.0f ? y.z : 0.0f;
      y.w = y.w > 0.0f ? y.w : 0.0f;
    }
    *reinterpret_cast<v4f*>(reinterpret_cast<float*>(out) + off) = y;
  }
};

// Arguments common to both GEMM kernel families.
struct GemmArgs {
  const int8_t* Aq;     // [M x K] + tail
  const int8_t* Bq;     // K*N bytes, K-blocked (see b_chunk_offset) + tail
  const float* bias;    // [N] or null
  const uint32_t* idx;  // [n_out] or null
  void* out;            // [M x n_out] fp32 (or int32 when dump)
  int M, K, N, n_out;
  float scale;
  int relu, dump;
#ifdef MARIAN_HIP_TUNING
  int dbg = 0;  // measurement switches (bit 0: no refetch, bit 1: no stores)
  long long* prof = nullptr;  // per-workgroup phase clocks
#endif
  // kAbsmaxSlots floats that receive values whose maximum is max|out| (the next call's abs-max,
  // taken where the tensor is produced), or null
  float* absmax_out = nullptr;
  int absmax_used = 0;   // large-M launches: how many slots the launch fills (one per workgroup)
  // write the output with non-temporal stores (set by the launchers for outputs of several MB,
  // which would otherwise sit dirty in L2 until the kernel ends and be written back then)
  int stream_out = 0;
};

constexpr int kAbsmaxSlots = 2048;

// The tuning build (-DMARIAN_HIP_TUNING, libmarian_hip_int8_tuning.so) carries measurement switches
// and per-workgroup phase clocks in the kernels; the shipped library compiles them out.
#ifdef MARIAN_HIP_TUNING
#define MH_DBG(args, bit) ((args).dbg & (bit))
#define MH_PROF(args) ((args).prof)
#define MH_CLOCK() clock64()
#define MH_WALL() wall_clock64()
#else
#define MH_DBG(args, bit) 0
#define MH_PROF(args) (static_cast<long long*>(nullptr))
#define MH_CLOCK() 0ll
#define MH_WALL() 0ll
#endif

__device__ __forceinline__ Epilogue make_epilogue(const GemmArgs& a) {
  Epilogue e;
  if(a.dump) {
    e.unquant = 0.0f;
  } else {
    float aqm = tail_quant_mult(a.Aq, (size_t)a.M * (size_t)a.K);
    float bqm = tail_quant_mult(a.Bq, (size_t)a.K * (size_t)a.N);
    e.unquant = unquant_mult(aqm, bqm, a.scale);
  }
  e.bias = a.bias;
  e.idx = a.idx;
  e.relu = a.relu;
  e.dump = a.dump;
  e.out = a.out;
  e.M = a.M;
  e.n_out = a.n_out;
  return e;
}

}  // namespace marian_hip
