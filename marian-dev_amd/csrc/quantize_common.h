// Device helpers of the quantizers: the int8 rounding and packing, wave and workgroup maxima, the
// quantMult, and the layout of the workspace.  Shared by every translation unit that quantizes.
#pragma once

#include "int8_common.h"

namespace marian_hip {

constexpr int kQuantThreads = 256;
constexpr int kMaxPartials = 1024;                  // floats of workspace used by the two-pass forms
// Workspace layout: [0, 4 KB) abs-max partials of the two-pass forms; then the hand-over area of the
// one-pass prepareA: 256 arrival slots of 8 bytes (a cache line each made no difference: 23.8 us
// either way for 4096 x 4096), one generation word, and 16 mailboxes 256 bytes apart.
constexpr int kOnePassMaxGroups = 256;              // workgroups of the one-pass form (one per CU)
constexpr int kOnePassMailboxes = 16;
constexpr int kOnePassStride = 1;                   // 8-byte words between two slots
constexpr size_t kOnePassSlotsOffset = kMaxPartials * sizeof(float);
constexpr size_t kOnePassGenOffset = kOnePassSlotsOffset + kOnePassMaxGroups * kOnePassStride * 8;
constexpr size_t kOnePassMailOffset = 8192;
constexpr size_t kWorkspaceBytes = kOnePassMailOffset + kOnePassMailboxes * 256;   // 12 KB
static_assert(kOnePassGenOffset + 8 <= kOnePassMailOffset, "workspace layout");
constexpr int kSingleBlockThreads = 1024;
constexpr int kSingleBlockMaxElems = 32 * 1024;     // one workgroup does abs-max and quantize (beyond: 8.6 us against 6.4 us for two launches)

// q = clamp(rne(fl32(x * qm)), -127, 127); products that are NaN or outside int32 give -127
// (x86 cvtps2dq integer-indefinite followed by saturating packs and max(-127)).
__device__ __forceinline__ int quantize_one(float x, float qm) {
  float v = x * qm;
  float r = __builtin_rintf(v);
  r = fminf(fmaxf(r, -127.0f), 127.0f);
  int q = (int)r;
  return (fabsf(v) < 2147483648.0f) ? q : -127;
}

// The value whose rounding to nearest-even is quantize_one(x, qm): clamping to [-127, 127] first
// commutes with rounding (the bounds are integers; med3 returns -127 for NaN).  Products >= 2^31
// (only possible for non-finite inputs) follow the x86 conversion and give -127.
__device__ __forceinline__ float quantize_clamped(float x, float qm) {
  const float v = x * qm;
  const float c = __builtin_amdgcn_fmed3f(v, -127.0f, 127.0f);
  return (v >= 2147483648.0f) ? -127.0f : c;
}

// Four clamped products -> four int8 in one word.  Adding 1.5 * 2^23 rounds to nearest-even and
// leaves the integer in the low byte of the sum; the SDWA form of the add writes that low byte
// straight into byte 0..3 of the destination, so no byte shuffles are needed afterwards.
__device__ __forceinline__ uint32_t round_pack4(float c0, float c1, float c2, float c3) {
  const float magic = 12582912.0f;
  uint32_t q;
  asm("v_add_f32_sdwa %0, %1, %2 dst_sel:BYTE_0 dst_unused:UNUSED_PAD src0_sel:DWORD src1_sel:DWORD"
      : "=v"(q) : "v"(c0), "v"(magic));
  asm("v_add_f32_sdwa %0, %1, %2 dst_sel:BYTE_1 dst_unused:UNUSED_PRESERVE src0_sel:DWORD src1_sel:DWORD"
      : "+v"(q) : "v"(c1), "v"(magic));
  asm("v_add_f32_sdwa %0, %1, %2 dst_sel:BYTE_2 dst_unused:UNUSED_PRESERVE src0_sel:DWORD src1_sel:DWORD"
      : "+v"(q) : "v"(c2), "v"(magic));
  asm("v_add_f32_sdwa %0, %1, %2 dst_sel:BYTE_3 dst_unused:UNUSED_PRESERVE src0_sel:DWORD src1_sel:DWORD"
      : "+v"(q) : "v"(c3), "v"(magic));
  return q;
}

// Fast form for the usual case (finite quantMult): every product lies within
// [-127.0001, 127.0001], so the out-of-range check of quantize_clamped can never fire (med3
// still maps a NaN among the values to -127).
__device__ __forceinline__ uint32_t quantize_pack4_finite(v4f x, float qm) {
  return round_pack4(__builtin_amdgcn_fmed3f(x.x * qm, -127.0f, 127.0f),
                     __builtin_amdgcn_fmed3f(x.y * qm, -127.0f, 127.0f),
                     __builtin_amdgcn_fmed3f(x.z * qm, -127.0f, 127.0f),
                     __builtin_amdgcn_fmed3f(x.w * qm, -127.0f, 127.0f));
}

__device__ __forceinline__ uint32_t quantize_pack4(v4f x, float qm) {
  return round_pack4(quantize_clamped(x.x, qm), quantize_clamped(x.y, qm), quantize_clamped(x.z, qm),
                     quantize_clamped(x.w, qm));
}

__device__ __forceinline__ float abs4max(v4f x, float m) {
  m = fmaxf(m, fabsf(x.x));
  m = fmaxf(m, fabsf(x.y));
  m = fmaxf(m, fabsf(x.z));
  m = fmaxf(m, fabsf(x.w));
  return m;
}

// Max over each row of 16 lanes, left in all 16 of them: four DPP steps (the two lane swaps within
// a quad, the mirror within half a row and within the row).  All lanes of the wave must be active.
// (fmaxf passes over NaN operands whatever the order, so the result does not depend on the order.)
__device__ __forceinline__ float row16_max(float m) {
  m = fmaxf(m, __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, m), 0xB1, 0xF, 0xF, false)));   // quad_perm [1,0,3,2]
  m = fmaxf(m, __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, m), 0x4E, 0xF, 0xF, false)));   // quad_perm [2,3,0,1]
  m = fmaxf(m, __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, m), 0x141, 0xF, 0xF, false)));  // row_half_mirror
  m = fmaxf(m, __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, m), 0x140, 0xF, 0xF, false)));  // row_mirror
  return m;
}
// Max over the wave, in all lanes: within the rows, then across them with the two row-broadcast
// DPP steps (rows 1 and 3 take in the last lane of the row before them, then rows 2 and 3 the last
// lane of row 1), which leaves the result in lane 63, read from there as a scalar.  No step goes
// through the LDS crossbar (a lane exchange there costs ten times a DPP step, and these reductions
// sit between the arrival of the activations and their quantization in every fused call).  All
// lanes of the wave must be active.
__device__ __forceinline__ float wave_max(float m) {
  m = row16_max(m);
  m = fmaxf(m, __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, m), __builtin_bit_cast(int, m), 0x142, 0xA, 0xF, false)));   // row_bcast:15
  m = fmaxf(m, __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, m), __builtin_bit_cast(int, m), 0x143, 0xC, 0xF, false)));   // row_bcast:31
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, m), 63));
}

// Max over the workgroup (whole waves, at most 16 of them); every thread returns the result.
// red: >= blockDim/64 floats of LDS.
__device__ __forceinline__ float block_max(float m, float* red) {
  m = wave_max(m);
  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
  const int nw = blockDim.x / kWave;
  __syncthreads();
  if(lane == 0) red[wave] = m;
  __syncthreads();
  // every row of 16 lanes reads all the wave maxima, so the rows need no exchange afterwards
  const float r = (lane % 16 < nw) ? red[lane % 16] : 0.0f;
  return row16_max(r);
}

// quantMult = 127.0f / maxabs as one correctly rounded fp32 division (via double).
__device__ __forceinline__ float quant_mult_from_maxabs(float maxabs) {
  return (float)(127.0 / (double)maxabs);
}

}  // namespace marian_hip
