/*
 * marian_hip_int16.h - C ABI of the 16-bit intgemm path (Marian Type::intgemm16) on gfx950.
 *
 * Same library and conventions as marian_hip_int8.h (device pointers, caller-owned buffers,
 * nothing retained, work enqueued on `stream`, status codes, no synchronisation).
 *
 * Quantized tensor layout (reference src/common/types.cpp:32-34 and
 * src/tensors/cpu/integer_common.h:101-106 with Integer = int16_t): `elements` int16 values
 * followed by one fp32 quantMult at byte offset 2 * elements.  The quantMult of every 16-bit tensor
 * is 1024 (src/tensors/cpu/integer_common.h:174-175), for activations and weights alike.
 *   activations  Aq : int16 row-major [M x K]        + tail  (2*M*K + 4 bytes)
 *   weights      Bq : int16 row-major [N x K] = W^T  + tail  (2*K*N + 4 bytes), the payload of a
 *                     Type::intgemm16 item of a .bin model file
 *                     (src/tensors/cpu/expression_graph_packable.h:203-235,242-250).
 * Shape rules: K % 32 == 0, N % 8 == 0.  Alignment: 16 bytes for matrices, 4 for the bias.
 *
 * gfx950 has no 16-bit integer matrix instruction; the products are taken with v_dot2_i32_i16 on
 * the vector units (two int16 products and the accumulator summed mod 2^32, which is what the
 * CPU's pmaddwd + paddd compute).  The path is exact, not fast: the 8-bit path is the one the
 * matrix cores serve.
 */
#ifndef MARIAN_HIP_INT16_H
#define MARIAN_HIP_INT16_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/*
 * Replaces the prepareA node body for a 16-bit weight type, reference
 * src/tensors/cpu/intgemm_interface.h:19-29: quantMult 1024 (no abs-max pass), Kernels16::PrepareA,
 * tail store.  q = saturate_int16(rne(fl32(a * 1024))).  Aq: 2*M*K + 4 bytes.
 */
int marian_hip_int16_prepare_a(const float* A, int16_t* Aq, int64_t M, int64_t K, void* stream);

/*
 * Replaces the 16-bit branch of the offline packer, reference
 * src/tensors/cpu/expression_graph_packable.h:203-235: quantMult 1024, Transpose10, Int16::PrepareA
 * on the transpose, tail at byte 2*K*N.  W: fp32 [K x N].  Bq: 2*K*N + 4 bytes.
 */
int marian_hip_int16_prepare_b(const float* W, int16_t* Bq, int64_t K, int64_t N, void* stream);

/*
 * Replaces prepareAndTransposeB<intgemm16>, reference src/tensors/cpu/integer_common.h:189-216 and
 * src/common/binary.cpp:108-110: the file payload is the GPU layout, so this is a copy of
 * 2*K*N + 4 bytes.  K % 32 == 0, N % 8 == 0; in == out is a no-op, buffers that overlap in part
 * return MARIAN_HIP_ERR_ALIAS.
 */
int marian_hip_int16_prepare_b_quantized_transposed(const int16_t* in, int16_t* out, int64_t K, int64_t N,
                                                    void* stream);

/*
 * Replaces the multiply node body for 16-bit operands, reference
 * src/tensors/cpu/intgemm_interface.h:60-88 (Kernels16::Multiply with UnquantizeAndWrite or
 * UnquantizeAndAddBiasAndWrite): unquant = (1.0f / (aqm * bqm)) * scale with both quantMults read
 * from the tails on the device; out[m,n] = float(acc[m,n]) * unquant (+ bias[n]); relu != 0 fuses
 * the ReLU node of src/graph/expression_operators.cpp:721-731.  out: fp32 [M x N].
 */
int marian_hip_int16_affine(const int16_t* Aq, const int16_t* Bq, const float* bias, float* out, int64_t M,
                            int64_t K, int64_t N, float scale, int relu, void* stream);

/* Parity hook: the int32 accumulators (sums mod 2^32) Kernels16::Multiply hands to its callback. */
int marian_hip_int16_multiply_i32(const int16_t* Aq, const int16_t* Bq, int32_t* acc, int64_t M, int64_t K,
                                  int64_t N, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* MARIAN_HIP_INT16_H */
