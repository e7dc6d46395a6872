/*
 * marian_hip_int8.h - C ABI of the gfx950 (MI355X) int8 affine/dot backend for Marian.
 *
 * The functions below are the device-side replacements for the intgemm static interface
 * as Marian calls it.  Every pointer is a DEVICE pointer unless stated otherwise, every
 * buffer is owned by the caller (Marian's Allocator slab), nothing is retained between
 * calls, and all work is enqueued on `stream` (a hipStream_t passed as void*; NULL = the
 * default stream).  No function synchronises the stream.
 *
 * Quantized tensor layout (Marian Type::intgemm8, reference src/common/types.cpp:32-34 and
 * src/tensors/cpu/integer_common.h:101-106): `elements` int8 values followed by one fp32
 * quantMult at byte offset `elements`.
 *   activations  Aq : int8 row-major [M x K]            + quantMult tail  (M*K + 4 bytes)
 *   weights      Bq : the K*N int8 values of W^T        + quantMult tail  (K*N + 4 bytes), in one of
 *                     two orders, like the reference's hardware-agnostic and hardware-specific types:
 *     file order     : row-major [N x K], logical B[k, n] at byte n*K + k - the payload of a
 *                      Type::intgemm8 item in a Marian .bin model file
 *                      (src/tensors/cpu/expression_graph_packable.h:160-201,242-250).  No GEMM entry
 *                      point takes it; marian_hip_int8_prepare_b_quantized_transposed converts it.
 *     prepared order : what marian_hip_int8_prepare_b and _prepare_b_quantized_transposed write and
 *                      every GEMM entry point reads ("K-blocked").  K is cut into sub-steps of 32
 *                      values; within a sub-step the N columns follow each other, 32 bytes each:
 *                        byte of B[k, n] = (k/32)*32*N + n*32 + k%32
 *                      (the counterpart of intgemm's own CPU tilings, which the reference produces
 *                      with PrepareBQuantizedTransposed, src/tensors/cpu/integer_common.h:189-216:
 *                      the operand of one gfx950 matrix instruction, 32 columns x 32 values of K,
 *                      is 1 KB of consecutive memory).
 *
 * Shape rules (intgemm's own): K % 64 == 0, N % 8 == 0, shortlist length % 8 == 0.
 * Alignment: A, Aq, Bq, out and acc 16 bytes; bias and idx 4 bytes.
 * M may be any value >= 0 (M == 0 or N == 0 is a no-op).
 *
 * Threads and streams (reference src/translator/translator.h:158-164: one graph and backend per
 * worker thread, several workers may share a device).  Every entry point may be called from any
 * number of host threads at once; the stream is passed per call and calls on different streams
 * may overlap on the device.  What may be shared between overlapping calls and what may not:
 *   - weights, bias, shortlist ids, any input: read only, share freely;
 *   - the workspace (marian_hip_int8_workspace_bytes()): ONE PER STREAM.  It holds the abs-max
 *     partials of the call in flight and the words the workgroups of a one-pass prepareA exchange;
 *     calls on one stream run one after the other and share it, calls on different streams must
 *     each bring their own (a backend object per worker, as in the reference, does that);
 *   - the n-best workspace of marian_hip_nbest_beams / marian_hip_logsoftmax_nbest_beams
 *     (include/marian_hip_ops.h): one per stream, for the same reason (arrival counters);
 *   - the static scratch behind marian_hip_int8_affine_f32_static: one per device, so those calls
 *     must not overlap on a device at all;
 *   - outputs and Aq: whatever the caller's graph guarantees, the library keeps no pointer.
 * The library's own process-wide state is limited to caches that are written once per device
 * (kernel attributes, the number of compute units, the address of the static scratch) and a
 * counter for tags, all atomics; the last HIP error is kept per thread.  A one-pass prepareA
 * puts a workgroup on every compute unit; while another stream keeps compute units busy its
 * workgroups may not all be resident, their waits for one another are bounded, and the call then
 * finishes by the slower route with the same result.
 *
 * Return value: MARIAN_HIP_OK or an error code; a HIP runtime failure returns
 * MARIAN_HIP_ERR_HIP and the hipError_t is available from marian_hip_last_hip_error().
 * Nothing aborts or throws across this boundary; the C++ wrappers turn codes into ABORT.
 */
#ifndef MARIAN_HIP_INT8_H
#define MARIAN_HIP_INT8_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum {
  MARIAN_HIP_OK = 0,
  MARIAN_HIP_ERR_NULL = 1,      /* a required pointer is NULL */
  MARIAN_HIP_ERR_SHAPE = 2,     /* negative size, K % 64, N % 8 or n_idx % 8 violated */
  MARIAN_HIP_ERR_ALIGN = 3,     /* pointer alignment violated */
  MARIAN_HIP_ERR_WORKSPACE = 4, /* workspace too small */
  MARIAN_HIP_ERR_HIP = 5,       /* HIP runtime error, see marian_hip_last_hip_error() */
  MARIAN_HIP_ERR_RANGE = 6,     /* size exceeds what the kernels index (2^31 - 1 elements) */
  MARIAN_HIP_ERR_STATIC_LIMIT = 7, /* M * K exceeds MARIAN_HIP_STATIC_MAX_ELEMS (static-scratch entry point) */
  MARIAN_HIP_ERR_ALIAS = 8      /* input and output overlap where the call cannot work in place */
};

/* Human-readable text for a status code (host pointer, static storage). */
const char* marian_hip_status_string(int status);

/* hipError_t of the last MARIAN_HIP_ERR_HIP on the calling thread (0 if none). */
int marian_hip_last_hip_error(void);

/* ABI version of this header; bumped when a signature changes. */
int marian_hip_int8_abi_version(void);

/* Bytes of device workspace marian_hip_int8_prepare_a / _prepare_b need (a constant). */
size_t marian_hip_int8_workspace_bytes(void);

/*
 * Replaces the prepareA node body, reference src/tensors/cpu/intgemm_interface.h:19-29:
 *   computeQuantMult (integer_common.h:169-173, intgemm::MaxAbsolute), Kernels8::PrepareA
 *   (quantize) and the getQuantMult(out) = quantMult store.
 * A: fp32 [M x K].  Aq: M*K + 4 bytes, receives payload and quantMult tail.
 * quantMult = 127.0f / max|A|; q = clamp(rne(fl32(a * quantMult)), -127, 127).
 */
int marian_hip_int8_prepare_a(const float* A, int8_t* Aq, int64_t M, int64_t K,
                              void* workspace, size_t workspace_bytes, void* stream);

/*
 * Replaces the intgemm8 branch of the offline packer, reference
 * src/tensors/cpu/expression_graph_packable.h:160-201: quantMult over the untransposed fp32
 * W [K x N], Transpose10, Int8::PrepareA on the transpose, quantMult stored at byte K*N.
 * Bq: K*N + 4 bytes, receives the payload in prepared order and the tail.
 */
int marian_hip_int8_prepare_b(const float* W, int8_t* Bq, int64_t K, int64_t N,
                              void* workspace, size_t workspace_bytes, void* stream);

/*
 * Replaces prepareAndTransposeB<intgemm8>, reference
 * src/tensors/cpu/integer_common.h:189-216 (Kernels8::PrepareBQuantizedTransposed + tail
 * copy), which re-tiles the file payload for the CPU it runs on; here: file order -> prepared
 * order, and the tail.  in, out: K*N + 4 bytes each, 16-byte aligned, not overlapping
 * (MARIAN_HIP_ERR_ALIAS).  K % 64 == 0, N % 8 == 0.
 */
int marian_hip_int8_prepare_b_quantized_transposed(const int8_t* in, int8_t* out, int64_t K,
                                                   int64_t N, void* stream);

/*
 * Replaces the multiply node body, reference src/tensors/cpu/intgemm_interface.h:60-88:
 *   Kernels8::Multiply with callbacks::UnquantizeAndWrite (bias == NULL, dot) or
 *   UnquantizeAndAddBiasAndWrite (affine).  Both quantMults are read on the device from the
 *   operand tails (the reference dereferences them on the host, :66-67).
 *   unquant = (1.0f / (aqm * bqm)) * scale;  out[m,n] = float(acc[m,n]) * unquant (+ bias[n]).
 * relu != 0 fuses the ReLU that the reference applies as a separate in-place node
 * (src/graph/expression_operators.cpp:721-731, src/functional/operators.h:128).
 * out: fp32 [M x N].
 */
int marian_hip_int8_affine(const int8_t* Aq, const int8_t* Bq, const float* bias, float* out,
                           int64_t M, int64_t K, int64_t N, float scale, int relu,
                           void* stream);

/*
 * prepareA node + multiply node in one call (reference src/tensors/cpu/intgemm_interface.h:52
 * builds the first inside affineOrDotTyped and :60-94 the second).  Results are those of
 * marian_hip_int8_prepare_a followed by marian_hip_int8_affine / _affine_shortlist: Aq (M*K + 4
 * bytes, required) receives the quantized activations and their quantMult, out the product.
 * For small activations both steps run in one kernel (every workgroup derives the same abs-max);
 * otherwise the two kernels are launched back to back.  idx == NULL selects the dense form.
 */
int marian_hip_int8_affine_f32(const float* A, int8_t* Aq, const int8_t* Bq, const float* bias,
                               const uint32_t* idx, int64_t n_idx, float* out, int64_t M,
                               int64_t K, int64_t N, float scale, int relu, void* workspace,
                               size_t workspace_bytes, void* stream);

/*
 * marian_hip_int8_affine_f32 with the activations' abs-max handed from the call that produced
 * them to the call that consumes them.  The reference recomputes max|A| in every prepareA node
 * (src/tensors/cpu/intgemm_interface.h:23); here the kernel that writes a tensor can leave values
 * whose maximum is that abs-max, and the next call takes them instead of scanning the tensor
 * again (one launch fewer per call in a decoder step).  Results are those of
 * marian_hip_int8_affine_f32, bit for bit (a maximum is exact in any grouping).
 *   absmax_in:  NULL, or MARIAN_HIP_ABSMAX_SLOTS floats whose maximum is max|A| - the absmax_out
 *               of the call that wrote A (this one, marian_hip_layer_norm or marian_hip_attention).
 *   absmax_out: NULL, or MARIAN_HIP_ABSMAX_SLOTS floats that receive values whose maximum is
 *               max|out|.
 */
#define MARIAN_HIP_ABSMAX_SLOTS 2048
int marian_hip_int8_affine_f32_chained(const float* A, int8_t* Aq, const int8_t* Bq,
                                       const float* bias, const uint32_t* idx, int64_t n_idx,
                                       float* out, int64_t M, int64_t K, int64_t N, float scale,
                                       int relu, const float* absmax_in, float* absmax_out,
                                       void* workspace, size_t workspace_bytes, void* stream);

/*
 * One activation tensor, several weight matrices, one call: the self-attention projections of a
 * transformer layer read the same input through three separate weight matrices with three
 * quantMults (reference src/models/transformer.h:290-325: Wq, Wk, Wv), which in the reference is
 * three affine nodes, each with its own prepareA node over the same tensor
 * (src/tensors/cpu/intgemm_interface.h:52).  Here max|A| is taken once, A is quantized once (Aq and
 * its tail are written once) and, for decode-size activations, one kernel multiplies it by all the
 * matrices.  out[g] is what marian_hip_int8_affine_f32(A, Aq, Bq[g], bias[g], NULL, 0, out[g], M, K,
 * N[g], scale, relu, ...) writes, bit for bit.
 *   Bq, bias, out, N: HOST arrays of n_groups (1 .. 4) entries, read during the call; their
 *   entries are device pointers / column counts.  bias may be NULL, and so may any bias[g].
 *   absmax_in: as for marian_hip_int8_affine_f32_chained, or NULL.
 */
int marian_hip_int8_affine_f32_grouped(const float* A, int8_t* Aq, int64_t n_groups,
                                       const int8_t* const* Bq, const float* const* bias,
                                       float* const* out, const int64_t* N, int64_t M, int64_t K,
                                       float scale, int relu, const float* absmax_in, void* workspace,
                                       size_t workspace_bytes, void* stream);

/*
 * The projections in front of an attention and the attention itself, for ONE new target position
 * per query row, in one launch (reference src/models/transformer.h:279-348, MultiHead: q =
 * affine(input, Wq, bq) and, for self-attention, k / v = affine(input, Wk / Wv, ..), the head
 * split, then Attention(), :240-277).  A workgroup owns the 64 columns of one head in every
 * projection for a few rows of the input and runs that head's attention for them before it exits,
 * so q (k, v) never travel through memory.  Head size 64; N = heads * 64 columns per matrix.
 *   n_proj = 3: Bq / bias / proj_out hold {Wq, Wk, Wv}; the new key and value rows are appended to
 *     the caches at position len - 1 (as marian_hip_attention_cached does with k_new / v_new) and
 *     the attention runs over positions 0 .. len - 1; batchKV = M * heads.
 *   n_proj = 1: Bq / bias / proj_out hold {Wq}; the caches are complete (the encoder's keys and
 *     values), query row r uses cache entry r % batchKV.  With batchKV = sentences * heads and
 *     M = hypotheses * sentences (row m of A belongs to sentence m % sentences, the reference's
 *     [beam, batch] order) and two or more hypotheses a sentence, a workgroup takes hypotheses
 *     of the same one or two sentences and reads their keys and values once (up to 96 positions;
 *     other shapes take the general path, same result).
 *   A: fp32 [M x K]; Aq receives what marian_hip_int8_prepare_a would write.  K % 128 == 0,
 *     K <= 1024, len <= 512.  Bq, bias, proj_out: HOST arrays of n_proj device pointers, read
 *     during the call; bias and proj_out (and their entries) may be NULL.  proj_out[g], where
 *     given, receives the projection itself, fp32 [M x N] - bit for bit what
 *     marian_hip_int8_affine_f32 writes.
 *   k_cache, v_cache: [batchKV, kv_capacity, 64] fp32, `len` positions in use; mask: NULL or
 *     [n_masks, len], row (r / heads) % n_masks for query row r of the [M * heads] rows;
 *     out: [M * heads, 64] = [M x N]; att_scale: the 1 / sqrt(64) of transformer.h:261.
 *   absmax_in / absmax_out / workspace: as for marian_hip_int8_affine_f32_chained (absmax_out
 *     needs M * heads <= 2048; the workspace is only used when absmax_in is NULL).
 * The result has the bits of the separate calls (marian_hip_int8_affine_f32_grouped, then
 * marian_hip_attention_cached).  When to use it (measured with d = 1024, 16 heads, 21 cached / 60
 * source positions, calls back to back): it is ahead of the two separate calls up to 128 rows
 * (n_proj = 3: 11.7 against 13.1 us, n_proj = 1: 9.5 against 11.5 us), level at 256 rows (23.2
 * against 22.7, 17.8 against 17.5 us) and behind beyond (512 rows: 41.8 against 43.4 us, but 34.1
 * against 28.1 us for n_proj = 1): every eight rows read the head's weights again.
 */
int marian_hip_int8_proj_attention(const float* A, int8_t* Aq, int64_t n_proj, const int8_t* const* Bq,
                                   const float* const* bias, float* const* proj_out, int64_t M, int64_t K,
                                   int64_t heads, float* k_cache, float* v_cache, int64_t batchKV, int64_t len,
                                   int64_t kv_capacity, const float* mask, int64_t n_masks, float att_scale,
                                   float* out, const float* absmax_in, float* absmax_out, void* workspace,
                                   size_t workspace_bytes, void* stream);

/*
 * marian_hip_int8_affine_f32 for callers that cannot allocate and have no workspace to pass: code
 * under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  It has no
 * counterpart in the reference (there the prepareA node's output and every temporary come from the
 * graph's allocator).  The caller passes inputs and the output only; the quantized activations
 * (M*K + 4 bytes) and the abs-max partials live in an array of
 * MARIAN_HIP_STATIC_MAX_ELEMS + 256 + marian_hip_int8_workspace_bytes() bytes that the library
 * holds on every GPU it runs on until the process ends (16 MiB + 256 B + the 12 KB workspace).
 * The words workgroups exchange through the workspace (one-pass prepareA, M * K >= 4 Mi) persist
 * between calls and are told apart by tags; nothing in the array is ever cleared.  The call makes
 * no hipMalloc / hipFree and no allocating library call.  `out` is what marian_hip_int8_affine_f32 writes, bit for bit.
 *   M * K > MARIAN_HIP_STATIC_MAX_ELEMS returns MARIAN_HIP_ERR_STATIC_LIMIT (checked first).
 *   The device must be current and `stream` must belong to it.  The first call on a device looks
 *   up the array's address (make that call outside a graph capture).
 *   All calls on one GPU share the array: calls that overlap on one GPU (two streams, two
 *   threads) race; serialise them or use marian_hip_int8_affine_f32 with buffers of your own.
 */
#define MARIAN_HIP_STATIC_MAX_ELEMS (16 * 1024 * 1024)
int marian_hip_int8_affine_f32_static(const float* A, const int8_t* Bq, const float* bias,
                                      const uint32_t* idx, int64_t n_idx, float* out, int64_t M,
                                      int64_t K, int64_t N, float scale, int relu, void* stream);

/*
 * Shortlisted output layer.  Reference (fp32): index_select(Wt, 0, idx), index_select(b, -1,
 * idx), then dot/affine with transB (src/data/shortlist.cpp:62-79,
 * src/layers/output.cpp:335-350).  Here columns idx[j] of the prepared weights (rows of W^T) and
 * bias[idx[j]] are gathered inside the GEMM; bqm is the quantMult of the full matrix.
 * idx: n_idx sorted unique uint32 ids < N.  out: fp32 [M x n_idx].
 */
int marian_hip_int8_affine_shortlist(const int8_t* Aq, const int8_t* Bq, const float* bias,
                                     const uint32_t* idx, int64_t n_idx, float* out,
                                     int64_t M, int64_t K, int64_t N, float scale, int relu,
                                     void* stream);

/*
 * Parity hooks: the same kernels with the epilogue replaced by a store of the raw int32
 * accumulators (what Kernels8::Multiply hands to its callback).  acc: int32 [M x N] or
 * [M x n_idx].  idx == NULL selects the dense form.
 */
int marian_hip_int8_multiply_i32(const int8_t* Aq, const int8_t* Bq, const uint32_t* idx,
                                 int64_t n_idx, int32_t* acc, int64_t M, int64_t K, int64_t N,
                                 void* stream);

#ifdef __cplusplus
}
#endif
#endif /* MARIAN_HIP_INT8_H */
