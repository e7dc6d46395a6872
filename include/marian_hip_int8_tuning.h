/*
 * marian_hip_int8_tuning.h - measurement switches of the tuning build of the int8 backend.
 *
 * These functions exist only in libmarian_hip_int8_tuning.so (built with
 * -DMARIAN_HIP_TUNING from the same sources as libmarian_hip_int8.so).  That build exports
 * everything include/marian_hip_int8.h and include/marian_hip_ops.h declare plus the
 * functions below, can pin every kernel family and tile shape the sources hold, whatever the
 * automatic selection would pick, and reads clocks inside its kernels.  The shipped library has none of this: no process-wide switch, no
 * retained pointer.  They have no counterpart in the reference; tests use them to run every
 * kernel family on every shape, measurements to compare kernels and to time their phases.
 */
#ifndef MARIAN_HIP_INT8_TUNING_H
#define MARIAN_HIP_INT8_TUNING_H

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

/*
 * Kernel selection override, PROCESS-WIDE (all threads, all streams): 0 = automatic (default),
 * other values pin one kernel family, or one choice inside a family, for every later
 * affine/multiply call.  `which / 1000` sets measurement bits of the large-M kernels (1: no
 * operand refetch, 2: no stores - results are then wrong on purpose).  Returns the previous value;
 * callers restore it when they are done.
 */
int marian_hip_int8_set_kernel(int which);

/*
 * Per-workgroup phase clocks: after this call every GEMM kernel of the process writes eight
 * 64-bit clock values per workgroup to `clocks` (device memory, 8 * sizeof(long long) * grid size
 * of the largest launch).  The pointer is RETAINED until the next call; pass NULL to switch the
 * recording off before the buffer is freed.
 */
void marian_hip_int8_debug_profile(long long* clocks);

/*
 * Machine-ceiling probes: the yardsticks the kernels' times are held against.
 *
 * marian_hip_probe_stream: `workgroups` x `threads` threads read read_bytes from src
 * (16 bytes per load, loads_in_flight of them outstanding per thread: 1, 4 or 8) and then write
 * write_bytes to dst (non-temporal stores if asked) - the data movement of a kernel without its
 * arithmetic.  read_bytes and write_bytes are multiples of 16; dst holds write_bytes.
 *
 * marian_hip_probe_mfma: `workgroups` workgroups of four waves issue iters x 8 independent
 * v_mfma_i32_32x32x32_i8 per wave on the 4 KB of operand bits at `data`; clocks[2 * w] and
 * clocks[2 * w + 1] receive the shader clocks and the 100 MHz reference clocks workgroup w spent
 * in the loop (sustained int8 rate = 2 * 32^3 * 8 * iters * 4 waves * workgroups / time; shader
 * clock = 100 MHz * clocks ratio).  sink: one int of device memory.
 */
int marian_hip_probe_stream(const void* src, size_t read_bytes, void* dst, size_t write_bytes, int workgroups,
                            int threads, int loads_in_flight, int nontemporal, void* stream);
int marian_hip_probe_mfma(const void* data, int iters, int workgroups, long long* clocks, int* sink, void* stream);

/*
 * marian_hip_probe_mix: what one compute unit's LDS, vector L1 and matrix cores deliver under a
 * chosen instruction mix.  `workgroups` workgroups of `waves` waves (4, 8 or 16: one, two or four per SIMD)
 * repeat `iters` times a body of 16 slots over which `reads` conflict-free ds_read_b128 (1 KB per
 * wave each), `mfmas` v_mfma_i32_32x32x32_i8, `dmas` global_load_lds_dwordx4 (1 KB per wave from
 * global memory straight into LDS) and `gloads` global_load_dwordx4 (1 KB per wave into registers)
 * are spread evenly.  The global addresses walk over span_bytes (a power of two, at least 64 KB)
 * behind src, workgroup b starting b * stagger_bytes in (a multiple of 1 KB): span and stagger decide
 * which cache serves them - 64 KB apart over a few MB: the XCD's L2; span / workgroups apart over
 * a GiB: HBM.  Only the mixes the measurements use are
 * instantiated; another one returns MARIAN_HIP_ERR_SHAPE.  split (eight waves only): the first four
 * waves issue the LDS reads and matrix instructions, the other four the global loads.  The time is
 * that of the slowest wave.  clocks as for marian_hip_probe_mfma.
 */
int marian_hip_probe_mix(const void* src, size_t span_bytes, size_t stagger_bytes, int waves, int reads, int mfmas, int dmas, int gloads,
                         int split, int iters, int workgroups, long long* clocks, int* sink, void* stream);

/*
 * The hand-over of candidates between the workgroups of marian_hip_nbest_beams and
 * marian_hip_logsoftmax_nbest_beams, PROCESS-WIDE: 0 (default) = what the shipped library does -
 * device-scope stores, a wait for their acknowledgement, a relaxed counter; 1 = the counter update
 * as an acquire-release operation at device scope, i.e. with the cache write-back and invalidation
 * the language's memory model asks for (about 8 us slower per call).  The two forms must give the
 * same bits; tests compare them.  Returns the previous value.
 */
int marian_hip_nbest_set_fenced(int on);

#ifdef __cplusplus
}
#endif
#endif /* MARIAN_HIP_INT8_TUNING_H */
