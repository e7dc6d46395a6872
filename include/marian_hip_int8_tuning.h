/*
 * marian_hip_int8_tuning.h - measurement switches of the tuning build of the int8 backend.
 *
 * These two functions exist only in libmarian_hip_int8_tuning.so (built with
 * -DMARIAN_HIP_TUNING from the same sources as libmarian_hip_int8.so).  That build exports
 * everything include/marian_hip_int8.h and include/marian_hip_ops.h declare plus the two
 * functions below, carries kernel families that the automatic selection never picks, and reads
 * clocks inside its kernels.  The shipped library has none of this: no process-wide switch, no
 * retained pointer.  They have no counterpart in the reference; tests use them to run every
 * kernel family on every shape, measurements to compare kernels and to time their phases.
 */
#ifndef MARIAN_HIP_INT8_TUNING_H
#define MARIAN_HIP_INT8_TUNING_H

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

#ifdef __cplusplus
}
#endif
#endif /* MARIAN_HIP_INT8_TUNING_H */
