/*
 * decx_hip_profiling.h -- measurement and test aids exported by libdecx_hip.so beside the product ABI of decx_hip.h.
 * Nothing in the DECX API layer calls it; bench.py does, to calibrate hardware traffic counters.
 */
#ifndef DECX_HIP_PROFILING_H_
#define DECX_HIP_PROFILING_H_

#include "decx_hip.h"

#ifdef __cplusplus
extern "C" {
#endif

/* A plain device-to-device copy kernel (128-bit loads and stores, `bytes` a multiple of 16,
 * both pointers 16-byte aligned).  It has no counterpart in the reference: it exists so that
 * hardware traffic counters can be scaled against a launch whose HBM traffic is known
 * (reads = writes = `bytes`). */
DECX_HIP_API int decx_hip_calibration_copy(void* dst, const void* src, size_t bytes, void* stream);

/* A read-only pass over `bytes` (a multiple of 2 MiB, 16-byte aligned) of device memory filled with ONE byte value
 * (decx_hip_memset_async): 128-bit loads in the order the matrix x vector kernel reads rows of 64 KB, nothing stored --
 * `sink` (at least bytes / 2048 words) is only written if the fold of the loaded words came out as a value such a fill
 * cannot give.  What the memory system gives a pure read stream, the yardstick for the matrix x vector kernels.  No
 * counterpart in the reference. */
DECX_HIP_API int decx_hip_calibration_read(const void* src, size_t bytes, uint32_t* sink, size_t sink_words, void* stream);

/* A register-only loop on the matrix cores: no loads, no LDS, no barriers -- what the matrix pipe sustains on this
 * board under its power management, for the operand values given.  One workgroup of 8 wavefronts per CU, each wavefront
 * `iters` times over 16 tiles of v_mfma_f32_16x16x32_f16 (elem_bytes 2: operands are halves) or 4 steps over 8 tiles of
 * v_mfma_f32_32x32x2_f32 (elem_bytes 4: floats).  `operands`: at least 16 bytes, 16-byte aligned, read cyclically
 * (128 bytes per lane); `sink`: one float per lane (CUs x 512), so that nothing is optimised away; *flops: the
 * floating-point operations of the launch.  No counterpart in the reference: bench.py times it next to the GEMM so
 * that the nominal peak can be read beside the rate this board really allows. */
DECX_HIP_API int decx_hip_calibration_mfma(int elem_bytes, const void* operands, size_t operand_bytes, float* sink,
                                           size_t sink_floats, uint32_t iters, double* flops, void* stream);

/* A GEMM on a plan of the caller's choosing instead of the planner's: tile class `tile` (DECX_HIP_TILE_*), and with
 * k_splits > 1 that many ranges of K for all tiles but the first `whole_tiles` (workspace: k_splits slots of
 * tile_m x tile_n accumulators, 4 bytes each, 8 for fp64, per split tile).  16-byte aligned operands only (the
 * direct-to-LDS kernels); plans that have no kernel -- a split on a tile class whose kernels do not split, ranges
 * shorter than a slab -- return DECX_HIP_E_INVALID_ARG.  alpha and beta as doubles for every type.  It exists so that
 * the planner's pick can be timed against every other plan on shapes it was not fitted on (bench.py --workload
 * planner_sweep); the product path never calls it. */
DECX_HIP_API int decx_hip_gemm_forced_plan(int elem_bytes, const void* A, const void* B, const void* C, void* D,
                                           uint32_t M, uint32_t N, uint32_t K, uint32_t lda, uint32_t ldb, uint32_t ldc,
                                           uint32_t ldd, double alpha, double beta, int tile, uint32_t k_splits,
                                           uint32_t whole_tiles, void* workspace, size_t workspace_bytes, void* stream);

/* What the split-K counter windows of the current device have seen so far: out[0] windows handed out, out[1] times
 * the ring wrapped round, out[2] requests refused (the product then ran unsplit), out[3] events recorded (only once
 * launches have come from more than one stream), out[4] counters given to launches recorded into graphs, out[5] the
 * counters the ring goes round in (the lower half of the array; graphs draw on the upper half).  For tests. */
DECX_HIP_API int decx_hip_split_counter_stats(uint64_t out[6]);

#ifdef __cplusplus
}
#endif
#endif  /* DECX_HIP_PROFILING_H_ */
