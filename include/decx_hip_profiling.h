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

/* A register-only loop on the matrix cores: no loads, no LDS, no barriers -- what the matrix pipe sustains on this
 * board under its power management, for the operand values given.  One workgroup of 8 wavefronts per CU, each wavefront
 * `iters` times over 16 tiles of v_mfma_f32_16x16x32_f16 (elem_bytes 2: operands are halves) or 4 steps over 8 tiles of
 * v_mfma_f32_32x32x2_f32 (elem_bytes 4: floats).  `operands`: at least 16 bytes, 16-byte aligned, read cyclically
 * (128 bytes per lane); `sink`: one float per lane (CUs x 512), so that nothing is optimised away; *flops: the
 * floating-point operations of the launch.  No counterpart in the reference: bench.py times it next to the GEMM so
 * that the nominal peak can be read beside the rate this board really allows. */
DECX_HIP_API int decx_hip_calibration_mfma(int elem_bytes, const void* operands, size_t operand_bytes, float* sink,
                                           size_t sink_floats, uint32_t iters, double* flops, void* stream);

/* What the split-K counter windows of the current device have seen so far: out[0] windows handed out, out[1] times
 * the ring wrapped round, out[2] requests refused (the product then ran unsplit), out[3] events recorded (only once
 * launches have come from more than one stream), out[4] counters given to launches recorded into graphs, out[5] the
 * counters left to the ring.  For tests. */
DECX_HIP_API int decx_hip_split_counter_stats(uint64_t out[6]);

#ifdef __cplusplus
}
#endif
#endif  /* DECX_HIP_PROFILING_H_ */
