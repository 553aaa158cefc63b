/*
 * decx_hip_profiling.h -- a measurement aid exported by libdecx_hip.so beside the product ABI of decx_hip.h.
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

#ifdef __cplusplus
}
#endif
#endif  /* DECX_HIP_PROFILING_H_ */
