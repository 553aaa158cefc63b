"""MI355X-native dense GEMM path of DECX: HIP kernels behind a C ABI (csrc/, include/decx_hip.h),
the C++ de:: host layer (host/, include/DECX.h), and this thin ctypes view for tests and benchmarks."""
