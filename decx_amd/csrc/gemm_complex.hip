// Complex GEMM (interleaved re, im; single and double precision) on the real matrix-core kernels.
//
// Replaces decx::blas::GEMM_cplxf / GEMM_cplxd and the cu_GEMM_cplxf_* / cu_GEMM_cplxd_* kernels
// (srcs/modules/BLAS/GEMM/CUDA/GEMM_LS.cu:214-312, large_squares/GEMM_kernels.cuh:190-207).
//
// A complex M x K matrix stored interleaved IS a real M x 2K matrix.  With B expanded to the real
// 2K x 2N matrix
//        B'(2k, 2n) =  Re b   B'(2k, 2n + 1) = Im b
//        B'(2k + 1, 2n) = -Im b   B'(2k + 1, 2n + 1) = Re b          (b = alpha * B(k, n))
// the real product A . B' is the interleaved complex product alpha * A . B: the same 8 real
// flops per complex multiply-add, all of them on the MFMA pipe, no complex arithmetic in the hot
// kernel.  The expansion costs one pass over B (4 K N reals written into a caller-provided
// workspace); beta * C is formed in D first and the GEMM accumulates onto it (C may alias D).
#include "gemm_common.hpp"

namespace decx_hip {

namespace {

template <typename T>
__global__ void __launch_bounds__(256) complex_expand_b_kernel(const T* __restrict__ B, T* __restrict__ Bx, uint32_t K, uint32_t N,
                                                               uint32_t ldb, uint32_t ldx, T ar, T ai)
{
    // 64 columns x 4 rows per workgroup on a 1-D grid (grid.y would cap the rows at 4 x 65 535)
    const uint32_t cols = (N + 63) / 64;
    const uint32_t n = (blockIdx.x % cols) * 64 + (threadIdx.x & 63), k = (blockIdx.x / cols) * 4 + (threadIdx.x >> 6);
    if (n >= N || k >= K) return;
    const T br = B[((size_t)k * ldb + n) * 2], bi = B[((size_t)k * ldb + n) * 2 + 1];
    const T re = ar * br - ai * bi, im = ar * bi + ai * br;
    T* r0 = Bx + (size_t)(2 * k) * ldx + 2 * n;
    T* r1 = r0 + ldx;
    r0[0] = re;  r0[1] = im;
    r1[0] = -im; r1[1] = re;
}

// D = beta * C (complex, elementwise); C may be D
template <typename T>
__global__ void __launch_bounds__(256) complex_scale_kernel(const T* __restrict__ C, T* __restrict__ D, uint32_t M, uint32_t N,
                                                            uint32_t ldc, uint32_t ldd, T br, T bi)
{
    const uint32_t cols = (N + 63) / 64;
    const uint32_t n = (blockIdx.x % cols) * 64 + (threadIdx.x & 63), m = (blockIdx.x / cols) * 4 + (threadIdx.x >> 6);
    if (n >= N || m >= M) return;
    const T cr = C[((size_t)m * ldc + n) * 2], ci = C[((size_t)m * ldc + n) * 2 + 1];
    D[((size_t)m * ldd + n) * 2] = br * cr - bi * ci;
    D[((size_t)m * ldd + n) * 2 + 1] = br * ci + bi * cr;
}

}  // namespace

template <typename T>
int launch_complex_expand_b(const T* B, T* Bx, uint32_t K, uint32_t N, uint32_t ldb, uint32_t ldx, T ar, T ai, hipStream_t stream)
{
    const uint64_t blocks = (uint64_t)((N + 63) / 64) * ((K + 3) / 4);
    if (blocks > 0x7fffffffull) return (int)hipErrorInvalidValue;
    hipLaunchKernelGGL((complex_expand_b_kernel<T>), dim3((unsigned)blocks), dim3(256), 0, stream, B, Bx, K, N, ldb, ldx, ar, ai);
    return (int)hipGetLastError();
}
template <typename T>
int launch_complex_scale(const T* C, T* D, uint32_t M, uint32_t N, uint32_t ldc, uint32_t ldd, T br, T bi, hipStream_t stream)
{
    const uint64_t blocks = (uint64_t)((N + 63) / 64) * ((M + 3) / 4);
    if (blocks > 0x7fffffffull) return (int)hipErrorInvalidValue;
    hipLaunchKernelGGL((complex_scale_kernel<T>), dim3((unsigned)blocks), dim3(256), 0, stream, C, D, M, N, ldc, ldd, br, bi);
    return (int)hipGetLastError();
}

template int launch_complex_expand_b<float>(const float*, float*, uint32_t, uint32_t, uint32_t, uint32_t, float, float, hipStream_t);
template int launch_complex_expand_b<double>(const double*, double*, uint32_t, uint32_t, uint32_t, uint32_t, double, double, hipStream_t);
template int launch_complex_scale<float>(const float*, float*, uint32_t, uint32_t, uint32_t, uint32_t, float, float, hipStream_t);
template int launch_complex_scale<double>(const double*, double*, uint32_t, uint32_t, uint32_t, uint32_t, double, double, hipStream_t);

}  // namespace decx_hip
