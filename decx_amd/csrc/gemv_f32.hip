// y = alpha * A.x (+ beta * c) for fp32, A row-major M x K: the N == 1 corner of the GEMM
// entry point, which is bound by HBM bandwidth (every element of A is used once).
//
// Replaces cu_mat_m_vec_fp32 and its second reduction pass
// (srcs/modules/BLAS/GEMM/CUDA/extreme_shapes/VMM_fp32.cu:104-146): here one wavefront
// owns whole rows, so there are no partial sums to reduce in a second kernel.
//
//   * A workgroup of 16 wavefronts handles 32 rows, two rows per wavefront, K in chunks of
//     KC floats: 8192 rows give one workgroup per CU with 64 KB of A in flight.
//   * The x chunk is staged in LDS once per workgroup, then read as 128-bit words,
//     conflict-free.  x may be strided (the single column of a pitched K x 1 matrix puts
//     every element in its own cache line), so staging it once per 32 rows rather than per
//     8 keeps that gather at a quarter of the L2 traffic.
//   * A is read with 128-bit loads, 64 lanes covering 1 KB of a row per instruction,
//     four loads in flight per lane.
//   * Sums: per lane an fp32 fma chain over its k's (ascending), then a butterfly over
//     the 64 lanes.
#include "gemm_common.hpp"

namespace decx_hip {

constexpr int GEMV_THREADS = 1024;
constexpr int GEMV_ROWS_PER_BLOCK = 32;
constexpr int GEMV_KC = 8192;            // floats of x staged per chunk (32 KB of LDS)

__device__ __forceinline__ float wave_sum(float v)
{
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) v += __shfl_xor(v, off, 64);
    return v;
}

__global__ void __launch_bounds__(GEMV_THREADS)
gemv_f32_kernel(const float* __restrict__ A, const float* __restrict__ x, const float* __restrict__ c,
                float* __restrict__ y, uint32_t M, uint32_t K, uint32_t lda, uint32_t incx, uint32_t incc,
                uint32_t incy, float alpha, float beta, uint32_t vec_ok)
{
    __shared__ __attribute__((aligned(16))) float xs[GEMV_KC];
    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const uint32_t row0 = blockIdx.x * GEMV_ROWS_PER_BLOCK + wave * 2;
    const bool has0 = row0 < M, has1 = row0 + 1 < M;
    const float* a0 = A + (size_t)(has0 ? row0 : 0) * lda;
    const float* a1 = A + (size_t)(has1 ? row0 + 1 : 0) * lda;
    float s0 = 0.f, s1 = 0.f;

    for (uint32_t kc = 0; kc < K; kc += GEMV_KC) {
        const uint32_t len = (K - kc) < (uint32_t)GEMV_KC ? (K - kc) : (uint32_t)GEMV_KC;
        __syncthreads();                                   // previous chunk fully consumed
        for (uint32_t i = t; i < len; i += GEMV_THREADS) xs[i] = x[(size_t)(kc + i) * incx];
        __syncthreads();
        const uint32_t len4 = vec_ok ? (len & ~3u) : 0u;   // part done with 128-bit loads
        if (has0) {
#pragma unroll 4
            for (uint32_t k = lane * 4; k < len4; k += 256) {
                const floatx4 xv = *(const floatx4*)&xs[k];
                const floatx4 av = *(const floatx4*)(a0 + kc + k);
                s0 = __builtin_fmaf(av.x, xv.x, s0); s0 = __builtin_fmaf(av.y, xv.y, s0);
                s0 = __builtin_fmaf(av.z, xv.z, s0); s0 = __builtin_fmaf(av.w, xv.w, s0);
                if (has1) {
                    const floatx4 bv = *(const floatx4*)(a1 + kc + k);
                    s1 = __builtin_fmaf(bv.x, xv.x, s1); s1 = __builtin_fmaf(bv.y, xv.y, s1);
                    s1 = __builtin_fmaf(bv.z, xv.z, s1); s1 = __builtin_fmaf(bv.w, xv.w, s1);
                }
            }
            for (uint32_t k = len4 + lane; k < len; k += 64) {
                s0 = __builtin_fmaf(a0[kc + k], xs[k], s0);
                if (has1) s1 = __builtin_fmaf(a1[kc + k], xs[k], s1);
            }
        }
    }
    s0 = wave_sum(s0);
    s1 = wave_sum(s1);
    if (lane == 0) {
        if (has0) {
            float o = s0;
            if (c) o = __builtin_fmaf(c[(size_t)row0 * incc], beta, alpha * o);
            y[(size_t)row0 * incy] = o;
        }
        if (has1) {
            float o = s1;
            if (c) o = __builtin_fmaf(c[(size_t)(row0 + 1) * incc], beta, alpha * o);
            y[(size_t)(row0 + 1) * incy] = o;
        }
    }
}

int launch_gemv_f32(const float* A, const float* x, const float* c, float* y, uint32_t M, uint32_t K,
                    uint32_t lda, uint32_t incx, uint32_t incc, uint32_t incy, float alpha, float beta,
                    hipStream_t stream)
{
    const uint32_t vec_ok = (((uintptr_t)A & 15u) == 0 && (lda & 3u) == 0) ? 1u : 0u;
    const dim3 grid((M + GEMV_ROWS_PER_BLOCK - 1) / GEMV_ROWS_PER_BLOCK), block(GEMV_THREADS);
    hipLaunchKernelGGL(gemv_f32_kernel, grid, block, 0, stream, A, x, c, y, M, K, lda, incx, incc, incy,
                       alpha, beta, vec_ok);
    return (int)hipGetLastError();
}

}  // namespace decx_hip
