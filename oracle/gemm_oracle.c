/*
 * TEST INFRASTRUCTURE ONLY -- never linked into, loaded by, or called from the
 * product library.  Only the test-suite, the smoke check and the CPU-baseline
 * leg of the benchmark may use this file.
 *
 * CPU restatement of the arithmetic of DECX's dense matrix product, used as the
 * parity oracle for the HIP kernels.
 *
 * What the reference computes (row-major, pitched matrices, M = A.Height,
 * N = B.Width, K = A.Width = B.Height):
 *
 *   fp32  D = A.B      every output element is one fused-multiply-add chain in
 *                      ascending k starting from 0: one SIMD lane per element,
 *                      `_mm256_fmadd_ps` per k, partial sums spilled to dst in
 *                      fp32 (lossless) between 128-deep K slabs.
 *                      srcs/modules/BLAS/GEMM/CPU/fp32/x86/GEMM_fp32_kernels_x86_64.h:86-127,222-242
 *   fp32  D = A.B + C  the same chain seeded with C[i][j] (the `_ABC` template
 *                      argument loads C instead of zero on the first slab).
 *                      .../GEMM_fp32_kernels_x86_64.h:90,149-150
 *   fp32  D = alpha.A.B + beta.C   (GPU-only entry point) chain from 0, then
 *                      t = alpha*acc (rounded), D = fma(C, beta, t).
 *                      srcs/modules/BLAS/GEMM/CUDA/large_squares/fp32/GEMM_fp32_B128_kernels.cu:725-744
 *   fp16               the reference has no CPU fp16 GEMM
 *                      (srcs/modules/BLAS/GEMM/CPU/GEMM.cxx:58-78); the oracle is
 *                      the fp32 chain on the half inputs widened to float, the
 *                      result rounded to nearest-even half (de::Float2Half is
 *                      `__float2half`, srcs/common/FP16/float_half_convert.cu:35-46).
 *
 * Pinning (see tests/test_oracle.py): the chain is checked against exact
 * rational arithmetic with a hand-written round-to-nearest-even on tiny inputs,
 * against a float64 brute force, against numpy float64 matmul, against the
 * closed forms identity.B == B, ones.ones == K, sum l^2 of the reference's
 * MatMul sample, and -- where oracle/_ref has been built -- bit-for-bit against
 * the compiled reference CPU GEMM.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

/* ---------------------------------------------------------------- half <-> float */

/* IEEE binary16 -> binary32, exact. */
float oracle_half_to_float(uint16_t h)
{
    const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t expo = (h >> 10) & 0x1fu;
    uint32_t mant = h & 0x3ffu;
    uint32_t bits;
    if (expo == 0x1fu) {                       /* inf / nan */
        bits = sign | 0x7f800000u | (mant << 13);
    } else if (expo != 0) {                    /* normal */
        bits = sign | ((expo + 112u) << 23) | (mant << 13);
    } else if (mant == 0) {                    /* zero */
        bits = sign;
    } else {                                   /* subnormal: renormalise */
        int e = -1;
        do { mant <<= 1; ++e; } while (!(mant & 0x400u));
        bits = sign | ((uint32_t)(112 - e) << 23) | ((mant & 0x3ffu) << 13);
    }
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

/* IEEE binary32 -> binary16, round to nearest, ties to even (what __float2half does). */
uint16_t oracle_float_to_half(float f)
{
    uint32_t x;
    memcpy(&x, &f, 4);
    const uint16_t sign = (uint16_t)((x >> 16) & 0x8000u);
    x &= 0x7fffffffu;
    if (x >= 0x7f800000u) {                    /* inf / nan */
        return (uint16_t)(sign | 0x7c00u | (x > 0x7f800000u ? 0x200u | ((x >> 13) & 0x3ffu) : 0));
    }
    if (x >= 0x477ff000u) {                    /* rounds to >= 65520 -> inf */
        return (uint16_t)(sign | 0x7c00u);
    }
    if (x < 0x33000001u) {                     /* <= 2^-25: rounds to zero (tie goes to even = 0) */
        return sign;
    }
    int32_t e = (int32_t)(x >> 23) - 127;      /* unbiased exponent */
    uint32_t m = (x & 0x7fffffu) | 0x800000u;  /* 24-bit significand */
    uint32_t shift, half_e;
    if (e < -14) {                             /* subnormal half */
        shift = (uint32_t)(13 + (-14 - e));
        half_e = 0;
    } else {
        shift = 13;
        half_e = (uint32_t)(e + 15);
    }
    uint32_t q = m >> shift;
    const uint32_t rem = m & ((1u << shift) - 1u);
    const uint32_t halfway = 1u << (shift - 1);
    if (rem > halfway || (rem == halfway && (q & 1u))) ++q;
    /* for normals q carries the implicit bit (0x400): adding instead of or-ing lets a
       mantissa overflow ripple into the exponent, which is the correct result */
    uint32_t out = (half_e ? ((half_e - 1) << 10) : 0) + q;
    return (uint16_t)(sign | out);
}

/* ---------------------------------------------------------------- seeded inputs */

/* Counter-based generator: value i of stream `seed` is a pure function of (seed, i). */
static inline uint64_t splitmix64_at(uint64_t seed, uint64_t i)
{
    uint64_t z = seed + (i + 1) * 0x9E3779B97F4A7C15ull;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}

/* iid uniform in [-1, 1): top 24 bits -> [0,1) exactly representable, times 2 minus 1. */
void oracle_fill_uniform_f32(float* dst, uint32_t rows, uint32_t cols, uint32_t pitch, uint64_t seed)
{
    for (uint32_t r = 0; r < rows; ++r)
        for (uint32_t c = 0; c < cols; ++c) {
            const uint64_t u = splitmix64_at(seed, (uint64_t)r * cols + c) >> 40;
            dst[(size_t)r * pitch + c] = (float)u * (1.0f / 8388608.0f) - 1.0f;
        }
}

/* ---------------------------------------------------------------- fp32 chains */

/*
 * D[i][j] = fma-chain over k ascending, seeded with 0 (C == NULL) or C[i][j].
 * The loop nest is k-outer / j-inner so the compiler can vectorise across j; every
 * element's chain is still strictly sequential in k, hence bit-identical to the
 * scalar loop `for k: acc = fmaf(A[i][k], B[k][j], acc)`.
 * `rows`/`nrows` select a subset of output rows (NULL = all M rows); row r of the
 * subset is written to D + r*ldd when rows != NULL (compact), else to row i.
 */
void oracle_gemm_f32_chain(const float* A, const float* B, const float* C, float* D,
                           uint32_t M, uint32_t N, uint32_t K,
                           uint32_t lda, uint32_t ldb, uint32_t ldc, uint32_t ldd,
                           const uint32_t* rows, uint32_t nrows)
{
    const uint32_t count = rows ? nrows : M;
#pragma omp parallel for schedule(dynamic, 1)
    for (uint32_t r = 0; r < count; ++r) {
        const uint32_t i = rows ? rows[r] : r;
        float* __restrict acc = D + (size_t)r * ldd;
        if (C) for (uint32_t j = 0; j < N; ++j) acc[j] = C[(size_t)i * ldc + j];
        else   for (uint32_t j = 0; j < N; ++j) acc[j] = 0.0f;
        for (uint32_t k = 0; k < K; ++k) {
            const float a = A[(size_t)i * lda + k];
            const float* __restrict b = B + (size_t)k * ldb;
            for (uint32_t j = 0; j < N; ++j) acc[j] = fmaf(a, b[j], acc[j]);
        }
    }
}

/* Plain scalar form of the same thing, no vectorisable nest: used to pin the one above. */
void oracle_gemm_f32_chain_scalar(const float* A, const float* B, const float* C, float* D,
                                  uint32_t M, uint32_t N, uint32_t K,
                                  uint32_t lda, uint32_t ldb, uint32_t ldc, uint32_t ldd)
{
    for (uint32_t i = 0; i < M; ++i)
        for (uint32_t j = 0; j < N; ++j) {
            volatile float acc = C ? C[(size_t)i * ldc + j] : 0.0f;
            for (uint32_t k = 0; k < K; ++k)
                acc = fmaf(A[(size_t)i * lda + k], B[(size_t)k * ldb + j], acc);
            D[(size_t)i * ldd + j] = acc;
        }
}

/* D = fma(C, beta, alpha * chain0(A,B)) -- the GPU-only four-matrix entry point. */
void oracle_gemm_f32_axpby(const float* A, const float* B, const float* C, float* D,
                           uint32_t M, uint32_t N, uint32_t K,
                           uint32_t lda, uint32_t ldb, uint32_t ldc, uint32_t ldd,
                           float alpha, float beta,
                           const uint32_t* rows, uint32_t nrows)
{
    oracle_gemm_f32_chain(A, B, NULL, D, M, N, K, lda, ldb, 0, ldd, rows, nrows);
    const uint32_t count = rows ? nrows : M;
    for (uint32_t r = 0; r < count; ++r) {
        const uint32_t i = rows ? rows[r] : r;
        for (uint32_t j = 0; j < N; ++j) {
            const float t = alpha * D[(size_t)r * ldd + j];
            D[(size_t)r * ldd + j] = fmaf(C[(size_t)i * ldc + j], beta, t);
        }
    }
}

/* ---------------------------------------------------------------- fp16 */

/*
 * Half inputs widened to float, fp32 chain, epilogue alpha/beta in fp32
 * (C == NULL: plain product), result rounded once to half.
 */
void oracle_gemm_f16(const uint16_t* A, const uint16_t* B, const uint16_t* C, uint16_t* D,
                     uint32_t M, uint32_t N, uint32_t K,
                     uint32_t lda, uint32_t ldb, uint32_t ldc, uint32_t ldd,
                     float alpha, float beta,
                     const uint32_t* rows, uint32_t nrows)
{
    const uint32_t count = rows ? nrows : M;
    float* Bf = (float*)malloc((size_t)K * N * sizeof(float));
    for (uint32_t k = 0; k < K; ++k)
        for (uint32_t j = 0; j < N; ++j)
            Bf[(size_t)k * N + j] = oracle_half_to_float(B[(size_t)k * ldb + j]);
#pragma omp parallel
    {
        float* acc = (float*)malloc((size_t)N * sizeof(float));
#pragma omp for schedule(dynamic, 1)
        for (uint32_t r = 0; r < count; ++r) {
            const uint32_t i = rows ? rows[r] : r;
            for (uint32_t j = 0; j < N; ++j) acc[j] = 0.0f;
            for (uint32_t k = 0; k < K; ++k) {
                const float a = oracle_half_to_float(A[(size_t)i * lda + k]);
                const float* __restrict b = Bf + (size_t)k * N;
                for (uint32_t j = 0; j < N; ++j) acc[j] = fmaf(a, b[j], acc[j]);
            }
            for (uint32_t j = 0; j < N; ++j) {
                float v = acc[j];
                if (C) v = fmaf(oracle_half_to_float(C[(size_t)i * ldc + j]), beta, alpha * v);
                D[(size_t)r * ldd + j] = oracle_float_to_half(v);
            }
        }
        free(acc);
    }
    free(Bf);
}

/* ---------------------------------------------------------------- float64 brute force */

/* Independent of the chain: double products, double accumulation. For small shapes only. */
void oracle_gemm_f64_brute(const float* A, const float* B, const float* C, double* D,
                           uint32_t M, uint32_t N, uint32_t K,
                           uint32_t lda, uint32_t ldb, uint32_t ldc, uint32_t ldd,
                           double alpha, double beta)
{
    for (uint32_t i = 0; i < M; ++i)
        for (uint32_t j = 0; j < N; ++j) {
            double s = 0.0;
            for (uint32_t k = 0; k < K; ++k)
                s += (double)A[(size_t)i * lda + k] * (double)B[(size_t)k * ldb + j];
            D[(size_t)i * ldd + j] = alpha * s + (C ? beta * (double)C[(size_t)i * ldc + j] : 0.0);
        }
}

/* ---------------------------------------------------------------- fp64 */

/*
 * Double precision: the same k-ascending chain with fma in double, seeded with 0 or C[i][j]
 * (what the reference's fp64 CPU GEMM computes: srcs/modules/BLAS/GEMM/CPU/fp64/, same structure as the
 * fp32 path), and the GPU entry point's D = fma(C, beta, alpha * chain0)
 * (srcs/modules/BLAS/GEMM/CUDA/GEMM_LS.cu:164-211).  Pinned by tests/test_oracle.py: exact rational
 * arithmetic on tiny shapes, integer closed forms, and bit-for-bit against the compiled reference and its
 * committed outputs (tests/golden/ref_f64_*.npz).
 */
void oracle_gemm_f64_chain(const double* A, const double* B, const double* C, double* D,
                           uint32_t M, uint32_t N, uint32_t K,
                           uint32_t lda, uint32_t ldb, uint32_t ldc, uint32_t ldd,
                           const uint32_t* rows, uint32_t nrows)
{
    const uint32_t count = rows ? nrows : M;
#pragma omp parallel for schedule(dynamic, 1)
    for (uint32_t r = 0; r < count; ++r) {
        const uint32_t i = rows ? rows[r] : r;
        double* __restrict acc = D + (size_t)r * ldd;
        if (C) for (uint32_t j = 0; j < N; ++j) acc[j] = C[(size_t)i * ldc + j];
        else   for (uint32_t j = 0; j < N; ++j) acc[j] = 0.0;
        for (uint32_t k = 0; k < K; ++k) {
            const double a = A[(size_t)i * lda + k];
            const double* __restrict b = B + (size_t)k * ldb;
            for (uint32_t j = 0; j < N; ++j) acc[j] = fma(a, b[j], acc[j]);
        }
    }
}

void oracle_gemm_f64_axpby(const double* A, const double* B, const double* C, double* D,
                           uint32_t M, uint32_t N, uint32_t K,
                           uint32_t lda, uint32_t ldb, uint32_t ldc, uint32_t ldd,
                           double alpha, double beta,
                           const uint32_t* rows, uint32_t nrows)
{
    oracle_gemm_f64_chain(A, B, NULL, D, M, N, K, lda, ldb, 0, ldd, rows, nrows);
    const uint32_t count = rows ? nrows : M;
    for (uint32_t r = 0; r < count; ++r) {
        const uint32_t i = rows ? rows[r] : r;
        for (uint32_t j = 0; j < N; ++j) {
            const double t = alpha * D[(size_t)r * ldd + j];
            D[(size_t)r * ldd + j] = fma(C[(size_t)i * ldc + j], beta, t);
        }
    }
}
