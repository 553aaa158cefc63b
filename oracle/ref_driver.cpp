// TEST INFRASTRUCTURE ONLY.  C-callable shim around the *reference's own* CPU GEMM
// (compiled from /root/reference by build_ref.sh into oracle/_ref/), so the tests can
// check the oracle bit-for-bit against the real thing in the build container.
// Calls only the reference's public API: de::CreateMatrixRef, de::Matrix::ptr,
// de::cpu::DecxSetThreadingNum, de::blas::cpu::GEMM (srcs/includes/DECX/BLAS/BLAS.h:57,60).
#include "DECX.h"
#include <cstring>
#include <chrono>

extern "C" int ref_cpu_gemm_f32(const float* A, const float* B, const float* C, float* D,
                                uint32_t M, uint32_t N, uint32_t K, uint32_t threads)
{
    de::cpu::DecxSetThreadingNum(threads);
    de::Matrix& mA = de::CreateMatrixRef(de::_FP32_, K, M);
    de::Matrix& mB = de::CreateMatrixRef(de::_FP32_, N, K);
    de::Matrix& mD = de::CreateMatrixRef(de::_FP32_, N, M);
    for (uint32_t i = 0; i < M; ++i) std::memcpy(mA.ptr<float>(i, 0), A + (size_t)i * K, K * sizeof(float));
    for (uint32_t i = 0; i < K; ++i) std::memcpy(mB.ptr<float>(i, 0), B + (size_t)i * N, N * sizeof(float));
    if (C) {
        de::Matrix& mC = de::CreateMatrixRef(de::_FP32_, N, M);
        for (uint32_t i = 0; i < M; ++i) std::memcpy(mC.ptr<float>(i, 0), C + (size_t)i * N, N * sizeof(float));
        de::blas::cpu::GEMM(mA, mB, mC, mD);
        mC.release();
    } else {
        de::blas::cpu::GEMM(mA, mB, mD);
    }
    const int err = de::GetLastError()->error_type;
    for (uint32_t i = 0; i < M; ++i) std::memcpy(D + (size_t)i * N, mD.ptr<float>(i, 0), N * sizeof(float));
    mA.release(); mB.release(); mD.release();
    return err;
}

// The same product `repeats` times over the same matrices, timing de::blas::cpu::GEMM alone (matrix creation and
// the copies in and out excluded): best_ms receives the shortest call.  For checking the timed restatement's clock.
extern "C" int ref_cpu_gemm_f32_timed(const float* A, const float* B, float* D, uint32_t M, uint32_t N, uint32_t K,
                                      uint32_t threads, uint32_t repeats, double* best_ms)
{
    de::cpu::DecxSetThreadingNum(threads);
    de::Matrix& mA = de::CreateMatrixRef(de::_FP32_, K, M);
    de::Matrix& mB = de::CreateMatrixRef(de::_FP32_, N, K);
    de::Matrix& mD = de::CreateMatrixRef(de::_FP32_, N, M);
    for (uint32_t i = 0; i < M; ++i) std::memcpy(mA.ptr<float>(i, 0), A + (size_t)i * K, K * sizeof(float));
    for (uint32_t i = 0; i < K; ++i) std::memcpy(mB.ptr<float>(i, 0), B + (size_t)i * N, N * sizeof(float));
    double best = 1e30;
    for (uint32_t r = 0; r < repeats; ++r) {
        const auto t0 = std::chrono::steady_clock::now();
        de::blas::cpu::GEMM(mA, mB, mD);
        const double ms = std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - t0).count();
        if (ms < best) best = ms;
    }
    if (best_ms) *best_ms = best;
    const int err = de::GetLastError()->error_type;
    for (uint32_t i = 0; i < M; ++i) std::memcpy(D + (size_t)i * N, mD.ptr<float>(i, 0), N * sizeof(float));
    mA.release(); mB.release(); mD.release();
    return err;
}

extern "C" int ref_cpu_gemm_f64(const double* A, const double* B, const double* C, double* D,
                                uint32_t M, uint32_t N, uint32_t K, uint32_t threads)
{
    de::cpu::DecxSetThreadingNum(threads);
    de::Matrix& mA = de::CreateMatrixRef(de::_FP64_, K, M);
    de::Matrix& mB = de::CreateMatrixRef(de::_FP64_, N, K);
    de::Matrix& mD = de::CreateMatrixRef(de::_FP64_, N, M);
    for (uint32_t i = 0; i < M; ++i) std::memcpy(mA.ptr<double>(i, 0), A + (size_t)i * K, K * sizeof(double));
    for (uint32_t i = 0; i < K; ++i) std::memcpy(mB.ptr<double>(i, 0), B + (size_t)i * N, N * sizeof(double));
    if (C) {
        de::Matrix& mC = de::CreateMatrixRef(de::_FP64_, N, M);
        for (uint32_t i = 0; i < M; ++i) std::memcpy(mC.ptr<double>(i, 0), C + (size_t)i * N, N * sizeof(double));
        de::blas::cpu::GEMM(mA, mB, mC, mD);
        mC.release();
    } else {
        de::blas::cpu::GEMM(mA, mB, mD);
    }
    const int err = de::GetLastError()->error_type;
    for (uint32_t i = 0; i < M; ++i) std::memcpy(D + (size_t)i * N, mD.ptr<double>(i, 0), N * sizeof(double));
    mA.release(); mB.release(); mD.release();
    return err;
}

// complex single precision, interleaved (re, im); pitches of the dense inputs in complex elements
extern "C" int ref_cpu_gemm_c32(const float* A, const float* B, const float* C, float* D,
                                uint32_t M, uint32_t N, uint32_t K, uint32_t threads)
{
    de::cpu::DecxSetThreadingNum(threads);
    de::Matrix& mA = de::CreateMatrixRef(de::_COMPLEX_F32_, K, M);
    de::Matrix& mB = de::CreateMatrixRef(de::_COMPLEX_F32_, N, K);
    de::Matrix& mD = de::CreateMatrixRef(de::_COMPLEX_F32_, N, M);
    for (uint32_t i = 0; i < M; ++i) std::memcpy(mA.ptr<de::CPf>(i, 0), A + (size_t)i * K * 2, K * sizeof(de::CPf));
    for (uint32_t i = 0; i < K; ++i) std::memcpy(mB.ptr<de::CPf>(i, 0), B + (size_t)i * N * 2, N * sizeof(de::CPf));
    if (C) {
        de::Matrix& mC = de::CreateMatrixRef(de::_COMPLEX_F32_, N, M);
        for (uint32_t i = 0; i < M; ++i) std::memcpy(mC.ptr<de::CPf>(i, 0), C + (size_t)i * N * 2, N * sizeof(de::CPf));
        de::blas::cpu::GEMM(mA, mB, mC, mD);
        mC.release();
    } else {
        de::blas::cpu::GEMM(mA, mB, mD);
    }
    const int err = de::GetLastError()->error_type;
    for (uint32_t i = 0; i < M; ++i) std::memcpy(D + (size_t)i * N * 2, mD.ptr<de::CPf>(i, 0), N * sizeof(de::CPf));
    mA.release(); mB.release(); mD.release();
    return err;
}
