// Exercises the public C++ API (include/DECX.h) the way a user of the original library
// would (cf. samples/Matrix_Multiplication/MatMul.cpp:74-113): factories, ptr<T>(),
// de::Memcpy, de::blas::cuda::GEMM, de::GetLastError.
//
//   de_api_test host                      checks that need no GPU; exit code 0 = all passed
//   de_api_test gpu                       self-contained GPU checks (closed forms, error paths)
//   de_api_test gemm <dir> <f32|f16> M N K <withC 0|1> <alpha> <beta>
//                                         reads dense A.bin B.bin [C.bin] from <dir>, writes D.bin
//   de_api_test hostgemm <dir> <f32|f16> M N K <withC 0|1|2> <pinned 0|1> <repeats>
//                                         the same through the host-matrix overloads (withC = 2: C is dst);
//                                         prints the wall time of each repeat
//   de_api_test threads                   several host threads through GEMM and Memcpy at once, each on matrices of its own
//   de_api_test tensor_host               tensor / tensor-array layouts and views, no GPU
//   de_api_test conv <dir> W H C OC KW KH sx sy <extend 0|2>
//                                         reads image.bin [H][W][C] and kernels.bin [OC][KH][KW][C] (dense fp32),
//                                         runs de::nn::cuda::Conv2D, writes out.bin [OH][OW][OC] and prints OW OH
//   de_api_test vmm <dir> <f32|f16> <mv|vm> W H <level 0|1|2>
//                                         reads M.bin (H rows x W) and V.bin, writes Y.bin (fp32 for f32
//                                         and for f16 at level 0, fp16 otherwise) through the host-object
//                                         vector forms of GEMM
#include "DECX.h"

#include <algorithm>
#include <chrono>
#include <cmath>
#include <cstdlib>
#include <cstring>
#include <fstream>
#include <iostream>
#include <atomic>
#include <string>
#include <thread>
#include <vector>

static int g_failures = 0;
#define CHECK(cond) do { if (!(cond)) { ++g_failures; std::cerr << "FAILED line " << __LINE__ << ": " #cond "\n"; } } while (0)

static int host_checks()
{
    // pitch rule of host matrices: rows padded to 32 bytes; storage zero-filled
    de::Matrix& a = de::CreateMatrixRef(de::_FP32_, 777, 5);
    CHECK(a.Width() == 777 && a.Height() == 5 && a.Type() == de::_FP32_ && a.Format() == de::_NA_);
    CHECK(a.ptr<float>(1, 0) - a.ptr<float>(0, 0) == 784);
    CHECK(((uintptr_t)a.ptr<float>(0, 0) & 31u) == 0);
    bool zero = true;
    for (int r = 0; r < 5; ++r) for (int c = 0; c < 784; ++c) zero &= (*a.ptr<float>(r, c) == 0.f);
    CHECK(zero);
    de::Matrix& h = de::CreateMatrixRef(de::_FP16_, 1, 3);
    CHECK(h.ptr<de::Half>(1, 0) - h.ptr<de::Half>(0, 0) == 16);
    de::Matrix* e = de::CreateMatrixPtr();
    CHECK(e->Width() == 0 && e->Height() == 0 && e->Type() == de::_VOID_);

    // SoftCopy aliases the storage
    de::Matrix& alias = de::CreateMatrixRef();
    alias.SoftCopy(a);
    *a.ptr<float>(2, 3) = 42.f;
    CHECK(alias.Width() == 777 && *alias.ptr<float>(2, 3) == 42.f);
    a.release();
    CHECK(*alias.ptr<float>(2, 3) == 42.f);            // still alive through the alias
    alias.Reinterpret(de::_INT32_);
    CHECK(alias.Type() == de::_INT32_ && alias.Width() == 777);

    // Number and Half
    de::Number n(1.5f);
    CHECK(n.Type() == de::_FP32_ && n.get_data<float>() == 1.5f);
    n = de::Float2Half(0.333251953125f);
    CHECK(n.Type() == de::_FP16_ && n.get_data<de::Half>().val == 0x3555);
    CHECK(sizeof(de::Number) == 32 && sizeof(de::DH) == 104 && sizeof(de::MatrixLayout) == 16);
    CHECK(de::Float2Half(1.0f).val == 0x3c00 && de::Float2Half(-2.0f).val == 0xc000);
    CHECK(de::Float2Half(65520.f).val == 0x7c00 && de::Float2Half(65519.f).val == 0x7bff);
    CHECK(de::Float2Half(1.0f + 0x1p-11f).val == 0x3c00 && de::Float2Half(1.0f + 3 * 0x1p-11f).val == 0x3c02);
    de::Half one; one.val = 0x3c00;
    CHECK(de::Half2Float(one) == 1.0f);
    de::Half sub; sub.val = 0x0001;
    CHECK(de::Half2Float(sub) == 0x1p-24f);

    // status handle; GPU entry points before InitCuda report "CUDA not initialised" (0x16)
    de::ResetLastError();
    CHECK(de::GetLastError()->error_type == 0 && std::string(de::GetLastError()->error_string) == "success: No error");
    de::Matrix& src = de::CreateMatrixRef(de::_FP32_, 8, 8);
    de::GPU_Matrix* none = de::CreateGPUMatrixPtr();
    de::DH r = de::Memcpy(src, *none, de::Point2D(0, 0), de::Point2D(0, 0), de::Point2D(8, 8), de::DECX_MEMCPY_H2D);
    CHECK(r.error_type == decx::DECX_FAIL_CUDA_not_init);
    de::blas::cuda::GEMM(*none, *none, *none);
    CHECK(de::GetLastError()->error_type == decx::DECX_FAIL_CUDA_not_init);
    de::ResetLastError();
    de::blas::cuda::GEMM(src, src, src);
    CHECK(de::GetLastError()->error_type == decx::DECX_FAIL_CUDA_not_init);
    CHECK(de::cuda::PinMemory(src).error_type == decx::DECX_FAIL_CUDA_not_init);
    de::InitCPUInfo();
    de::cpu::DecxSetThreadingNum(4);
    return g_failures;
}

template <typename T> static void fill(de::Matrix& m, T (*f)(int, int))
{
    for (int i = 0; i < (int)m.Height(); ++i) for (int j = 0; j < (int)m.Width(); ++j) *m.ptr<T>(i, j) = f(i, j);
}

static int gpu_checks()
{
    de::InitCPUInfo();
    de::InitCuda();
    de::ResetLastError();
    const de::Point2D O(0, 0);

    // the original sample: A[i][j] = j, B[i][j] = i  =>  every element = sum l^2, l < L
    const uint32_t W = 1013, H = 1077, L = 1005;
    de::Matrix& A = de::CreateMatrixRef(de::_FP32_, L, H);
    de::Matrix& B = de::CreateMatrixRef(de::_FP32_, W, L);
    de::Matrix& D = de::CreateMatrixRef(de::_FP32_, W, H);
    fill<float>(A, [](int, int j) { return (float)j; });
    fill<float>(B, [](int i, int) { return (float)i; });
    de::GPU_Matrix& dA = de::CreateGPUMatrixRef(de::_FP32_, L, H);
    de::GPU_Matrix& dB = de::CreateGPUMatrixRef(de::_FP32_, W, L);
    de::GPU_Matrix& dD = de::CreateGPUMatrixRef();                     // empty: GEMM shapes it
    CHECK(de::Memcpy(A, dA, O, O, de::Point2D(L, H), de::DECX_MEMCPY_H2D).error_type == 0);
    CHECK(de::Memcpy(B, dB, O, O, de::Point2D(W, L), de::DECX_MEMCPY_H2D).error_type == 0);
    de::blas::cuda::GEMM(dA, dB, dD);
    CHECK(de::GetLastError()->error_type == 0);
    CHECK(dD.Width() == W && dD.Height() == H && dD.Type() == de::_FP32_);
    CHECK(de::Memcpy(D, dD, O, O, de::Point2D(W, H), de::DECX_MEMCPY_D2H).error_type == 0);
    double worst = 0;
    for (uint32_t i = 0; i < H; ++i) for (uint32_t j = 0; j < W; ++j)
        worst = std::fmax(worst, std::fabs((double)*D.ptr<float>(i, j) - 337853530.0) / 337853530.0);
    CHECK(worst < 4e-6);

    // pageable host matrices travel through bounce buffers in pieces: sub-regions at offsets, rows wider than a
    // piece (split by columns), page-locked storage (copied directly) and a round trip of each
    {
        const uint32_t WW = 5000011, HH = 3;                                   // 20 MB rows, 60 MB in all
        de::Matrix& wide = de::CreateMatrixRef(de::_INT32_, WW, HH);
        de::Matrix& back = de::CreateMatrixRef(de::_INT32_, WW, HH);
        de::GPU_Matrix& dwide = de::CreateGPUMatrixRef(de::_INT32_, WW, HH);
        for (uint32_t i = 0; i < HH; ++i) for (uint32_t j = 0; j < WW; ++j) *wide.ptr<int>(i, j) = (int)(i * 7919u + j * 31u);
        CHECK(de::Memcpy(wide, dwide, O, O, de::Point2D(WW, HH), de::DECX_MEMCPY_H2D).error_type == 0);
        CHECK(de::Memcpy(back, dwide, O, O, de::Point2D(WW, HH), de::DECX_MEMCPY_D2H).error_type == 0);
        bool same = true;
        for (uint32_t i = 0; i < HH && same; ++i) same = std::memcmp(wide.ptr<int>(i, 0), back.ptr<int>(i, 0), (size_t)WW * 4) == 0;
        CHECK(same);
        const uint32_t TW = 3001, TH = 2999;                                   // 36 MB, copied as an inner region
        de::Matrix& tall = de::CreateMatrixRef(de::_FP32_, TW, TH);
        de::Matrix& tall_back = de::CreateMatrixRef(de::_FP32_, TW, TH);
        de::GPU_Matrix& dtall = de::CreateGPUMatrixRef(de::_FP32_, TW + 10, TH + 10);
        fill<float>(tall, [](int i, int j) { return (float)(i * 3 + j); });
        CHECK(de::Memcpy(tall, dtall, de::Point2D(5, 7), de::Point2D(9, 3), de::Point2D(TW - 5, TH - 7), de::DECX_MEMCPY_H2D).error_type == 0);
        CHECK(de::Memcpy(tall_back, dtall, de::Point2D(9, 3), de::Point2D(5, 7), de::Point2D(TW - 5, TH - 7), de::DECX_MEMCPY_D2H).error_type == 0);
        same = true;
        for (uint32_t i = 7; i < TH && same; ++i) same = std::memcmp(tall.ptr<float>(i, 5), tall_back.ptr<float>(i, 5), (size_t)(TW - 5) * 4) == 0;
        CHECK(same && *tall_back.ptr<float>(0, 0) == 0.f && *tall_back.ptr<float>(6, TW - 1) == 0.f && *tall_back.ptr<float>(TH - 1, 4) == 0.f);
        CHECK(de::cuda::PinMemory(tall).error_type == 0);
        de::Matrix& pinned_back = de::CreateMatrixRef(de::_FP32_, TW, TH);
        CHECK(de::cuda::PinMemory(pinned_back).error_type == 0);
        CHECK(de::Memcpy(tall, dtall, O, O, de::Point2D(TW, TH), de::DECX_MEMCPY_H2D).error_type == 0);
        CHECK(de::Memcpy(pinned_back, dtall, O, O, de::Point2D(TW, TH), de::DECX_MEMCPY_D2H).error_type == 0);
        same = true;
        for (uint32_t i = 0; i < TH && same; ++i) same = std::memcmp(tall.ptr<float>(i, 0), pinned_back.ptr<float>(i, 0), (size_t)TW * 4) == 0;
        CHECK(same);
        wide.release(); back.release(); dwide.release(); tall.release(); tall_back.release(); dtall.release(); pinned_back.release();
    }

    // four-matrix form, alpha = 2, beta = -1, C = ones: 2 * sum - 1; C aliasing dst
    de::GPU_Matrix& dC = de::CreateGPUMatrixRef(de::_FP32_, W, H);
    de::Matrix& C = de::CreateMatrixRef(de::_FP32_, W, H);
    fill<float>(C, [](int, int) { return 1.f; });
    CHECK(de::Memcpy(C, dC, O, O, de::Point2D(W, H), de::DECX_MEMCPY_H2D).error_type == 0);
    de::blas::cuda::GEMM(dA, dB, dC, dC, de::Number(2.f), de::Number(-1.f));
    CHECK(de::GetLastError()->error_type == 0);
    CHECK(de::Memcpy(D, dC, O, O, de::Point2D(W, H), de::DECX_MEMCPY_D2H).error_type == 0);
    worst = 0;
    for (uint32_t i = 0; i < H; ++i) for (uint32_t j = 0; j < W; ++j)
        worst = std::fmax(worst, std::fabs((double)*D.ptr<float>(i, j) - (2 * 337853530.0 - 1)) / 675707059.0);
    CHECK(worst < 4e-6);

    // dst shrinks without reallocation, grows with it; sub-region copies honour both pitches
    de::GPU_Matrix& dS = de::CreateGPUMatrixRef(de::_FP32_, 40, 50);
    de::Matrix& S = de::CreateMatrixRef(de::_FP32_, 40, 50);
    fill<float>(S, [](int i, int j) { return (float)(i * 100 + j); });
    CHECK(de::Memcpy(S, dS, de::Point2D(3, 2), de::Point2D(5, 7), de::Point2D(10, 20), de::DECX_MEMCPY_H2D).error_type == 0);
    de::Matrix& back = de::CreateMatrixRef(de::_FP32_, 40, 50);
    CHECK(de::Memcpy(back, dS, de::Point2D(5, 7), de::Point2D(1, 1), de::Point2D(10, 20), de::DECX_MEMCPY_D2H).error_type == 0);
    bool same = true;
    for (int i = 0; i < 20; ++i) for (int j = 0; j < 10; ++j) same &= (*back.ptr<float>(1 + i, 1 + j) == *S.ptr<float>(2 + i, 3 + j));
    CHECK(same && *back.ptr<float>(0, 0) == 0.f && *back.ptr<float>(21, 11) == 0.f);
    CHECK(de::Memcpy(S, dS, O, O, de::Point2D(41, 50), de::DECX_MEMCPY_H2D).error_type == decx::DECX_FAIL_MEMCPY_OVERRANGED);
    CHECK(de::Memcpy(S, dS, de::Point2D(35, 0), O, de::Point2D(10, 1), de::DECX_MEMCPY_H2D).error_type == decx::DECX_FAIL_MEMCPY_OVERRANGED);

    // error paths: shape, type, scalar type, unsupported type; nothing is launched
    de::ResetLastError();
    de::blas::cuda::GEMM(dA, dA, dD);                                   // 1005 != 1077
    CHECK(de::GetLastError()->error_type == decx::DECX_FAIL_DimsNotMatching);
    de::ResetLastError();
    de::GPU_Matrix& dH = de::CreateGPUMatrixRef(de::_FP16_, W, L);
    de::blas::cuda::GEMM(dA, dH, dD);
    CHECK(de::GetLastError()->error_type == decx::DECX_FAIL_TYPE_MOT_MATCH);
    de::ResetLastError();
    de::blas::cuda::GEMM(dA, dB, dC, dD, de::Number(1.0), de::Number(1.f));    // alpha is fp64
    CHECK(de::GetLastError()->error_type == decx::DECX_FAIL_TYPE_MOT_MATCH);
    de::ResetLastError();
    de::blas::cuda::GEMM(dA, dB, dS, dD, de::Number(1.f), de::Number(1.f));    // C has the wrong shape
    CHECK(de::GetLastError()->error_type == decx::DECX_FAIL_DimsNotMatching);
    de::ResetLastError();
    de::GPU_Matrix& dint = de::CreateGPUMatrixRef(de::_INT32_, 8, 8);
    de::blas::cuda::GEMM(dint, dint, dD);
    CHECK(de::GetLastError()->error_type == decx::DECX_FAIL_UNSUPPORTED_TYPE);
    de::ResetLastError();
    // complex single precision: (1 + i) I . X = (1 + i) X, then alpha = i, beta = 2: i (1 + i) X + 2 X = (1 + i) X
    de::Matrix& Ic = de::CreateMatrixRef(de::_COMPLEX_F32_, 20, 20);
    de::Matrix& Xc = de::CreateMatrixRef(de::_COMPLEX_F32_, 9, 20);
    for (int i = 0; i < 20; ++i) { *Ic.ptr<de::CPf>(i, i) = de::CPf(1.f, 1.f); for (int j = 0; j < 9; ++j) *Xc.ptr<de::CPf>(i, j) = de::CPf((float)(i - 7), (float)(2 * j - 5)); }
    CHECK(Xc.ptr<de::CPf>(1, 0) - Xc.ptr<de::CPf>(0, 0) == 12);                               // 32-byte rule: 4 complex
    de::GPU_Matrix& dIc = de::CreateGPUMatrixRef(de::_COMPLEX_F32_, 20, 20);
    de::GPU_Matrix& dXc = de::CreateGPUMatrixRef(de::_COMPLEX_F32_, 9, 20);
    de::GPU_Matrix& dRc = de::CreateGPUMatrixRef();
    CHECK(de::Memcpy(Ic, dIc, O, O, de::Point2D(20, 20), de::DECX_MEMCPY_H2D).error_type == 0);
    CHECK(de::Memcpy(Xc, dXc, O, O, de::Point2D(9, 20), de::DECX_MEMCPY_H2D).error_type == 0);
    de::blas::cuda::GEMM(dIc, dXc, dRc);
    CHECK(de::GetLastError()->error_type == 0 && dRc.Type() == de::_COMPLEX_F32_ && dRc.Width() == 9 && dRc.Height() == 20);
    de::Matrix& Rc = de::CreateMatrixRef(de::_COMPLEX_F32_, 9, 20);
    CHECK(de::Memcpy(Rc, dRc, O, O, de::Point2D(9, 20), de::DECX_MEMCPY_D2H).error_type == 0);
    bool samec = true;
    for (int i = 0; i < 20; ++i) for (int j = 0; j < 9; ++j) {
        const de::CPf x = *Xc.ptr<de::CPf>(i, j), r = *Rc.ptr<de::CPf>(i, j);
        samec &= (r.real == x.real - x.image) && (r.image == x.real + x.image);
    }
    CHECK(samec);
    de::blas::cuda::GEMM(dIc, dXc, dXc, dRc, de::Number(de::CPf(0.f, 1.f)), de::Number(de::CPf(2.f, 0.f)));
    CHECK(de::GetLastError()->error_type == 0);
    CHECK(de::Memcpy(Rc, dRc, O, O, de::Point2D(9, 20), de::DECX_MEMCPY_D2H).error_type == 0);
    samec = true;
    for (int i = 0; i < 20; ++i) for (int j = 0; j < 9; ++j) {
        const de::CPf x = *Xc.ptr<de::CPf>(i, j), r = *Rc.ptr<de::CPf>(i, j);
        samec &= (r.real == x.real - x.image) && (r.image == x.real + x.image);
    }
    CHECK(samec);
    de::blas::cuda::GEMM(Ic, Xc, Rc);                                                         // host-matrix form: real types only
    CHECK(de::GetLastError()->error_type == decx::DECX_FAIL_UNSUPPORTED_TYPE);
    de::ResetLastError();
    // double precision: identity, and alpha / beta carried as doubles
    de::Matrix& I64 = de::CreateMatrixRef(de::_FP64_, 24, 24);
    de::Matrix& X64 = de::CreateMatrixRef(de::_FP64_, 17, 24);
    for (int i = 0; i < 24; ++i) { *I64.ptr<double>(i, i) = 1.0; for (int j = 0; j < 17; ++j) *X64.ptr<double>(i, j) = 1.0 / 3.0 + i * 17 + j; }
    CHECK(I64.ptr<double>(1, 0) - I64.ptr<double>(0, 0) == 24 && X64.ptr<double>(1, 0) - X64.ptr<double>(0, 0) == 20);   // 32-byte rule
    de::GPU_Matrix& dI64 = de::CreateGPUMatrixRef(de::_FP64_, 24, 24);
    de::GPU_Matrix& dX64 = de::CreateGPUMatrixRef(de::_FP64_, 17, 24);
    de::GPU_Matrix& dR64 = de::CreateGPUMatrixRef();
    CHECK(de::Memcpy(I64, dI64, O, O, de::Point2D(24, 24), de::DECX_MEMCPY_H2D).error_type == 0);
    CHECK(de::Memcpy(X64, dX64, O, O, de::Point2D(17, 24), de::DECX_MEMCPY_H2D).error_type == 0);
    de::blas::cuda::GEMM(dI64, dX64, dX64, dR64, de::Number(2.0), de::Number(-0.5));        // 2 I X - X / 2 = 1.5 X
    CHECK(de::GetLastError()->error_type == 0 && dR64.Type() == de::_FP64_ && dR64.Width() == 17 && dR64.Height() == 24);
    de::Matrix& R64 = de::CreateMatrixRef(de::_FP64_, 17, 24);
    CHECK(de::Memcpy(R64, dR64, O, O, de::Point2D(17, 24), de::DECX_MEMCPY_D2H).error_type == 0);
    bool same64 = true;
    for (int i = 0; i < 24; ++i) for (int j = 0; j < 17; ++j) same64 &= (*R64.ptr<double>(i, j) == 1.5 * *X64.ptr<double>(i, j));
    CHECK(same64);
    de::blas::cuda::GEMM(dI64, dX64, dX64, dR64, de::Number(2.0f), de::Number(-0.5f));      // float scalars for double matrices
    CHECK(de::GetLastError()->error_type == decx::DECX_FAIL_TYPE_MOT_MATCH);
    de::ResetLastError();
    de::ResetLastError();
    CHECK(de::Memcpy(A, dH, O, O, de::Point2D(1, 1), de::DECX_MEMCPY_H2D).error_type == decx::DECX_FAIL_TYPE_MOT_MATCH);
    CHECK(dD.Width() == W && dD.Height() == H);                          // failed calls left dst alone

    // fp16 through the objects: ones(64 x 96) . ones(96 x 32) = 96, alpha/beta as de::Half
    de::Matrix& hA = de::CreateMatrixRef(de::_FP16_, 96, 64);
    de::Matrix& hB = de::CreateMatrixRef(de::_FP16_, 32, 96);
    de::Matrix& hD = de::CreateMatrixRef(de::_FP16_, 32, 64);
    fill<de::Half>(hA, [](int, int) { de::Half h; h.val = 0x3c00; return h; });
    fill<de::Half>(hB, [](int, int) { de::Half h; h.val = 0x3c00; return h; });
    de::GPU_Matrix& gA = de::CreateGPUMatrixRef(de::_FP16_, 96, 64);
    de::GPU_Matrix& gB = de::CreateGPUMatrixRef(de::_FP16_, 32, 96);
    de::GPU_Matrix& gD = de::CreateGPUMatrixRef(de::_FP16_, 32, 64);
    de::Memcpy(hA, gA, O, O, de::Point2D(96, 64), de::DECX_MEMCPY_H2D);
    de::Memcpy(hB, gB, O, O, de::Point2D(32, 96), de::DECX_MEMCPY_H2D);
    de::blas::cuda::GEMM(gA, gB, gD);
    de::blas::cuda::GEMM(gA, gB, gD, gD, de::Number(de::Float2Half(0.5f)), de::Number(de::Float2Half(2.f)));   // 48 + 192
    CHECK(de::GetLastError()->error_type == 0);
    de::Memcpy(hD, gD, O, O, de::Point2D(32, 64), de::DECX_MEMCPY_D2H);
    bool ok = true;
    for (int i = 0; i < 64; ++i) for (int j = 0; j < 32; ++j) ok &= (de::Half2Float(*hD.ptr<de::Half>(i, j)) == 240.f);
    CHECK(ok);

    // single columns (stored dense on the device): y = M x with exact small integers, a copy into the column between
    // two products is what the next product multiplies, the result column feeds the next product, sub-region copies
    // of a column, a column as the LEFT operand (outer product) and as C
    {
        const uint32_t R = 300, Kc = 5000;
        de::Matrix& Mh = de::CreateMatrixRef(de::_FP32_, Kc, R);
        de::Matrix& xh = de::CreateMatrixRef(de::_FP32_, 1, Kc);
        de::Matrix& yh = de::CreateMatrixRef(de::_FP32_, 1, R);
        fill<float>(Mh, [](int i, int j) { return (float)((i + 2 * j) % 5 - 2); });
        fill<float>(xh, [](int i, int) { return (float)(i % 3 - 1); });
        de::GPU_Matrix& dM = de::CreateGPUMatrixRef(de::_FP32_, Kc, R);
        de::GPU_Matrix& dx = de::CreateGPUMatrixRef(de::_FP32_, 1, Kc);
        de::GPU_Matrix& dy = de::CreateGPUMatrixRef();
        CHECK(de::Memcpy(Mh, dM, O, O, de::Point2D(Kc, R), de::DECX_MEMCPY_H2D).error_type == 0);
        CHECK(de::Memcpy(xh, dx, O, O, de::Point2D(1u, Kc), de::DECX_MEMCPY_H2D).error_type == 0);
        auto expect = [&](const de::Matrix& x, uint32_t row) {
            double s = 0;
            for (uint32_t k = 0; k < Kc; ++k) s += (double)*Mh.ptr<float>(row, k) * (double)*const_cast<de::Matrix&>(x).ptr<float>(k, 0);
            return (float)s;
        };
        de::blas::cuda::GEMM(dM, dx, dy);
        CHECK(de::GetLastError()->error_type == 0 && dy.Width() == 1 && dy.Height() == R);
        CHECK(de::Memcpy(yh, dy, O, O, de::Point2D(1u, R), de::DECX_MEMCPY_D2H).error_type == 0);
        bool okc = true;
        for (uint32_t i = 0; i < R; ++i) okc &= (*yh.ptr<float>(i, 0) == expect(xh, i));
        CHECK(okc);
        // rows 100 .. 2099 of the column change on the device: the next product sees them
        de::Matrix& patch = de::CreateMatrixRef(de::_FP32_, 1, 2000);
        fill<float>(patch, [](int i, int) { return (float)(i % 7 - 3); });
        CHECK(de::Memcpy(patch, dx, O, de::Point2D(0, 100), de::Point2D(1, 2000), de::DECX_MEMCPY_H2D).error_type == 0);
        for (uint32_t k = 0; k < 2000; ++k) *xh.ptr<float>(100 + k, 0) = *patch.ptr<float>(k, 0);
        de::blas::cuda::GEMM(dM, dx, dy);
        CHECK(de::Memcpy(yh, dy, O, O, de::Point2D(1u, R), de::DECX_MEMCPY_D2H).error_type == 0);
        okc = true;
        for (uint32_t i = 0; i < R; ++i) okc &= (*yh.ptr<float>(i, 0) == expect(xh, i));
        CHECK(okc);
        // ... and reads back what was written, from an offset
        de::Matrix& xback = de::CreateMatrixRef(de::_FP32_, 1, Kc);
        CHECK(de::Memcpy(xback, dx, de::Point2D(0, 50), de::Point2D(0, 50), de::Point2D(1u, Kc - 50), de::DECX_MEMCPY_D2H).error_type == 0);
        okc = *xback.ptr<float>(49, 0) == 0.f;
        for (uint32_t k = 50; k < Kc; ++k) okc &= (*xback.ptr<float>(k, 0) == *xh.ptr<float>(k, 0));
        CHECK(okc);
        // the result column as the next product's vector: z = T y, T 40 x 300 of ones and minus ones; y as C: T y + 2 z0
        de::Matrix& Th = de::CreateMatrixRef(de::_FP32_, R, 40);
        fill<float>(Th, [](int i, int j) { return (i + j) % 2 ? 1.f : -1.f; });
        de::GPU_Matrix& dT = de::CreateGPUMatrixRef(de::_FP32_, R, 40);
        de::GPU_Matrix& dz = de::CreateGPUMatrixRef();
        CHECK(de::Memcpy(Th, dT, O, O, de::Point2D(R, 40u), de::DECX_MEMCPY_H2D).error_type == 0);
        de::blas::cuda::GEMM(dT, dy, dz);
        CHECK(de::GetLastError()->error_type == 0 && dz.Width() == 1 && dz.Height() == 40);
        de::Matrix& zh = de::CreateMatrixRef(de::_FP32_, 1, 40);
        CHECK(de::Memcpy(zh, dz, O, O, de::Point2D(1, 40), de::DECX_MEMCPY_D2H).error_type == 0);
        okc = true;
        for (uint32_t i = 0; i < 40; ++i) {
            double s = 0;
            for (uint32_t k = 0; k < R; ++k) s += (double)*Th.ptr<float>(i, k) * (double)*yh.ptr<float>(k, 0);
            okc &= (*zh.ptr<float>(i, 0) == (float)s);
        }
        CHECK(okc);
        de::blas::cuda::GEMM(dT, dy, dz, dz, de::Number(1.f), de::Number(2.f));            // C = dst = the column z
        de::Matrix& z2 = de::CreateMatrixRef(de::_FP32_, 1, 40);
        CHECK(de::Memcpy(z2, dz, O, O, de::Point2D(1, 40), de::DECX_MEMCPY_D2H).error_type == 0);
        okc = true;
        for (uint32_t i = 0; i < 40; ++i) okc &= (*z2.ptr<float>(i, 0) == 3.f * *zh.ptr<float>(i, 0));
        CHECK(okc);
        // outer product: the column z (40 x 1) times a row (1 x 33)
        de::Matrix& rowh = de::CreateMatrixRef(de::_FP32_, 33, 1);
        fill<float>(rowh, [](int, int j) { return (float)(j - 16); });
        de::GPU_Matrix& drow = de::CreateGPUMatrixRef(de::_FP32_, 33, 1);
        de::GPU_Matrix& douter = de::CreateGPUMatrixRef();
        CHECK(de::Memcpy(rowh, drow, O, O, de::Point2D(33, 1), de::DECX_MEMCPY_H2D).error_type == 0);
        de::blas::cuda::GEMM(dz, drow, douter);
        CHECK(de::GetLastError()->error_type == 0 && douter.Width() == 33 && douter.Height() == 40);
        de::Matrix& outerh = de::CreateMatrixRef(de::_FP32_, 33, 40);
        CHECK(de::Memcpy(outerh, douter, O, O, de::Point2D(33, 40), de::DECX_MEMCPY_D2H).error_type == 0);
        okc = true;
        for (uint32_t i = 0; i < 40; ++i) for (uint32_t j = 0; j < 33; ++j) okc &= (*outerh.ptr<float>(i, j) == *z2.ptr<float>(i, 0) * (float)((int)j - 16));
        CHECK(okc);
        // fp16 column: ones(64 x 4096) . halves of 0.5 = 2048
        de::Matrix& hM = de::CreateMatrixRef(de::_FP16_, 4096, 64);
        de::Matrix& hx = de::CreateMatrixRef(de::_FP16_, 1, 4096);
        fill<de::Half>(hM, [](int, int) { de::Half h; h.val = 0x3c00; return h; });
        fill<de::Half>(hx, [](int, int) { de::Half h; h.val = 0x3800; return h; });
        de::GPU_Matrix& ghM = de::CreateGPUMatrixRef(de::_FP16_, 4096, 64);
        de::GPU_Matrix& ghx = de::CreateGPUMatrixRef(de::_FP16_, 1, 4096);
        de::GPU_Matrix& ghy = de::CreateGPUMatrixRef();
        de::Memcpy(hM, ghM, O, O, de::Point2D(4096, 64), de::DECX_MEMCPY_H2D);
        de::Memcpy(hx, ghx, O, O, de::Point2D(1, 4096), de::DECX_MEMCPY_H2D);
        de::blas::cuda::GEMM(ghM, ghx, ghy);
        de::Matrix& hy = de::CreateMatrixRef(de::_FP16_, 1, 64);
        CHECK(de::Memcpy(hy, ghy, O, O, de::Point2D(1, 64), de::DECX_MEMCPY_D2H).error_type == 0);
        okc = true;
        for (int i = 0; i < 64; ++i) okc &= (de::Half2Float(*hy.ptr<de::Half>(i, 0)) == 2048.f);
        CHECK(okc);
    }

    // host-matrix overload and pinned staging
    de::Matrix& I = de::CreateMatrixRef(de::_FP32_, 50, 50);
    fill<float>(I, [](int i, int j) { return i == j ? 1.f : 0.f; });
    de::Matrix& R = de::CreateMatrixRef();
    CHECK(de::cuda::PinMemory(S).error_type == 0);
    CHECK(de::cuda::PinMemory(S).error_type == decx::DECX_FAIL_HOST_MEM_REGISTERED);
    de::blas::cuda::GEMM(I, S, R);                                       // I(50x50) . S(50 rows x 40 cols)
    CHECK(de::GetLastError()->error_type == 0 && R.Width() == 40 && R.Height() == 50);
    same = true;
    for (int i = 0; i < 50; ++i) for (int j = 0; j < 40; ++j) same &= (*R.ptr<float>(i, j) == *S.ptr<float>(i, j));
    CHECK(same);
    de::blas::cuda::GEMM(I, S, S, R);                                    // + C
    same = true;
    for (int i = 0; i < 50; ++i) for (int j = 0; j < 40; ++j) same &= (*R.ptr<float>(i, j) == 2 * *S.ptr<float>(i, j));
    CHECK(same);
    CHECK(de::cuda::UnpinMemory(S).error_type == 0);
    CHECK(de::cuda::UnpinMemory(S).error_type == decx::DECX_FAIL_HOST_MEM_UNREGISTERED);
    de::cuda::DECX_CUDA_exit();
    return g_failures;
}

static int vector_host_checks()
{
    // storage rule of vectors: length rounded up to 32 bytes, zero-filled, 32-byte aligned
    de::Vector& v = de::CreateVectorRef(de::_FP32_, 13);
    CHECK(v.Len() == 13 && v.Type() == de::_FP32_ && ((uintptr_t)v.ptr<float>(0) & 31u) == 0);
    bool zero = true;
    for (int i = 0; i < 16; ++i) zero &= (*v.ptr<float>(i) == 0.f);          // 13 -> 16 elements allocated
    CHECK(zero);
    de::Vector* e = de::CreateVectorPtr();
    CHECK(e->Len() == 0 && e->Type() == de::_VOID_);
    de::Vector& alias = de::CreateVectorRef();
    alias.SoftCopy(v);
    *v.ptr<float>(5) = 7.f;
    CHECK(alias.Len() == 13 && *alias.ptr<float>(5) == 7.f);
    v.release();
    CHECK(*alias.ptr<float>(5) == 7.f);
    alias.Reinterpret(de::_INT32_);
    CHECK(alias.Type() == de::_INT32_ && alias.Len() == 13);
    CHECK(de::Fp16_Accurate_L1 == 0 && de::Fp16_Accurate_L2 == 1 && de::Fp16_Accurate_L3 == 2);

    // without InitCuda every GPU-facing vector call reports 0x16 and does nothing else
    de::Vector& x = de::CreateVectorRef(de::_FP32_, 4);
    de::Vector& y = de::CreateVectorRef(de::_FP32_, 4);
    de::Matrix& m = de::CreateMatrixRef(de::_FP32_, 4, 4);
    de::GPU_Vector& g = de::CreateGPUVectorRef();
    CHECK(de::Memcpy(x, g, 0, 0, 4, de::DECX_MEMCPY_H2D).error_type == decx::DECX_FAIL_CUDA_not_init);
    de::blas::cuda::GEMM(x, m, y);
    CHECK(de::GetLastError()->error_type == decx::DECX_FAIL_CUDA_not_init);
    de::blas::cuda::GEMM(m, x, y);
    CHECK(de::GetLastError()->error_type == decx::DECX_FAIL_CUDA_not_init);
    CHECK(de::cuda::PinMemory(x).error_type == decx::DECX_FAIL_CUDA_not_init);
    de::ResetLastError();
    return g_failures;
}

static int vector_gpu_checks()
{
    de::InitCuda();
    de::ResetLastError();
    // transfers with offsets, and their range / type checks
    de::Vector& a = de::CreateVectorRef(de::_FP32_, 100);
    de::Vector& b = de::CreateVectorRef(de::_FP32_, 100);
    for (int i = 0; i < 100; ++i) *a.ptr<float>(i) = (float)i;
    de::GPU_Vector& g = de::CreateGPUVectorRef(de::_FP32_, 60);
    CHECK(g.Len() == 60 && g.Type() == de::_FP32_);
    CHECK(de::Memcpy(a, g, 10, 20, 30, de::DECX_MEMCPY_H2D).error_type == 0);        // a[10..40) -> g[20..50)
    CHECK(de::Memcpy(b, g, 0, 5, 60, de::DECX_MEMCPY_D2H).error_type == 0);          // g[0..60)  -> b[5..65)
    bool same = true;
    for (int i = 0; i < 100; ++i) {
        const float want = (i >= 25 && i < 55) ? (float)(i - 25 + 10) : 0.f;         // device storage starts zeroed
        same &= (*b.ptr<float>(i) == want);
    }
    CHECK(same);
    CHECK(de::Memcpy(a, g, 0, 31, 30, de::DECX_MEMCPY_H2D).error_type == decx::DECX_FAIL_MEMCPY_OVERRANGED);
    CHECK(de::Memcpy(a, g, 90, 0, 11, de::DECX_MEMCPY_H2D).error_type == decx::DECX_FAIL_MEMCPY_OVERRANGED);
    CHECK(de::Memcpy(b, g, 41, 0, 20, de::DECX_MEMCPY_D2H).error_type == decx::DECX_FAIL_MEMCPY_OVERRANGED);
    de::GPU_Vector& gh = de::CreateGPUVectorRef(de::_FP16_, 60);
    CHECK(de::Memcpy(a, gh, 0, 0, 1, de::DECX_MEMCPY_H2D).error_type == decx::DECX_FAIL_TYPE_MOT_MATCH);
    de::GPU_Vector& galias = de::CreateGPUVectorRef();
    galias.SoftCopy(g);
    g.release();
    CHECK(galias.Len() == 60 && de::Memcpy(b, galias, 20, 0, 1, de::DECX_MEMCPY_D2H).error_type == 0 && *b.ptr<float>(0) == 10.f);

    // closed forms: ones . M sums columns, M . ones sums rows (small integers: exact)
    const uint32_t W = 300, H = 200;
    de::Matrix& M = de::CreateMatrixRef(de::_FP32_, W, H);
    for (uint32_t i = 0; i < H; ++i) for (uint32_t j = 0; j < W; ++j) *M.ptr<float>(i, j) = (float)((int)((i * 7 + j * 3) % 11) - 5);
    de::Vector& onesH = de::CreateVectorRef(de::_FP32_, H);
    de::Vector& onesW = de::CreateVectorRef(de::_FP32_, W);
    for (uint32_t i = 0; i < H; ++i) *onesH.ptr<float>(i) = 1.f;
    for (uint32_t j = 0; j < W; ++j) *onesW.ptr<float>(j) = 1.f;
    de::Vector& cols = de::CreateVectorRef();                                        // empty: created by the call
    de::blas::cuda::GEMM(onesH, M, cols);
    CHECK(de::GetLastError()->error_type == 0 && cols.Len() == W && cols.Type() == de::_FP32_);
    same = true;
    for (uint32_t j = 0; j < W; ++j) { float s = 0; for (uint32_t i = 0; i < H; ++i) s += *M.ptr<float>(i, j); same &= (*cols.ptr<float>(j) == s); }
    CHECK(same);
    de::Vector& rows = de::CreateVectorRef(de::_FP32_, H);                           // exact size: storage kept
    float* before = rows.ptr<float>(0);
    de::blas::cuda::GEMM(M, onesW, rows);
    CHECK(de::GetLastError()->error_type == 0 && rows.Len() == H && rows.ptr<float>(0) == before);
    same = true;
    for (uint32_t i = 0; i < H; ++i) { float s = 0; for (uint32_t j = 0; j < W; ++j) s += *M.ptr<float>(i, j); same &= (*rows.ptr<float>(i) == s); }
    CHECK(same);

    // fp16: level 1 gives an fp32 result, level 2 an fp16 one
    de::Matrix& Mh = de::CreateMatrixRef(de::_FP16_, W, H);
    for (uint32_t i = 0; i < H; ++i) for (uint32_t j = 0; j < W; ++j) *Mh.ptr<de::Half>(i, j) = de::Float2Half((float)((int)((i + j) % 5) - 2));
    de::Vector& hx = de::CreateVectorRef(de::_FP16_, W);
    for (uint32_t j = 0; j < W; ++j) *hx.ptr<de::Half>(j) = de::Float2Half((float)((int)(j % 3) - 1));
    de::Vector& r1 = de::CreateVectorRef();
    de::Vector& r2 = de::CreateVectorRef();
    de::blas::cuda::GEMM(Mh, hx, r1, de::Fp16_Accurate_L1);
    CHECK(de::GetLastError()->error_type == 0 && r1.Len() == H && r1.Type() == de::_FP32_);
    de::blas::cuda::GEMM(Mh, hx, r2, de::Fp16_Accurate_L2);
    CHECK(de::GetLastError()->error_type == 0 && r2.Len() == H && r2.Type() == de::_FP16_);
    same = true;
    for (uint32_t i = 0; i < H; ++i) {
        float s = 0;
        for (uint32_t j = 0; j < W; ++j) s += (float)((int)((i + j) % 5) - 2) * (float)((int)(j % 3) - 1);
        same &= (*r1.ptr<float>(i) == s) && (de::Half2Float(*r2.ptr<de::Half>(i)) == s);
    }
    CHECK(same);

    // error paths: nothing is launched, dst is left alone
    de::Vector& shortv = de::CreateVectorRef(de::_FP32_, W - 1);
    de::blas::cuda::GEMM(M, shortv, rows);
    CHECK(de::GetLastError()->error_type == decx::DECX_FAIL_DimsNotMatching);
    de::blas::cuda::GEMM(onesW, M, cols);                                            // needs H elements
    CHECK(de::GetLastError()->error_type == decx::DECX_FAIL_DimsNotMatching);
    de::blas::cuda::GEMM(Mh, onesW, rows);
    CHECK(de::GetLastError()->error_type == decx::DECX_FAIL_TYPE_MOT_MATCH);
    de::Matrix& Mi = de::CreateMatrixRef(de::_INT32_, W, H);
    de::Vector& vi = de::CreateVectorRef(de::_INT32_, W);
    de::blas::cuda::GEMM(Mi, vi, rows);
    CHECK(de::GetLastError()->error_type == decx::DECX_FAIL_UNSUPPORTED_TYPE);
    de::Vector& none = de::CreateVectorRef();
    de::blas::cuda::GEMM(M, none, rows);
    CHECK(de::GetLastError()->error_type == decx::DECX_FAIL_CLASS_NOT_INIT);
    de::blas::cuda::GEMM(Mh, hx, r2, 3);
    CHECK(de::GetLastError()->error_type == decx::DECX_FAIL_INVALID_PARAM);
    de::blas::cuda::GEMM(M, onesW, rows);                                            // and a good call clears the status
    CHECK(de::GetLastError()->error_type == 0);

    // pinned host vectors behave the same
    CHECK(de::cuda::PinMemory(onesW).error_type == 0);
    CHECK(de::cuda::PinMemory(onesW).error_type == decx::DECX_FAIL_HOST_MEM_REGISTERED);
    de::blas::cuda::GEMM(M, onesW, rows);
    CHECK(de::GetLastError()->error_type == 0 && *onesW.ptr<float>(W - 1) == 1.f);
    CHECK(de::cuda::UnpinMemory(onesW).error_type == 0);
    CHECK(de::cuda::UnpinMemory(onesW).error_type == decx::DECX_FAIL_HOST_MEM_UNREGISTERED);
    de::cuda::DECX_CUDA_exit();
    return g_failures;
}

template <typename T> static int vmm_files(const std::string& dir, de::_DATA_TYPES_FLAGS_ ty, bool mat_times_vec,
                                           uint32_t W, uint32_t H, uint32_t level)
{
    de::InitCuda();
    de::ResetLastError();
    de::Matrix& M = de::CreateMatrixRef(ty, W, H);
    de::Vector& V = de::CreateVectorRef(ty, mat_times_vec ? W : H);
    de::Vector& Y = de::CreateVectorRef();
    std::ifstream fm(dir + "/M.bin", std::ios::binary), fv(dir + "/V.bin", std::ios::binary);
    if (!fm || !fv) return 2;
    for (uint32_t i = 0; i < H; ++i) fm.read((char*)M.ptr<T>(i, 0), (std::streamsize)W * sizeof(T));
    fv.read((char*)V.ptr<T>(0), (std::streamsize)V.Len() * sizeof(T));
    if (!fm || !fv) return 2;
    if (mat_times_vec) de::blas::cuda::GEMM(M, V, Y, level); else de::blas::cuda::GEMM(V, M, Y, level);
    if (de::GetLastError()->error_type != 0) { std::cerr << de::GetLastError()->error_string << "\n"; return 3; }
    const size_t es = Y.Type() == de::_FP32_ ? 4 : 2;
    if (Y.Len() != (mat_times_vec ? H : W)) return 4;
    std::ofstream out(dir + "/Y.bin", std::ios::binary);
    out.write((const char*)Y.ptr<char>(0), (std::streamsize)(Y.Len() * es));
    return out ? 0 : 2;
}

template <typename T> static bool read_into(de::Matrix& m, const std::string& path)
{
    std::ifstream f(path, std::ios::binary);
    if (!f) return false;
    for (uint32_t i = 0; i < m.Height(); ++i) f.read((char*)m.ptr<T>(i, 0), (std::streamsize)m.Width() * sizeof(T));
    return (bool)f;
}

template <typename T> static int gemm_files(const std::string& dir, de::_DATA_TYPES_FLAGS_ ty, uint32_t M, uint32_t N,
                                            uint32_t K, bool with_c, float alpha, float beta)
{
    de::InitCuda();
    de::ResetLastError();
    const de::Point2D O(0, 0);
    de::Matrix& A = de::CreateMatrixRef(ty, K, M);
    de::Matrix& B = de::CreateMatrixRef(ty, N, K);
    de::Matrix& C = de::CreateMatrixRef(ty, N, M);
    de::Matrix& D = de::CreateMatrixRef(ty, N, M);
    if (!read_into<T>(A, dir + "/A.bin") || !read_into<T>(B, dir + "/B.bin")) return 2;
    if (with_c && !read_into<T>(C, dir + "/C.bin")) return 2;
    de::GPU_Matrix& dA = de::CreateGPUMatrixRef(ty, K, M);
    de::GPU_Matrix& dB = de::CreateGPUMatrixRef(ty, N, K);
    de::GPU_Matrix& dC = de::CreateGPUMatrixRef(ty, N, M);
    de::GPU_Matrix& dD = de::CreateGPUMatrixRef(ty, N, M);
    de::Memcpy(A, dA, O, O, de::Point2D(K, M), de::DECX_MEMCPY_H2D);
    de::Memcpy(B, dB, O, O, de::Point2D(N, K), de::DECX_MEMCPY_H2D);
    if (with_c) {
        de::Memcpy(C, dC, O, O, de::Point2D(N, M), de::DECX_MEMCPY_H2D);
        if (ty == de::_FP32_) de::blas::cuda::GEMM(dA, dB, dC, dD, de::Number(alpha), de::Number(beta));
        else if (ty == de::_FP64_) de::blas::cuda::GEMM(dA, dB, dC, dD, de::Number((double)alpha), de::Number((double)beta));
        else de::blas::cuda::GEMM(dA, dB, dC, dD, de::Number(de::Float2Half(alpha)), de::Number(de::Float2Half(beta)));
    } else {
        de::blas::cuda::GEMM(dA, dB, dD);
    }
    if (de::GetLastError()->error_type != 0) { std::cerr << de::GetLastError()->error_string << "\n"; return 3; }
    de::Memcpy(D, dD, O, O, de::Point2D(N, M), de::DECX_MEMCPY_D2H);
    std::ofstream out(dir + "/D.bin", std::ios::binary);
    for (uint32_t i = 0; i < M; ++i) out.write((const char*)D.ptr<T>(i, 0), (std::streamsize)N * sizeof(T));
    return out ? 0 : 2;
}

// Several host threads call GEMM and Memcpy at the same time, each on matrices of its own.  The original allows one
// caller at a time; this module serialises them, so every thread must get its own product, bit for bit what the same
// call gave before the threads started.  (The last-error handle is one per process, as in the original: with several
// callers it says what the latest of them did, so the threads look at their results, not at it.)
struct ThreadJob {
    de::_DATA_TYPES_FLAGS_ type; uint32_t M, N, K; bool with_c;
    de::Matrix *A, *B, *C, *D; de::GPU_Matrix *dA, *dB, *dC, *dD;
    std::vector<char> want;
};
static size_t elem_size(de::_DATA_TYPES_FLAGS_ t) { return t == de::_FP64_ ? 8 : t == de::_FP16_ ? 2 : 4; }
static void put(de::Matrix& m, de::_DATA_TYPES_FLAGS_ t, uint32_t i, uint32_t j, float v)
{
    if (t == de::_FP32_) *m.ptr<float>(i, j) = v;
    else if (t == de::_FP64_) *m.ptr<double>(i, j) = v;
    else *m.ptr<de::Half>(i, j) = de::Float2Half(v);
}
static void run_job(ThreadJob& jb)
{
    if (!jb.with_c) { de::blas::cuda::GEMM(*jb.dA, *jb.dB, *jb.dD); return; }
    if (jb.type == de::_FP32_) de::blas::cuda::GEMM(*jb.dA, *jb.dB, *jb.dC, *jb.dD, de::Number(0.75f), de::Number(-1.25f));
    else if (jb.type == de::_FP64_) de::blas::cuda::GEMM(*jb.dA, *jb.dB, *jb.dC, *jb.dD, de::Number(0.75), de::Number(-1.25));
    else de::blas::cuda::GEMM(*jb.dA, *jb.dB, *jb.dC, *jb.dD, de::Number(de::Float2Half(0.75f)), de::Number(de::Float2Half(-1.25f)));
}
static std::vector<char> fetch(ThreadJob& jb)
{
    const de::Point2D O(0, 0);
    de::Memcpy(*jb.D, *jb.dD, O, O, de::Point2D(jb.N, jb.M), de::DECX_MEMCPY_D2H);
    const size_t row = (size_t)jb.N * elem_size(jb.type);
    std::vector<char> out((size_t)jb.M * row);
    for (uint32_t i = 0; i < jb.M; ++i) {
        const void* src = jb.type == de::_FP32_ ? (const void*)jb.D->ptr<float>(i, 0)
                        : jb.type == de::_FP64_ ? (const void*)jb.D->ptr<double>(i, 0) : (const void*)jb.D->ptr<de::Half>(i, 0);
        std::memcpy(out.data() + i * row, src, row);
    }
    return out;
}
static int threads_checks()
{
    de::InitCPUInfo();
    de::InitCuda();
    de::ResetLastError();
    const de::Point2D O(0, 0);
    // a product split along K, a ragged one with a C term, fp16, fp64, and the two vector corners with their workspaces
    ThreadJob jobs[] = {{de::_FP32_, 300, 300, 8192, false}, {de::_FP32_, 1000, 1500, 777, true}, {de::_FP16_, 257, 130, 515, true},
                        {de::_FP64_, 500, 300, 333, true}, {de::_FP32_, 1100, 1, 8200, false}, {de::_FP16_, 1, 513, 33000, false}};
    const int n_jobs = (int)(sizeof jobs / sizeof jobs[0]);
    for (int t = 0; t < n_jobs; ++t) {
        ThreadJob& jb = jobs[t];
        jb.A = &de::CreateMatrixRef(jb.type, jb.K, jb.M); jb.B = &de::CreateMatrixRef(jb.type, jb.N, jb.K);
        jb.C = &de::CreateMatrixRef(jb.type, jb.N, jb.M); jb.D = &de::CreateMatrixRef(jb.type, jb.N, jb.M);
        // small multiples of 1/8: exact in half, different from job to job
        for (uint32_t i = 0; i < jb.M; ++i) for (uint32_t k = 0; k < jb.K; ++k) put(*jb.A, jb.type, i, k, (float)((int)((i * 7u + k * 13u + t) % 17u) - 8) / 8.f);
        for (uint32_t k = 0; k < jb.K; ++k) for (uint32_t j = 0; j < jb.N; ++j) put(*jb.B, jb.type, k, j, (float)((int)((k * 5u + j * 11u + 3u * t) % 19u) - 9) / 8.f);
        for (uint32_t i = 0; i < jb.M; ++i) for (uint32_t j = 0; j < jb.N; ++j) put(*jb.C, jb.type, i, j, (float)((int)((i + 3u * j + t) % 23u) - 11) / 4.f);
        jb.dA = &de::CreateGPUMatrixRef(jb.type, jb.K, jb.M); jb.dB = &de::CreateGPUMatrixRef(jb.type, jb.N, jb.K);
        jb.dC = &de::CreateGPUMatrixRef(jb.type, jb.N, jb.M); jb.dD = &de::CreateGPUMatrixRef();
        CHECK(de::Memcpy(*jb.A, *jb.dA, O, O, de::Point2D(jb.K, jb.M), de::DECX_MEMCPY_H2D).error_type == 0);
        CHECK(de::Memcpy(*jb.B, *jb.dB, O, O, de::Point2D(jb.N, jb.K), de::DECX_MEMCPY_H2D).error_type == 0);
        CHECK(de::Memcpy(*jb.C, *jb.dC, O, O, de::Point2D(jb.N, jb.M), de::DECX_MEMCPY_H2D).error_type == 0);
        run_job(jb);
        CHECK(de::GetLastError()->error_type == 0);
        jb.want = fetch(jb);
        // the product is not all zeros, and job 0 is what its closed form says: small integers over 64, summed exactly
        bool any = false;
        for (char c : jb.want) any |= c != 0;
        CHECK(any);
    }
    {
        const ThreadJob& jb = jobs[0];
        double worst = 0;
        for (uint32_t i = 0; i < jb.M; i += 37) for (uint32_t j = 0; j < jb.N; j += 41) {
            double sum = 0;
            for (uint32_t k = 0; k < jb.K; ++k)
                sum += (double)((int)((i * 7u + k * 13u) % 17u) - 8) / 8.0 * ((double)((int)((k * 5u + j * 11u) % 19u) - 9) / 8.0);
            worst = std::fmax(worst, std::fabs(sum - (double)((const float*)jb.want.data())[(size_t)i * jb.N + j]));
        }
        if (worst != 0) std::cerr << "closed form: worst difference " << worst << "\n";
        CHECK(worst == 0);                                  // every partial sum is a multiple of 1/64 below 2^24 / 64
    }
    std::atomic<int> wrong(0), calls(0);
    std::vector<std::thread> threads;
    for (int t = 0; t < n_jobs; ++t)
        threads.emplace_back([&jobs, &wrong, &calls, t]() {
            ThreadJob& jb = jobs[t];
            for (int rep = 0; rep < 40; ++rep) {
                run_job(jb);
                if (fetch(jb) != jb.want) ++wrong;
                ++calls;
            }
        });
    for (std::thread& th : threads) th.join();
    CHECK(wrong.load() == 0);
    CHECK(calls.load() == 40 * n_jobs);
    std::cout << "threads: " << n_jobs << " threads x 40 products, " << wrong.load() << " wrong\n";
    return g_failures == 0 ? 0 : 1;
}

static int tensor_host_checks()
{
    // host tensors: width padded to 4 columns, depth to 16 bytes of elements; element (row, column, channel)
    de::Tensor& t = de::CreateTensorRef(de::_FP32_, 10, 6, 3);
    CHECK(t.Width() == 10 && t.Height() == 6 && t.Depth() == 3 && t.Type() == de::_FP32_);
    CHECK(t.ptr<float>(0, 1, 0) - t.ptr<float>(0, 0, 0) == 4);            // dpitch
    CHECK(t.ptr<float>(1, 0, 0) - t.ptr<float>(0, 0, 0) == 4 * 12);       // dpitch * wpitch
    bool zero = true;
    for (int i = 0; i < 6 * 12 * 4; ++i) zero &= (t.ptr<float>(0, 0, 0)[i] == 0.f);
    CHECK(zero);
    de::Tensor& th = de::CreateTensorRef(de::_FP16_, 3, 2, 9);
    CHECK(th.ptr<de::Half>(0, 1, 0) - th.ptr<de::Half>(0, 0, 0) == 16 && th.ptr<de::Half>(1, 0, 0) - th.ptr<de::Half>(0, 0, 0) == 64);
    de::Tensor& alias = de::CreateTensorRef();
    alias.SoftCopy(t);
    *t.ptr<float>(2, 3, 1) = 5.f;
    CHECK(alias.Width() == 10 && *alias.ptr<float>(2, 3, 1) == 5.f);
    // tensor arrays: tensors back to back, views by Extract_SoftCopy
    de::TensorArray& a = de::CreateTensorArrayRef(de::_FP32_, 3, 3, 5, 7);
    CHECK(a.Width() == 3 && a.Height() == 3 && a.Depth() == 5 && a.TensorNum() == 7);
    CHECK(a.ptr<float>(0, 0, 0, 1) - a.ptr<float>(0, 0, 0, 0) == 8 * 4 * 3);          // dpitch 8, wpitch 4, 3 rows
    *a.ptr<float>(1, 2, 4, 6) = 9.f;
    de::Tensor& view = de::CreateTensorRef();
    CHECK(a.Extract_SoftCopy(6, view).error_type == 0 && view.Depth() == 5 && *view.ptr<float>(1, 2, 4) == 9.f);
    CHECK(a.Extract_SoftCopy(7, view).error_type == decx::DECX_FAIL_INVALID_PARAM);
    a.release();
    CHECK(*view.ptr<float>(1, 2, 4) == 9.f);                              // the view keeps the storage alive
    CHECK(sizeof(de::Point3D) == 16 && de::_EXTEND_CONSTANT_ == 2);
    // without InitCuda
    de::GPU_Tensor& g = de::CreateGPUTensorRef();
    de::GPU_TensorArray& gk = de::CreateGPUTensorArrayRef();
    CHECK(de::Memcpy(t, g, de::Point3D(0, 0, 0), de::Point3D(0, 0, 0), de::Point3D(1, 1, 1), de::DECX_MEMCPY_H2D).error_type == decx::DECX_FAIL_CUDA_not_init);
    CHECK(de::nn::cuda::Conv2D(g, gk, g).error_type == decx::DECX_FAIL_CUDA_not_init);
    de::ResetLastError();
    return g_failures;
}

static int conv_files(const std::string& dir, uint32_t W, uint32_t H, uint32_t C, uint32_t OC, uint32_t KW, uint32_t KH,
                      int sx, int sy, int extend)
{
    de::InitCuda();
    de::ResetLastError();
    de::Tensor& img = de::CreateTensorRef(de::_FP32_, W, H, C);
    de::TensorArray& ker = de::CreateTensorArrayRef(de::_FP32_, KW, KH, C, OC);
    std::ifstream fi(dir + "/image.bin", std::ios::binary), fk(dir + "/kernels.bin", std::ios::binary);
    if (!fi || !fk) return 2;
    for (uint32_t y = 0; y < H; ++y) for (uint32_t x = 0; x < W; ++x) fi.read((char*)img.ptr<float>(y, x, 0), C * 4);
    for (uint32_t o = 0; o < OC; ++o) for (uint32_t y = 0; y < KH; ++y) for (uint32_t x = 0; x < KW; ++x) fk.read((char*)ker.ptr<float>(y, x, 0, o), C * 4);
    if (!fi || !fk) return 2;
    de::GPU_Tensor& dimg = de::CreateGPUTensorRef(de::_FP32_, W, H, C);
    de::GPU_TensorArray& dker = de::CreateGPUTensorArrayRef(de::_FP32_, KW, KH, C, OC);
    de::GPU_Tensor& dout = de::CreateGPUTensorRef();
    const de::Point3D O(0, 0, 0);
    if (de::Memcpy(img, dimg, O, O, de::Point3D(C, W, H), de::DECX_MEMCPY_H2D).error_type) return 3;
    de::Tensor& hv = de::CreateTensorRef();
    de::GPU_Tensor& dv = de::CreateGPUTensorRef();
    for (uint32_t o = 0; o < OC; ++o) {                                   // kernels go up one by one through views
        if (ker.Extract_SoftCopy(o, hv).error_type || dker.Extract_SoftCopy(o, dv).error_type) return 3;
        if (de::Memcpy(hv, dv, O, O, de::Point3D(C, KW, KH), de::DECX_MEMCPY_H2D).error_type) return 3;
    }
    de::DH r = de::nn::cuda::Conv2D(dimg, dker, dout, de::Point2D(sx, sy), (de::extend_label)extend);
    if (r.error_type) { std::cerr << r.error_string << "\n"; return 4; }
    r = de::nn::cuda::Conv2D(dimg, dker, dout, de::Point2D(sx, sy), (de::extend_label)extend);    // again: scratch reused
    if (r.error_type) return 4;
    const uint32_t OW = dout.Width(), OH = dout.Height();
    if (dout.Depth() != OC) return 5;
    de::Tensor& out = de::CreateTensorRef(de::_FP32_, OW, OH, OC);
    if (OW && OH && de::Memcpy(out, dout, O, O, de::Point3D(OC, OW, OH), de::DECX_MEMCPY_D2H).error_type) return 3;
    std::ofstream fo(dir + "/out.bin", std::ios::binary);
    for (uint32_t y = 0; y < OH; ++y) for (uint32_t x = 0; x < OW; ++x) fo.write((const char*)out.ptr<float>(y, x, 0), OC * 4);
    std::cout << "conv out " << OW << " " << OH << "\n";
    // error paths
    de::GPU_TensorArray& bad = de::CreateGPUTensorArrayRef(de::_FP32_, KW, KH, C + 1, OC);
    if (de::nn::cuda::Conv2D(dimg, bad, dout, de::Point2D(sx, sy), (de::extend_label)extend).error_type != decx::DECX_FAIL_DimsNotMatching) return 6;
    if (de::nn::cuda::Conv2D(dimg, dker, dout, de::Point2D(sx, sy), de::_EXTEND_REFLECT_).error_type != decx::DECX_FAIL_ErrorFlag) return 6;
    if (de::nn::cuda::Conv2D(dimg, dker, dout, de::Point2D(0, sy), (de::extend_label)extend).error_type != decx::DECX_FAIL_INVALID_PARAM) return 6;
    de::GPU_Tensor& half_img = de::CreateGPUTensorRef(de::_FP16_, W, H, C);
    if (de::nn::cuda::Conv2D(half_img, dker, dout).error_type != decx::DECX_FAIL_TYPE_MOT_MATCH) return 6;
    if (dout.Width() != OW || dout.Height() != OH) return 6;             // failed calls left dst alone
    return fo ? 0 : 2;
}

template <typename T> static int hostgemm_files(const std::string& dir, de::_DATA_TYPES_FLAGS_ ty, uint32_t M, uint32_t N,
                                                uint32_t K, int with_c, bool pinned, int repeats)
{
    de::InitCuda();
    de::ResetLastError();
    de::Matrix& A = de::CreateMatrixRef(ty, K, M);
    de::Matrix& B = de::CreateMatrixRef(ty, N, K);
    de::Matrix& C = de::CreateMatrixRef(ty, N, M);
    // dst: C itself, an empty matrix the call has to create, or (pinned) one made page-locked beforehand
    de::Matrix& D = with_c == 2 ? C : (pinned ? de::CreateMatrixRef(ty, N, M) : de::CreateMatrixRef());
    if (!read_into<T>(A, dir + "/A.bin") || !read_into<T>(B, dir + "/B.bin")) return 2;
    if (pinned) {
        if (de::cuda::PinMemory(A).error_type || de::cuda::PinMemory(B).error_type || de::cuda::PinMemory(C).error_type) return 5;
        if (with_c != 2 && de::cuda::PinMemory(D).error_type) return 5;
    }
    for (int r = 0; r < repeats; ++r) {
        if (with_c && !read_into<T>(C, dir + "/C.bin")) return 2;           // C is overwritten when it is dst
        const auto t0 = std::chrono::steady_clock::now();
        if (with_c) de::blas::cuda::GEMM(A, B, C, D); else de::blas::cuda::GEMM(A, B, D);
        const double ms = std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - t0).count();
        std::cout << "hostgemm repeat " << r << ": " << ms << " ms\n";
        if (de::GetLastError()->error_type != 0) { std::cerr << de::GetLastError()->error_string << "\n"; return 3; }
    }
    if (D.Width() != N || D.Height() != M) return 4;
    std::ofstream out(dir + "/D.bin", std::ios::binary);
    for (uint32_t i = 0; i < M; ++i) out.write((const char*)D.ptr<T>(i, 0), (std::streamsize)N * sizeof(T));
    return out ? 0 : 2;
}

template <typename T> static T from_float(float v) { return (T)v; }
template <> de::Half from_float<de::Half>(float v) { return de::Float2Half(v); }

// Wall time of de::blas::cuda::GEMM(GPU_Matrix x 3) as a caller sees it (the call returns when dst is complete).
template <typename T> static int gemm_wall_time(de::_DATA_TYPES_FLAGS_ ty, uint32_t M, uint32_t N, uint32_t K, int repeats)
{
    de::InitCuda();
    de::ResetLastError();
    de::Matrix& A = de::CreateMatrixRef(ty, K, M);
    de::Matrix& B = de::CreateMatrixRef(ty, N, K);
    uint64_t state = 0x9E3779B97F4A7C15ull;                               // any non-constant data will do
    auto next = [&]() { state = state * 6364136223846793005ull + 1442695040888963407ull; return (float)((state >> 40) & 0xFFFF) / 32768.f - 1.f; };
    for (uint32_t i = 0; i < M; ++i) for (uint32_t k = 0; k < K; ++k) *A.ptr<T>(i, k) = from_float<T>(next());
    for (uint32_t k = 0; k < K; ++k) for (uint32_t j = 0; j < N; ++j) *B.ptr<T>(k, j) = from_float<T>(next());
    de::GPU_Matrix& dA = de::CreateGPUMatrixRef(ty, K, M);
    de::GPU_Matrix& dB = de::CreateGPUMatrixRef(ty, N, K);
    de::GPU_Matrix& dD = de::CreateGPUMatrixRef();
    auto now = [] { return std::chrono::steady_clock::now(); };
    auto since = [&](std::chrono::steady_clock::time_point t0) { return std::chrono::duration<double, std::milli>(now() - t0).count(); };
    if (de::Memcpy(A, dA, de::Point2D(0, 0), de::Point2D(0, 0), de::Point2D(K, M), de::DECX_MEMCPY_H2D).error_type) return 3;
    auto t_up = now();
    if (de::Memcpy(B, dB, de::Point2D(0, 0), de::Point2D(0, 0), de::Point2D(N, K), de::DECX_MEMCPY_H2D).error_type) return 3;
    const double up_ms = since(t_up);
    std::vector<double> ms;
    const auto begin = std::chrono::steady_clock::now();
    for (int r = 0; r < repeats + 3 || std::chrono::duration<double>(std::chrono::steady_clock::now() - begin).count() < 0.3; ++r) {
        const auto t0 = std::chrono::steady_clock::now();
        de::blas::cuda::GEMM(dA, dB, dD);
        ms.push_back(std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - t0).count());
        if (de::GetLastError()->error_type != 0) { std::cerr << de::GetLastError()->error_string << "\n"; return 3; }
    }
    std::vector<double> last(ms.end() - repeats, ms.end());               // what came before is warm-up
    std::sort(last.begin(), last.end());
    std::cout << "gemmtime median_ms " << last[last.size() / 2] << " min_ms " << last.front() << " calls " << last.size() << "\n";
    de::Matrix& D = de::CreateMatrixRef(ty, N, M);
    if (de::Memcpy(D, dD, de::Point2D(0, 0), de::Point2D(0, 0), de::Point2D(N, M), de::DECX_MEMCPY_D2H).error_type) return 3;   // touches D's pages
    auto t_down = now();
    if (de::Memcpy(D, dD, de::Point2D(0, 0), de::Point2D(0, 0), de::Point2D(N, M), de::DECX_MEMCPY_D2H).error_type) return 3;
    const double down_ms = since(t_down);
    std::cout << "memcpytime pageable h2d_ms " << up_ms << " (" << (double)K * N * sizeof(T) / up_ms / 1e6 << " GB/s) d2h_ms " << down_ms
              << " (" << (double)M * N * sizeof(T) / down_ms / 1e6 << " GB/s)\n";
    return (dD.Width() == N && dD.Height() == M) ? 0 : 4;
}

// Wall time of the host-matrix form de::blas::cuda::GEMM(Matrix x 3): staging in, multiply, staging out.
template <typename T> static int hostgemm_wall_time(de::_DATA_TYPES_FLAGS_ ty, uint32_t M, uint32_t N, uint32_t K, int repeats, bool pinned)
{
    de::InitCuda();
    de::ResetLastError();
    de::Matrix& A = de::CreateMatrixRef(ty, K, M);
    de::Matrix& B = de::CreateMatrixRef(ty, N, K);
    de::Matrix& D = de::CreateMatrixRef(ty, N, M);
    uint64_t state = 0x9E3779B97F4A7C15ull;
    auto next = [&]() { state = state * 6364136223846793005ull + 1442695040888963407ull; return (float)((state >> 40) & 0xFFFF) / 32768.f - 1.f; };
    for (uint32_t i = 0; i < M; ++i) for (uint32_t k = 0; k < K; ++k) *A.ptr<T>(i, k) = from_float<T>(next());
    for (uint32_t k = 0; k < K; ++k) for (uint32_t j = 0; j < N; ++j) *B.ptr<T>(k, j) = from_float<T>(next());
    if (pinned && (de::cuda::PinMemory(A).error_type || de::cuda::PinMemory(B).error_type || de::cuda::PinMemory(D).error_type)) return 5;
    std::vector<double> ms;
    for (int r = 0; r < repeats + 1; ++r) {
        const auto t0 = std::chrono::steady_clock::now();
        de::blas::cuda::GEMM(A, B, D);
        ms.push_back(std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - t0).count());
        if (de::GetLastError()->error_type != 0) { std::cerr << de::GetLastError()->error_string << "\n"; return 3; }
    }
    std::vector<double> last(ms.begin() + 1, ms.end());                   // the first call creates streams and buffers
    std::sort(last.begin(), last.end());
    std::cout << "hostgemmtime " << (pinned ? "pinned" : "pageable") << " median_ms " << last[last.size() / 2] << " min_ms " << last.front()
              << " first_ms " << ms.front() << "\n";
    return 0;
}

int main(int argc, char** argv)
{
    const std::string mode = argc > 1 ? argv[1] : "host";
    int rc;
    if (mode == "host") rc = host_checks();
    else if (mode == "gpu") rc = gpu_checks();
    else if (mode == "hostgemm" && argc == 10) {
        const bool f16 = std::string(argv[3]) == "f16";
        const uint32_t M = std::atoi(argv[4]), N = std::atoi(argv[5]), K = std::atoi(argv[6]);
        const int with_c = std::atoi(argv[7]), repeats = std::atoi(argv[9]);
        const bool pinned = std::atoi(argv[8]) != 0;
        rc = f16 ? hostgemm_files<de::Half>(argv[2], de::_FP16_, M, N, K, with_c, pinned, repeats)
                 : std::string(argv[3]) == "f64" ? hostgemm_files<double>(argv[2], de::_FP64_, M, N, K, with_c, pinned, repeats)
                 : hostgemm_files<float>(argv[2], de::_FP32_, M, N, K, with_c, pinned, repeats);
    }
    else if (mode == "gemmtime" && argc == 7) {
        const uint32_t M = std::atoi(argv[3]), N = std::atoi(argv[4]), K = std::atoi(argv[5]);
        const int repeats = std::max(1, std::atoi(argv[6]));
        rc = std::string(argv[2]) == "f16" ? gemm_wall_time<de::Half>(de::_FP16_, M, N, K, repeats)
                                           : gemm_wall_time<float>(de::_FP32_, M, N, K, repeats);
    }
    else if (mode == "hostgemmtime" && argc == 8) {
        const uint32_t M = std::atoi(argv[3]), N = std::atoi(argv[4]), K = std::atoi(argv[5]);
        const int repeats = std::max(1, std::atoi(argv[6]));
        const bool pinned = std::atoi(argv[7]) != 0;
        rc = std::string(argv[2]) == "f16" ? hostgemm_wall_time<de::Half>(de::_FP16_, M, N, K, repeats, pinned)
                                           : hostgemm_wall_time<float>(de::_FP32_, M, N, K, repeats, pinned);
    }
    else if (mode == "threads") rc = threads_checks();
    else if (mode == "tensor_host") rc = tensor_host_checks();
    else if (mode == "conv" && argc == 12)
        rc = conv_files(argv[2], std::atoi(argv[3]), std::atoi(argv[4]), std::atoi(argv[5]), std::atoi(argv[6]), std::atoi(argv[7]),
                        std::atoi(argv[8]), std::atoi(argv[9]), std::atoi(argv[10]), std::atoi(argv[11]));
    else if (mode == "vector_host") rc = vector_host_checks();
    else if (mode == "vector_gpu") rc = vector_gpu_checks();
    else if (mode == "vmm" && argc == 8) {
        const bool f16 = std::string(argv[3]) == "f16", mv = std::string(argv[4]) == "mv";
        const uint32_t W = std::atoi(argv[5]), H = std::atoi(argv[6]), level = std::atoi(argv[7]);
        rc = f16 ? vmm_files<de::Half>(argv[2], de::_FP16_, mv, W, H, level)
                 : vmm_files<float>(argv[2], de::_FP32_, mv, W, H, level);
    }
    else if (mode == "gemm" && argc == 10) {
        const bool f16 = std::string(argv[3]) == "f16";
        const uint32_t M = std::atoi(argv[4]), N = std::atoi(argv[5]), K = std::atoi(argv[6]);
        const bool with_c = std::atoi(argv[7]) != 0;
        const float alpha = (float)std::atof(argv[8]), beta = (float)std::atof(argv[9]);
        rc = f16 ? gemm_files<de::Half>(argv[2], de::_FP16_, M, N, K, with_c, alpha, beta)
                 : std::string(argv[3]) == "f64" ? gemm_files<double>(argv[2], de::_FP64_, M, N, K, with_c, alpha, beta)
                 : gemm_files<float>(argv[2], de::_FP32_, M, N, K, with_c, alpha, beta);
    } else {
        std::cerr << "usage: de_api_test host | gpu | threads | vector_host | vector_gpu | gemm <dir> <f32|f16> M N K withC alpha beta"
                     " | vmm <dir> <f32|f16> <mv|vm> W H level | gemmtime <f32|f16> M N K repeats | hostgemmtime <f32|f16> M N K repeats pinned\n";
        return 64;
    }
    std::cout << (rc == 0 ? "de_api_test: all checks passed" : "de_api_test: FAILED") << " (" << mode << ")\n";
    return rc;
}
