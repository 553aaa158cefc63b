"""The public C++ API (include/DECX.h) driven through tests/cpp/de_api_test, a program written
the way the original library's sample uses it."""
import os
import subprocess
import tempfile

import numpy as np
import pytest

from decx_amd import synth

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
EXE = os.path.join(ROOT, "tests", "cpp", "de_api_test")


def run_exe(*args, timeout=300):
    assert os.path.exists(EXE), "tests/cpp/de_api_test missing: run `python -m decx_amd.build`"
    done = subprocess.run([EXE] + [str(a) for a in args], stdout=subprocess.PIPE, stderr=subprocess.STDOUT,
                          text=True, timeout=timeout)
    return done.returncode, done.stdout


def test_host_side_objects_and_error_codes():
    rc, out = run_exe("host")
    assert rc == 0, out


def test_host_side_vectors_and_error_codes():
    rc, out = run_exe("vector_host")
    assert rc == 0, out


def test_host_side_tensors_and_views():
    rc, out = run_exe("tensor_host")
    assert rc == 0, out


def test_host_library_exports_the_public_entry_points():
    lib = os.path.join(ROOT, "decx_amd", "lib", "libDECX_BLAS_HIP.so")
    syms = subprocess.run(["nm", "-D", "-C", "--defined-only", lib], stdout=subprocess.PIPE, text=True).stdout
    for needle in ["de::blas::cuda::GEMM(de::GPU_Matrix&, de::GPU_Matrix&, de::GPU_Matrix&)",
                   "de::blas::cuda::GEMM(de::GPU_Matrix&, de::GPU_Matrix&, de::GPU_Matrix&, de::GPU_Matrix&, de::Number, de::Number)",
                   "de::blas::cuda::GEMM(de::Matrix&, de::Matrix&, de::Matrix&)",
                   "de::CreateGPUMatrixRef(de::_DATA_TYPES_FLAGS_, unsigned int, unsigned int, de::_DATA_FORMATS_)",
                   "de::CreateMatrixRef(de::_DATA_TYPES_FLAGS_, unsigned int, unsigned int, de::_DATA_FORMATS_)",
                   "de::Memcpy(de::Matrix&, de::GPU_Matrix&, de::Point2D, de::Point2D, de::Point2D, int)",
                   "de::GetLastError()", "de::InitCuda()", "de::Float2Half(float const&)",
                   "de::cuda::PinMemory(de::Matrix&)", "de::cuda::PinMemory(de::Vector&)",
                   "de::blas::cuda::GEMM(de::Vector&, de::Matrix&, de::Vector&, unsigned int)",
                   "de::blas::cuda::GEMM(de::Matrix&, de::Vector&, de::Vector&, unsigned int)",
                   "de::CreateVectorRef(de::_DATA_TYPES_FLAGS_, unsigned long)",
                   "de::nn::cuda::Conv2D(de::GPU_Tensor&, de::GPU_TensorArray&, de::GPU_Tensor&, de::Point2D, de::extend_label)",
                   "de::CreateGPUTensorArrayRef(de::_DATA_TYPES_FLAGS_, unsigned int, unsigned int, unsigned int, unsigned int)",
                   "de::Memcpy(de::Tensor&, de::GPU_Tensor&, de::Point3D, de::Point3D, de::Point3D, int)",
                   "de::CreateGPUVectorRef(de::_DATA_TYPES_FLAGS_, unsigned long)",
                   "de::Memcpy(de::Vector&, de::GPU_Vector&, unsigned long, unsigned long, unsigned long, int)"]:
        assert needle in syms, needle


@pytest.mark.gpu
def test_gpu_side_closed_forms_and_error_paths():
    rc, out = run_exe("gpu")
    assert rc == 0, out


@pytest.mark.gpu
def test_several_host_threads_each_get_their_own_product():
    """Six host threads in GEMM and Memcpy at once, each on its own matrices (a product split along K, a ragged one with
    C, fp16, fp64, the two vector corners): the module serialises them, every result bit-equal to the same call alone."""
    rc, out = run_exe("threads")
    assert rc == 0, out
    assert "0 wrong" in out


@pytest.mark.gpu
@pytest.mark.parametrize("dt,M,N,K,with_c,alpha,beta", [
    ("f32", 1000, 1500, 777, False, 1.0, 1.0),
    ("f32", 1000, 1500, 777, True, 1.0, 1.0),
    ("f32", 300, 1, 500, True, -0.5, 2.0),          # N == 1: the row-dot path behind the same entry point
    ("f16", 257, 130, 515, False, 1.0, 1.0),
    ("f16", 257, 130, 515, True, 1.5, -0.5),
    ("f64", 1000, 700, 333, False, 1.0, 1.0),
    ("f64", 1000, 700, 333, True, -0.5, 2.0),
    # the vector corners with the module's workspace: column operand copied into a dense vector, K of a row
    # operand split over workgroups, fp64 on the vector kernels
    ("f32", 1100, 1, 8200, True, 1.5, -0.5),
    ("f16", 2100, 1, 4100, False, 1.0, 1.0),
    ("f32", 1, 70, 20000, True, 1.5, -0.5),
    ("f16", 1, 513, 33000, False, 1.0, 1.0),
    ("f64", 2100, 1, 4100, True, -0.5, 2.0),
    ("f64", 1, 100, 33000, False, 1.0, 1.0),
])
def test_gemm_through_the_objects_matches_oracle(oracle, dt, M, N, K, with_c, alpha, beta):
    if dt == "f32":
        A = synth.uniform_f32(M, K, 201); B = synth.uniform_f32(K, N, 202); C = synth.uniform_f32(M, N, 203)
    elif dt == "f64":
        A = synth.uniform_f64(M, K, 201); B = synth.uniform_f64(K, N, 202); C = synth.uniform_f64(M, N, 203)
    else:
        A = synth.normal_half(M, K, 201); B = synth.normal_half(K, N, 202); C = synth.normal_half(M, N, 203)
    with tempfile.TemporaryDirectory() as tmp:
        A.tofile(os.path.join(tmp, "A.bin")); B.tofile(os.path.join(tmp, "B.bin")); C.tofile(os.path.join(tmp, "C.bin"))
        rc, out = run_exe("gemm", tmp, dt, M, N, K, int(with_c), alpha, beta)
        assert rc == 0, out
        D = np.fromfile(os.path.join(tmp, "D.bin"), A.dtype).reshape(M, N)
    if dt == "f32":
        ref = oracle.gemm_f32(A, B, C, alpha, beta) if with_c else oracle.gemm_f32(A, B)
        tol = 1e-5
    elif dt == "f64":
        ref = oracle.gemm_f64(A, B, C, alpha, beta) if with_c else oracle.gemm_f64(A, B)
        tol = 1e-14
    else:
        ref = oracle.gemm_f16(A, B, C if with_c else None, alpha, beta)
        tol = 2e-3
    ref = ref.astype(np.float64)
    err = np.max(np.abs(D.astype(np.float64) - ref)) / (np.max(np.abs(ref)) * np.sqrt(K))
    assert err <= tol


@pytest.mark.gpu
def test_gpu_side_vectors_closed_forms_and_error_paths():
    rc, out = run_exe("vector_gpu")
    assert rc == 0, out


@pytest.mark.gpu
@pytest.mark.parametrize("dt,form,W,H,level", [
    ("f32", "mv", 1030, 700, 0), ("f32", "vm", 1030, 700, 0),
    ("f32", "mv", 8200, 33, 0), ("f32", "vm", 33, 8200, 0),
    ("f16", "mv", 1030, 700, 0), ("f16", "vm", 1030, 700, 0),      # level 1: fp32 result
    ("f16", "mv", 1030, 700, 1), ("f16", "vm", 1030, 700, 2),      # levels 2, 3: fp16 result
])
def test_vector_forms_through_the_objects_match_oracle(oracle, dt, form, W, H, level):
    """de::blas::cuda::GEMM(Matrix, Vector, Vector) / (Vector, Matrix, Vector) on host objects against the
    oracle's GEMM with one column / one row (fp16 inputs widened exactly to fp32)."""
    n_in = W if form == "mv" else H
    if dt == "f32":
        M = synth.uniform_f32(H, W, 301); V = synth.uniform_f32(1, n_in, 302).reshape(-1)
    else:
        M = synth.normal_half(H, W, 301); V = synth.normal_half(1, n_in, 302).reshape(-1)
    out_f32 = dt == "f32" or level == 0
    with tempfile.TemporaryDirectory() as tmp:
        M.tofile(os.path.join(tmp, "M.bin")); V.tofile(os.path.join(tmp, "V.bin"))
        rc, out = run_exe("vmm", tmp, dt, form, W, H, level)
        assert rc == 0, out
        Y = np.fromfile(os.path.join(tmp, "Y.bin"), np.float32 if out_f32 else np.float16)
    Mf, Vf = M.astype(np.float32), V.astype(np.float32)
    ref = (oracle.gemm_f32(Mf, Vf.reshape(-1, 1)) if form == "mv" else oracle.gemm_f32(Vf.reshape(1, -1), Mf)).reshape(-1)
    K = n_in
    assert Y.shape == ref.shape
    if not out_f32:
        ref = ref.astype(np.float16)
    ref = ref.astype(np.float64)
    err = np.max(np.abs(Y.astype(np.float64) - ref)) / (np.max(np.abs(ref)) * np.sqrt(K))
    assert err <= (1e-5 if out_f32 else 2e-3)


@pytest.mark.gpu
@pytest.mark.parametrize("dt,M,N,K,with_c,pinned", [
    ("f32", 1000, 1500, 777, 0, 0),        # 4 row panels, the last one ragged
    ("f32", 1000, 1500, 777, 1, 1),
    ("f32", 1000, 1500, 777, 2, 1),        # C is dst
    ("f32", 5000, 300, 260, 2, 0),         # 10 panels of 512 rows, the last one ragged
    ("f32", 100, 70, 33, 1, 0),            # a single panel
    ("f32", 4100, 2300, 4700, 1, 0),       # pageable operands larger than the ring of bounce buffers (B: 43 MB)
    ("f16", 1300, 520, 515, 0, 1),
    ("f16", 1300, 520, 515, 2, 0),
    ("f64", 700, 300, 129, 1, 1),
])
def test_host_matrix_forms_match_oracle(oracle, dt, M, N, K, with_c, pinned):
    """de::blas::cuda::GEMM(Matrix, Matrix[, Matrix], Matrix): operands staged in row panels on three streams;
    pageable and page-locked host storage, C as a separate matrix and as dst."""
    if dt == "f32":
        A = synth.uniform_f32(M, K, 401); B = synth.uniform_f32(K, N, 402); C = synth.uniform_f32(M, N, 403)
    elif dt == "f64":
        A = synth.uniform_f64(M, K, 401); B = synth.uniform_f64(K, N, 402); C = synth.uniform_f64(M, N, 403)
    else:
        A = synth.normal_half(M, K, 401); B = synth.normal_half(K, N, 402); C = synth.normal_half(M, N, 403)
    with tempfile.TemporaryDirectory() as tmp:
        A.tofile(os.path.join(tmp, "A.bin")); B.tofile(os.path.join(tmp, "B.bin")); C.tofile(os.path.join(tmp, "C.bin"))
        rc, out = run_exe("hostgemm", tmp, dt, M, N, K, with_c, pinned, 2)
        assert rc == 0, out
        D = np.fromfile(os.path.join(tmp, "D.bin"), A.dtype).reshape(M, N)
    if dt == "f32":
        ref = oracle.gemm_f32(A, B, C, 1.0, 1.0) if with_c else oracle.gemm_f32(A, B)
        tol = 1e-5
    elif dt == "f64":
        ref = oracle.gemm_f64(A, B, C, 1.0, 1.0) if with_c else oracle.gemm_f64(A, B)
        tol = 1e-14
    else:
        ref = oracle.gemm_f16(A, B, C if with_c else None, 1.0, 1.0)
        tol = 2e-3
    ref = ref.astype(np.float64)
    err = np.max(np.abs(D.astype(np.float64) - ref)) / (np.max(np.abs(ref)) * np.sqrt(K))
    assert err <= tol


@pytest.mark.gpu
@pytest.mark.parametrize("W,H,C,OC,KW,KH,sx,sy,extend", [
    (20, 17, 5, 3, 4, 2, 2, 1, 0), (20, 17, 5, 3, 4, 2, 2, 1, 2),
    (57, 43, 13, 70, 3, 3, 1, 1, 0), (57, 43, 13, 70, 3, 3, 1, 1, 2),
    (64, 48, 16, 64, 5, 5, 2, 2, 2), (9, 9, 4, 8, 9, 9, 1, 1, 0),
])
def test_conv2d_through_the_objects_matches_oracle(oracle, W, H, C, OC, KW, KH, sx, sy, extend):
    """de::nn::cuda::Conv2D on GPU_Tensor / GPU_TensorArray objects filled through de::Memcpy and views."""
    image = synth.uniform_f32(H, W * C, 601).reshape(H, W, C)
    kernels = synth.uniform_f32(OC, KH * KW * C, 602).reshape(OC, KH, KW, C)
    ref = oracle.conv2d_f32(image, kernels, sx, sy, extend == 2)
    with tempfile.TemporaryDirectory() as tmp:
        image.tofile(os.path.join(tmp, "image.bin")); kernels.tofile(os.path.join(tmp, "kernels.bin"))
        rc, out = run_exe("conv", tmp, W, H, C, OC, KW, KH, sx, sy, extend)
        assert rc == 0, out
        got = np.fromfile(os.path.join(tmp, "out.bin"), np.float32).reshape(ref.shape)
    assert ("conv out %d %d" % (ref.shape[1], ref.shape[0])) in out
    r = ref.astype(np.float64)
    assert np.max(np.abs(got - r)) / (np.max(np.abs(r)) * np.sqrt(KW * KH * C)) <= 1e-5
