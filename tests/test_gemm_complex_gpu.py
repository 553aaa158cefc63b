"""Parity of the complex GEMM (through the C ABI) against the CPU oracle.
Bar: max|d| / (max|ref| * sqrt(2 K)) <= 1e-5 (complex64), <= 1e-14 (complex128); Gaussian integers exact."""
import numpy as np
import pytest

from decx_amd import synth

pytestmark = pytest.mark.gpu
TOL = {np.dtype(np.complex64): 1e-5, np.dtype(np.complex128): 1e-14}


@pytest.fixture(scope="module")
def hip():
    from decx_amd import hip as h
    h.init()
    return h


def cplx(rows, cols, seed, dtype):
    if dtype == np.complex64:
        return synth.uniform_f32(rows, 2 * cols, seed).view(np.complex64)
    return synth.uniform_f64(rows, 2 * cols, seed).view(np.complex128)


def rel_err(got, ref, K):
    return float(np.max(np.abs(got - ref))) / (max(float(np.max(np.abs(ref))), 1e-300) * np.sqrt(2 * max(K, 1)))


def run(hip, A, B, C=None, alpha=1.0, beta=1.0, alias=False):
    dt = A.dtype
    M, K = A.shape
    N = B.shape[1]
    per = 128 // dt.itemsize                                    # the device pitch rule
    pitch = lambda v: (v + per - 1) // per * per
    dA = hip.DeviceMatrix(M, K, dt, pitch(K), A, pad_value=np.nan)
    dB = hip.DeviceMatrix(K, N, dt, pitch(N), B, pad_value=np.nan)
    dD = hip.DeviceMatrix(M, N, dt, pitch(N))
    if alias:
        dD.upload_raw(np.pad(C, ((0, 0), (0, pitch(N) - N)), constant_values=-777))
        dC = dD
    else:
        dD.upload_raw(np.full((M, pitch(N)), -777, dt))
        dC = hip.DeviceMatrix(M, N, dt, pitch(N), C, pad_value=np.nan) if C is not None else None
    hip.gemm(dA, dB, dD, dC, alpha, beta)
    hip.sync()
    raw = dD.download_raw()
    assert np.all(raw[:, N:] == -777), "padding columns of D were written"
    out = raw[:, :N].copy()
    assert not np.isnan(out).any()
    return out


SHAPES = [(1, 1, 1), (1, 7, 3), (7, 1, 3), (31, 33, 17), (65, 63, 15), (129, 257, 100), (300, 20, 40), (20, 300, 1025), (512, 384, 96)]


@pytest.mark.parametrize("dt", [np.complex64, np.complex128])
@pytest.mark.parametrize("M,N,K", SHAPES)
def test_against_oracle(hip, oracle, dt, M, N, K):
    A = cplx(M, K, 941, dt); B = cplx(K, N, 942, dt); C = cplx(M, N, 943, dt)
    tol = TOL[np.dtype(dt)]
    assert rel_err(run(hip, A, B), oracle.gemm_complex(A, B), K) <= tol
    # alpha = beta = 1: the oracle's chain seeded with C differs from D = C + A.B by rounding order only
    assert rel_err(run(hip, A, B, C), oracle.gemm_complex(A, B, C), K) <= tol
    alpha, beta = 0.75 - 0.5j, -1.25 + 2j
    hi = np.clongdouble
    want = alpha * (A.astype(hi) @ B.astype(hi)) + beta * C.astype(hi)
    assert rel_err(run(hip, A, B, C, alpha, beta), want, K) <= tol
    assert rel_err(run(hip, A, B, C, alpha, beta, alias=True), want, K) <= tol        # C is D


@pytest.mark.parametrize("dt", [np.complex64, np.complex128])
def test_gaussian_integers_exact(hip, dt):
    rng = np.random.default_rng(2)
    A = (rng.integers(-9, 10, (130, 96)) + 1j * rng.integers(-9, 10, (130, 96))).astype(dt)
    B = (rng.integers(-9, 10, (96, 140)) + 1j * rng.integers(-9, 10, (96, 140))).astype(dt)
    want = (A.astype(np.complex128) @ B.astype(np.complex128)).astype(dt)
    assert np.array_equal(run(hip, A, B), want)
    assert np.array_equal(run(hip, A, B, None, 2j), (2j * want).astype(dt))            # alpha = 2i: exact too
    eye = np.eye(96, dtype=dt)
    assert np.array_equal(run(hip, A, eye), A)


def test_1024_cubed_complex64_sampled(hip, oracle):
    n = 1024
    A = cplx(n, n, 951, np.complex64); B = cplx(n, n, 952, np.complex64)
    got = run(hip, A, B)
    rows = [0, 511, 1023]
    want = A[rows].astype(np.complex128) @ B.astype(np.complex128)
    assert rel_err(got[rows], want, n) <= 1e-5
    colsum = A.astype(np.complex128).sum(axis=0) @ B.astype(np.complex128)
    assert np.max(np.abs(got.astype(np.complex128).sum(axis=0) - colsum)) / np.max(np.abs(colsum)) < 1e-5


def test_workspace_contract(hip):
    L = hip.lib()
    assert L.decx_hip_gemm_complex_workspace(4, 100, 50) == 2 * 50 * 208 * 4
    assert L.decx_hip_gemm_complex_workspace(8, 100, 50) == 2 * 50 * 208 * 8
    assert L.decx_hip_gemm_complex_workspace(2, 100, 50) == 0
    d = hip.DeviceMatrix(4, 4, np.complex64, data=np.ones((4, 4), np.complex64))
    ws = hip.DeviceMatrix(1, 64, np.complex64)
    args = [d.ptr, d.ptr, None, d.ptr, 4, 4, 4, 4, 4, 0, 4, 1.0, 0.0, 1.0, 0.0]
    assert L.decx_hip_gemm_c32(*args, ws.ptr, 2 * 4 * 16 * 4, None) == 0
    assert L.decx_hip_gemm_c32(*args, ws.ptr, 2 * 4 * 16 * 4 - 1, None) == -1         # workspace too small
    assert L.decx_hip_gemm_c32(*args, None, 1 << 20, None) == -1
    hip.sync()


@pytest.mark.parametrize("dtype", [np.complex64, np.complex128])
def test_k_zero_needs_no_workspace(hip, dtype):
    """K == 0: D = beta * C (or zero); the workspace query returns 0 and a null workspace is accepted."""
    L = hip.lib()
    M, N = 37, 21
    rng = np.random.default_rng(5)
    C = (rng.standard_normal((M, N)) + 1j * rng.standard_normal((M, N))).astype(dtype)
    rb = 4 if dtype == np.complex64 else 8
    assert L.decx_hip_gemm_complex_workspace(rb, N, 0) == 0
    dA = hip.DeviceMatrix(M, 1, dtype, 4); dB = hip.DeviceMatrix(1, N, dtype, 24)
    dC = hip.DeviceMatrix(M, N, dtype, 24, C); dD = hip.DeviceMatrix(M, N, dtype, 24)
    fn = L.decx_hip_gemm_c32 if rb == 4 else L.decx_hip_gemm_c64
    hip.check(fn(dA.ptr, dB.ptr, dC.ptr, dD.ptr, M, N, 0, 4, 24, 24, 24, 1.0, 0.0, 0.5, -2.0, None, 0, None), "complex K = 0")
    hip.sync()
    want = (C.astype(np.complex128) * (0.5 - 2.0j))
    assert np.max(np.abs(dD.download() - want)) <= 1e-5 * np.max(np.abs(want))
    hip.check(fn(dA.ptr, dB.ptr, None, dD.ptr, M, N, 0, 4, 24, 0, 24, 1.0, 0.0, 1.0, 0.0, None, 0, None), "complex K = 0, no C")
    hip.sync()
    assert np.all(dD.download() == 0)
