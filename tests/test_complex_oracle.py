"""Pins the complex GEMM oracle (oracle.binding.gemm_complex: the real fma chain on the real expansion of B)."""
import glob
import os
import zlib

import numpy as np
import pytest

from decx_amd import synth

GOLD = os.path.join(os.path.dirname(__file__), "golden")


def cplx(rows, cols, seed, dtype=np.complex64):
    if dtype == np.complex64:
        return synth.uniform_f32(rows, 2 * cols, seed).view(np.complex64)
    return synth.uniform_f64(rows, 2 * cols, seed).view(np.complex128)


def test_gaussian_integers_are_exact(oracle):
    """Small Gaussian integers: every partial sum is an exactly representable integer, so a wrong sign of the
    imaginary cross terms, swapped re / im or a conjugated operand gives a different integer matrix."""
    rng = np.random.default_rng(1)
    for dt in (np.complex64, np.complex128):
        A = (rng.integers(-9, 10, (13, 21)) + 1j * rng.integers(-9, 10, (13, 21))).astype(dt)
        B = (rng.integers(-9, 10, (21, 8)) + 1j * rng.integers(-9, 10, (21, 8))).astype(dt)
        C = (rng.integers(-9, 10, (13, 8)) + 1j * rng.integers(-9, 10, (13, 8))).astype(dt)
        want = A.astype(np.complex128) @ B.astype(np.complex128)
        assert np.array_equal(oracle.gemm_complex(A, B), want.astype(dt))
        assert np.array_equal(oracle.gemm_complex(A, B, C), (want + C).astype(dt))
    X = oracle.complex_embed(np.array([[1 + 2j]], np.complex64))
    assert np.array_equal(X, np.array([[1, 2], [-2, 1]], np.float32))


@pytest.mark.parametrize("dt,tol", [(np.complex64, 2e-7), (np.complex128, 4e-16)])
def test_against_numpy_in_double_the_precision(oracle, dt, tol):
    M, N, K = 37, 53, 129
    A = cplx(M, K, 11, dt); B = cplx(K, N, 12, dt)
    want = A.astype(np.clongdouble) @ B.astype(np.clongdouble)
    got = oracle.gemm_complex(A, B)
    assert np.max(np.abs(got - want)) / (np.max(np.abs(want)) * np.sqrt(2 * K)) < tol


@pytest.mark.parametrize("path", sorted(glob.glob(os.path.join(GOLD, "ref_c32_*.npz"))))
def test_reference_outputs_within_rounding(oracle, path):
    """Outputs of the reference's complex single-precision CPU GEMM.  Its blocked complex arithmetic sums in
    another order than the chain, so the comparison carries a tolerance: a few ulp times sqrt(2 K)."""
    g = np.load(path)
    M, N, K = int(g["M"]), int(g["N"]), int(g["K"])
    A = cplx(M, K, int(g["seed_a"])); B = cplx(K, N, int(g["seed_b"]))
    assert zlib.crc32(g["D"].tobytes()) & 0xFFFFFFFF == int(g["crc"])
    got = oracle.gemm_complex(A, B)
    assert np.max(np.abs(got - g["D"])) / (np.max(np.abs(g["D"])) * np.sqrt(2 * K)) < 2e-7


def test_golden_complex_set_is_complete():
    assert len(glob.glob(os.path.join(GOLD, "ref_c32_*.npz"))) == 2


@pytest.mark.parametrize("M,N,K,threads", [(64, 64, 64, 1), (100, 150, 77, 4), (256, 256, 256, 8)])
def test_compiled_reference_within_rounding(oracle, M, N, K, threads):
    if not oracle.reference_available():
        pytest.skip("compiled reference (oracle/_ref) not present on this host")
    A = cplx(M, K, 21); B = cplx(K, N, 22)
    try:
        D, err = oracle.reference_cpu_gemm_c32(A, B, None, threads)
    except RuntimeError as e:
        pytest.skip(str(e))
    assert err == 0
    got = oracle.gemm_complex(A, B)
    assert np.max(np.abs(got - D)) / (np.max(np.abs(D)) * np.sqrt(2 * K)) < 2e-7
