"""Parity of the fp64 GEMM (through the C ABI) against the CPU oracle.

Bar: max|d| / (max|ref| * sqrt(K)) <= 1e-14 for the matrix-core kernels (they sum in another order than the
oracle's chain; fp64 unit roundoff is 1.1e-16); the one-thread-per-element kernel runs the oracle's own chain
and must be bit-exact; small-integer products are exact on every path."""
import glob
import os

import numpy as np
import pytest

from decx_amd import synth

pytestmark = pytest.mark.gpu
GOLD = os.path.join(os.path.dirname(__file__), "golden")
TOL = 1e-14


@pytest.fixture(scope="module")
def hip():
    from decx_amd import hip as h
    h.init()
    return h


def rel_err(got, ref, K):
    scale = max(float(np.max(np.abs(ref))), 1e-300) * np.sqrt(max(K, 1))
    return float(np.max(np.abs(got - ref))) / scale


def run(hip, A, B, C=None, alpha=1.0, beta=1.0, tile=-1, plain=False, pitches=None, offsets=(0, 0, 0, 0)):
    M, K = A.shape
    N = B.shape[1]
    r16 = lambda v: (v + 15) // 16 * 16                       # the device pitch rule: 128 bytes
    pa, pb, pc, pd = pitches or (r16(K), r16(N), r16(N), r16(N))
    dA = hip.DeviceMatrix(M, K, np.float64, pa, A, pad_value=np.nan, offset_elems=offsets[0])
    dB = hip.DeviceMatrix(K, N, np.float64, pb, B, pad_value=np.nan, offset_elems=offsets[1])
    dC = hip.DeviceMatrix(M, N, np.float64, pc, C, pad_value=np.nan, offset_elems=offsets[2]) if C is not None else None
    dD = hip.DeviceMatrix(M, N, np.float64, pd, offset_elems=offsets[3])
    dD.upload_raw(np.full((M, pd), -12345.0))
    hip.gemm(dA, dB, dD, dC, alpha, beta, tile=tile, force_edge=plain)
    hip.sync()
    raw = dD.download_raw()
    assert np.all(raw[:, N:] == -12345.0), "padding columns of D were written"
    out = raw[:, :N].copy()
    assert not np.isnan(out).any(), "NaN leaked from pitch padding into the result"
    for d in (dA, dB, dC, dD):
        if d is not None:
            d.free()
    return out


SHAPES = [(1, 1, 1), (1, 7, 3), (7, 1, 3), (3, 5, 1), (31, 33, 17), (64, 64, 16), (65, 63, 15), (129, 257, 100),
          (255, 256, 257), (300, 20, 40), (20, 300, 1025), (2, 2, 4097), (256, 128, 64), (512, 384, 96)]


@pytest.mark.parametrize("M,N,K", SHAPES)
@pytest.mark.parametrize("tile", [0, 1, 2])
def test_ragged_shapes_every_tile(hip, oracle, M, N, K, tile):
    A = synth.uniform_f64(M, K, 901); B = synth.uniform_f64(K, N, 902); C = synth.uniform_f64(M, N, 903)
    assert rel_err(run(hip, A, B, tile=tile), oracle.gemm_f64(A, B), K) <= TOL
    assert rel_err(run(hip, A, B, C, 1.5, -0.5, tile=tile), oracle.gemm_f64(A, B, C, 1.5, -0.5), K) <= TOL


@pytest.mark.parametrize("K", [1, 2, 3, 7, 8, 9, 15, 16, 17, 23, 24, 25, 40, 101])
@pytest.mark.parametrize("tile", [0, 1, 2])
def test_every_k_remainder(hip, oracle, K, tile):
    A = synth.uniform_f64(70, K, 911); B = synth.uniform_f64(K, 91, 912)
    assert rel_err(run(hip, A, B, tile=tile), oracle.gemm_f64(A, B), K) <= TOL


def test_row_pitch_of_16_mib_takes_the_plain_kernel(hip, oracle):
    """256 rows of a 16 MiB pitch overflow the 32-bit lane offsets of the direct-load kernels: such
    operands run on the plain kernel, bit-exact to the oracle's chain."""
    M, N, K = 3, 40, 72
    A = synth.uniform_f64(M, K, 931); B = synth.uniform_f64(K, N, 932)
    got = run(hip, A, B, pitches=((1 << 21) + 64, 48, 48, 48))
    assert np.array_equal(got.view(np.uint64), oracle.gemm_f64(A, B).view(np.uint64))


@pytest.mark.parametrize("M,N,K", [(300, 300, 8192), (70, 130, 4099)])
def test_split_k_through_a_workspace(hip, oracle, M, N, K):
    """Few output tiles and a long K: partial products in double, added in a fixed order."""
    A = synth.uniform_f64(M, K, 941); B = synth.uniform_f64(K, N, 942); C = synth.uniform_f64(M, N, 943)
    need = hip.lib().decx_hip_gemm_workspace(8, M, N, K)
    assert need > 0
    ws = hip.DeviceMatrix(1, need // 8, np.float64)
    ws.upload_raw(np.full((1, ws.pitch), np.nan, np.float64))
    r16 = lambda v: (v + 15) // 16 * 16                       # the device pitch rule: 128 bytes

    def product(c, alpha, beta, workspace):
        dA = hip.DeviceMatrix(M, K, np.float64, r16(K), A, pad_value=np.nan); dB = hip.DeviceMatrix(K, N, np.float64, r16(N), B, pad_value=np.nan)
        dC = hip.DeviceMatrix(M, N, np.float64, r16(N), c, pad_value=np.nan) if c is not None else None
        dD = hip.DeviceMatrix(M, N, np.float64, r16(N))
        dD.upload_raw(np.full((M, r16(N)), -12345.0))
        hip.gemm(dA, dB, dD, dC, alpha, beta, workspace=workspace)
        hip.sync()
        raw = dD.download_raw()
        for d in (dA, dB, dC, dD):
            if d is not None:
                d.free()
        assert np.all(raw[:, N:] == -12345.0)
        return raw[:, :N].copy()

    first = product(None, 1.0, 1.0, ws)
    assert rel_err(first, oracle.gemm_f64(A, B), K) <= TOL
    assert np.array_equal(first, product(None, 1.0, 1.0, ws))
    assert rel_err(product(C, 1.5, -0.5, ws), oracle.gemm_f64(A, B, C, 1.5, -0.5), K) <= TOL
    ws.free()


def test_split_k_for_a_few_hundred_tiles(hip, oracle):
    """320 tiles of 64 x 64 (1.25 per CU) and a long K: with a workspace a tile per CU stays whole and the other 64 are
    cut along K, one range per CU.  Parity on sampled rows, the same result from run to run, untouched padding."""
    M, N, K = 1280, 1024, 4100
    A = synth.uniform_f64(M, K, 961); B = synth.uniform_f64(K, N, 962)
    plan = hip.plan(8, M, N, K)
    assert plan.k_splits > 1 and plan.tile_m == 64
    need = hip.lib().decx_hip_gemm_workspace(8, M, N, K)
    assert need == (20 * 16 - plan.whole_tiles) * plan.k_splits * 64 * 64 * 8        # a slot per workgroup of a split tile
    ws = hip.DeviceMatrix(1, need // 8, np.float64)
    ws.upload_raw(np.full((1, ws.pitch), np.nan, np.float64))
    r16 = lambda v: (v + 15) // 16 * 16
    dA = hip.DeviceMatrix(M, K, np.float64, r16(K), A, pad_value=np.nan); dB = hip.DeviceMatrix(K, N, np.float64, r16(N), B, pad_value=np.nan)

    def product(workspace):
        dD = hip.DeviceMatrix(M, N, np.float64, r16(N) + 16)
        dD.upload_raw(np.full((M, r16(N) + 16), -12345.0))
        hip.gemm(dA, dB, dD, workspace=workspace)
        hip.sync()
        raw = dD.download_raw()
        dD.free()
        assert np.all(raw[:, N:] == -12345.0)
        return raw[:, :N].copy()

    split = product(ws)
    rows = np.array([0, 1, 63, 64, 640, 1000, 1279], np.uint32)
    assert rel_err(split[rows], oracle.gemm_f64(A, B, rows=rows), K) <= TOL
    assert np.array_equal(split, product(ws))
    whole = product(None)
    assert np.max(np.abs(split - whole)) <= 1e-12 * np.sqrt(K)
    for d in (dA, dB, ws):
        d.free()


@pytest.mark.parametrize("M,N,K", [(4096, 1, 8192), (700, 1, 1030), (8200, 1, 33), (2100, 1, 4100), (33, 1, 257), (1, 1, 5),
                                   (1, 3000, 4096), (1, 100, 33000), (1, 9, 70), (1, 5000, 300), (1, 513, 16390)])
def test_vector_corners(hip, oracle, M, N, K):
    """N = 1 and M = 1 run on the bandwidth-bound vector kernels with sums in double; with the workspace the planner
    asks for, the column operand is copied into a dense vector first / a long K is split over workgroups."""
    A = synth.uniform_f64(M, K, 951); B = synth.uniform_f64(K, N, 952); C = synth.uniform_f64(M, N, 953)
    assert hip.plan(8, M, N, K).path == (hip.PATH_GEMV if N == 1 else hip.PATH_GEVM)
    need = hip.lib().decx_hip_gemm_workspace(8, M, N, K)
    assert (need > 0) == ((M, N, K) in [(4096, 1, 8192), (2100, 1, 4100), (1, 100, 33000), (1, 513, 16390)])
    ws = hip.DeviceMatrix(1, max(need // 8, 2), np.float64)
    ws.upload_raw(np.full((1, ws.pitch), np.nan, np.float64))
    r16 = lambda v: (v + 15) // 16 * 16

    def product(c, alpha, beta, workspace, pitches):
        pk, pn = pitches
        dA = hip.DeviceMatrix(M, K, np.float64, pk, A, pad_value=np.nan); dB = hip.DeviceMatrix(K, N, np.float64, pn, B, pad_value=np.nan)
        dC = hip.DeviceMatrix(M, N, np.float64, pn, c, pad_value=np.nan) if c is not None else None
        dD = hip.DeviceMatrix(M, N, np.float64, pn)
        dD.upload_raw(np.full((M, pn), -12345.0))
        hip.gemm(dA, dB, dD, dC, alpha, beta, workspace=workspace)
        hip.sync()
        raw = dD.download_raw()
        for d in (dA, dB, dC, dD):
            if d is not None:
                d.free()
        assert np.all(raw[:, N:] == -12345.0)
        return raw[:, :N].copy()

    for pitches in ((r16(K), r16(N)), (K + 1, N + 1)):          # 128-bit loads, then element loads
        for workspace in (None, ws):
            got = product(None, 1.0, 1.0, workspace, pitches)
            assert rel_err(got, oracle.gemm_f64(A, B), K) <= TOL
            assert np.array_equal(got, product(None, 1.0, 1.0, workspace, pitches))
            assert rel_err(product(C, 1.5, -0.5, workspace, pitches), oracle.gemm_f64(A, B, C, 1.5, -0.5), K) <= TOL
    ws.free()


def test_plain_kernel_is_the_oracle_chain(hip, oracle):
    """Unaligned operands (and K == 0) take the one-thread-per-element kernel: the oracle's own k-ascending fma chain."""
    M, N, K = 70, 90, 50
    A = synth.uniform_f64(M, K, 921); B = synth.uniform_f64(K, N, 922); C = synth.uniform_f64(M, N, 923)
    got = run(hip, A, B, C, 2.0, 1.0, pitches=(K + 1, N + 3, N + 5, N + 1), offsets=(1, 3, 1, 1))
    assert np.array_equal(got.view(np.uint64), oracle.gemm_f64(A, B, C, 2.0, 1.0).view(np.uint64))
    got = run(hip, A, B, plain=True)
    assert np.array_equal(got.view(np.uint64), oracle.gemm_f64(A, B).view(np.uint64))
    zero_k = run(hip, np.zeros((5, 0)), np.zeros((0, 7)), np.ones((5, 7)), 3.0, 0.5)
    assert np.all(zero_k == 0.5)
    assert hip.plan(8, 70, 90, 50, aligned=False).edge == 1 and hip.plan(8, 4096, 4096, 4096).tile_n == 128


@pytest.mark.parametrize("path", sorted(glob.glob(os.path.join(GOLD, "ref_f64_*.npz"))))
def test_against_reference_outputs(hip, path):
    """Outputs of the reference's double-precision CPU GEMM, committed as data."""
    g = np.load(path)
    M, N, K = int(g["M"]), int(g["N"]), int(g["K"])
    A = synth.uniform_f64(M, K, int(g["seed_a"])); B = synth.uniform_f64(K, N, int(g["seed_b"]))
    C = synth.uniform_f64(M, N, int(g["seed_c"])) if bool(g["with_c"]) else None
    assert rel_err(run(hip, A, B, C), g["D"], K) <= TOL
    got = run(hip, A, B, C, plain=True)
    if C is None:
        assert np.array_equal(got.view(np.uint64), g["D"].view(np.uint64))     # same chain, bit for bit


def test_exact_closed_forms(hip):
    n = 200
    rng = np.random.default_rng(5)
    X = rng.integers(-8, 9, (n, 150)).astype(np.float64)
    assert np.array_equal(run(hip, np.eye(n), X), X)
    a = rng.integers(-99, 100, (130, 96)).astype(np.float64); b = rng.integers(-99, 100, (96, 140)).astype(np.float64)
    for tile in (0, 1, 2):
        assert np.array_equal(run(hip, a, b, tile=tile), (a.astype(np.int64) @ b.astype(np.int64)).astype(np.float64))
    big = np.full((40, 3000), 2.0 ** 20) ; ones = np.ones((3000, 33))
    assert np.all(run(hip, big, ones) == 3000 * 2.0 ** 20)


def test_2048_cubed_sampled_and_checksum(hip, oracle):
    n = 2048
    A = synth.uniform_f64(n, n, 931); B = synth.uniform_f64(n, n, 932)
    got = run(hip, A, B)
    rows = np.array([0, 1, 255, 256, 1000, 2047], np.uint32)
    assert rel_err(got[rows], oracle.gemm_f64(A, B, rows=rows), n) <= TOL
    colsum = A.sum(axis=0) @ B
    assert np.max(np.abs(got.sum(axis=0) - colsum)) / np.max(np.abs(colsum)) < 1e-12


def test_invalid_arguments(hip):
    L = hip.lib()
    d = hip.DeviceMatrix(4, 4, np.float64, data=np.ones((4, 4)))
    assert L.decx_hip_gemm_f64(None, d.ptr, None, d.ptr, 4, 4, 4, 4, 4, 0, 4, 1.0, 1.0, None) == -1
    assert L.decx_hip_gemm_f64(d.ptr, d.ptr, None, d.ptr, 4, 4, 4, 3, 4, 0, 4, 1.0, 1.0, None) == -1
    assert L.decx_hip_gemm_f64_tile(d.ptr, d.ptr, None, d.ptr, 4, 4, 4, 4, 4, 0, 4, 1.0, 1.0, None, 7, 0) == -1
    assert L.decx_hip_gemm_f64(d.ptr, d.ptr, None, d.ptr, 0, 4, 4, 4, 4, 0, 4, 1.0, 1.0, None) == 0
