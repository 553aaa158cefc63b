"""Parity of the two vector corners (matrix x vector, vector x matrix) through the C ABI
against the CPU oracle (its GEMM with N == 1 / M == 1: the same sum, k ascending).

The kernels sum in another order than the oracle's chain, so the bar is the GEMM one:
max|d| / (max|ref| * sqrt(K)) <= 1e-5 with fp32 inputs, <= 2e-3 with fp16 inputs and fp16
output, <= 1e-5 with fp16 inputs and fp32 output (products of halves are exact in fp32);
bit-exact where every partial sum is exactly representable.
"""
import numpy as np
import pytest

from decx_amd import synth

pytestmark = pytest.mark.gpu

TOL_F32 = 1e-5
TOL_F16 = 2e-3


@pytest.fixture(scope="module")
def hip():
    from decx_amd import hip as h
    h.init()
    return h


def rel_err(got, ref, K):
    ref = ref.astype(np.float64)
    scale = max(float(np.max(np.abs(ref))), 1e-30) * np.sqrt(max(K, 1))
    return float(np.max(np.abs(got.astype(np.float64) - ref))) / scale


def inputs(dtype, rows, cols, seed):
    return synth.uniform_f32(rows, cols, seed) if dtype == np.float32 else synth.normal_half(rows, cols, seed)


def vec(hip, data, column, pad=3):
    """A device vector: contiguous (1 x n) or strided (n x 1 with a pitch of `pad` elements), NaN in the gaps."""
    data = np.ascontiguousarray(data).reshape(-1)
    if column:
        return hip.DeviceMatrix(data.size, 1, data.dtype, pad, data[:, None], pad_value=np.nan)
    return hip.DeviceMatrix(1, data.size, data.dtype, data.size, data[None, :])


def out_vec(hip, n, dtype, column, pad=3):
    d = hip.DeviceMatrix(n, 1, dtype, pad) if column else hip.DeviceMatrix(1, n, dtype, n)
    d.upload_raw(np.full((d.rows, d.pitch), -777.0, dtype))
    return d


def read_vec(d):
    raw = d.download_raw()
    if d.cols == 1 and d.rows > 1 or d.pitch > d.cols:
        assert np.all(raw[:, 1:] == raw.dtype.type(-777.0)), "gaps of a strided output were written"
        return raw[:, 0].copy()
    return raw[0, :d.cols].copy()


def oracle_mv(oracle, A, x, c, alpha, beta, out_dtype):
    """Row dots as the oracle's GEMM with one column; fp16 inputs widen exactly to fp32."""
    Af, xf = A.astype(np.float32), x.astype(np.float32).reshape(-1, 1)
    cf = None if c is None else c.astype(np.float32).reshape(-1, 1)
    ref = oracle.gemm_f32(Af, xf, cf, alpha, beta) if cf is not None else oracle.gemm_f32(Af, xf)
    return ref.reshape(-1).astype(out_dtype)


def oracle_vm(oracle, x, B, c, alpha, beta, out_dtype):
    xf, Bf = x.astype(np.float32).reshape(1, -1), B.astype(np.float32)
    cf = None if c is None else c.astype(np.float32).reshape(1, -1)
    ref = oracle.gemm_f32(xf, Bf, cf, alpha, beta) if cf is not None else oracle.gemm_f32(xf, Bf)
    return ref.reshape(-1).astype(out_dtype)


CASES = [  # (in dtype, out dtype, tolerance)
    (np.float32, np.float32, TOL_F32),
    (np.float16, np.float32, TOL_F32),
    (np.float16, np.float16, TOL_F16),
]
MV_SHAPES = [(1, 1), (3, 5), (33, 63), (64, 256), (65, 257), (1000, 1), (257, 8200), (2, 20000), (700, 1030),
             # one shape per number of wavefronts that share a row (8, 4, 2, 1) and for two rows per wavefront
             (600, 300), (1100, 9001), (2100, 4100), (4100, 40), (8200, 33)]


@pytest.mark.parametrize("tin,tout,tol", CASES)
@pytest.mark.parametrize("M,K", MV_SHAPES)
@pytest.mark.parametrize("strided", [False, True])
def test_gemv_against_oracle(hip, oracle, tin, tout, tol, M, K, strided):
    A = inputs(tin, M, K, 201); x = inputs(tin, 1, K, 202).reshape(-1); c = inputs(tin, 1, M, 203).reshape(-1)
    per = 16 // np.dtype(tin).itemsize
    for pitch in ((K + per - 1) // per * per, K + 1):               # vector-load rows, then element-load rows
        dA = hip.DeviceMatrix(M, K, tin, pitch, A, pad_value=np.nan)
        dx = vec(hip, x, strided); dc = vec(hip, c, strided)
        dy = out_vec(hip, M, tout, strided)
        hip.gemv(dA, dx, dy); hip.sync()
        assert rel_err(read_vec(dy), oracle_mv(oracle, A, x, None, 1, 1, tout), K) <= tol
        hip.gemv(dA, dx, dy, dc, 0.5, -2.0); hip.sync()
        assert rel_err(read_vec(dy), oracle_mv(oracle, A, x, c, 0.5, -2.0, tout), K) <= tol


VM_SHAPES = [(1, 1), (5, 3), (63, 33), (256, 64), (257, 65), (1, 1000), (8200, 257), (20000, 2), (1030, 700)]


@pytest.mark.parametrize("tin,tout,tol", CASES)
@pytest.mark.parametrize("K,N", VM_SHAPES)
@pytest.mark.parametrize("strided", [False, True])
def test_gevm_against_oracle(hip, oracle, tin, tout, tol, K, N, strided):
    B = inputs(tin, K, N, 211); x = inputs(tin, 1, K, 212).reshape(-1); c = inputs(tin, 1, N, 213).reshape(-1)
    per = 16 // np.dtype(tin).itemsize
    for pitch in ((N + per - 1) // per * per, N + 1):
        dB = hip.DeviceMatrix(K, N, tin, pitch, B, pad_value=np.nan)
        dx = vec(hip, x, strided); dc = vec(hip, c, strided)
        dy = out_vec(hip, N, tout, strided)
        hip.gevm(dx, dB, dy); hip.sync()
        assert rel_err(read_vec(dy), oracle_vm(oracle, x, B, None, 1, 1, tout), K) <= tol
        hip.gevm(dx, dB, dy, dc, 0.5, -2.0); hip.sync()
        assert rel_err(read_vec(dy), oracle_vm(oracle, x, B, c, 0.5, -2.0, tout), K) <= tol


@pytest.mark.parametrize("tin,tout,tol", CASES)
@pytest.mark.parametrize("K,N", [(8192, 2048), (33000, 100)])
def test_gevm_split_over_k_through_a_workspace(hip, oracle, tin, tout, tol, K, N):
    """Few columns and a long K through decx_hip_gevm_*_ws: ranges of K on workgroups of their own, partial sums added
    in range order by the last workgroup of each column group.  Dense and strided x, y and c."""
    esz = np.dtype(tin).itemsize
    B = inputs(tin, K, N, 221); x = inputs(tin, 1, K, 222).reshape(-1); c = inputs(tin, 1, N, 223).reshape(-1)
    need = hip.lib().decx_hip_gemm_workspace(esz, 1, N, K)
    assert need > 0
    ws = hip.DeviceMatrix(1, need // 4, np.float32)
    ws.upload_raw(np.full((1, ws.pitch), np.nan, np.float32))
    per = 16 // esz
    dB = hip.DeviceMatrix(K, N, tin, (N + per - 1) // per * per, B, pad_value=np.nan)
    for strided_x, strided_y in ((False, False), (True, False), (False, True)):
        dx = vec(hip, x, strided_x); dc = vec(hip, c, strided_y)
        dy = out_vec(hip, N, tout, strided_y)
        hip.gevm(dx, dB, dy, workspace=ws); hip.sync()
        first = read_vec(dy)
        assert rel_err(first, oracle_vm(oracle, x, B, None, 1, 1, tout), K) <= tol
        hip.gevm(dx, dB, dy, workspace=ws); hip.sync()
        assert np.array_equal(read_vec(dy).view(np.uint8), first.view(np.uint8))
        hip.gevm(dx, dB, dy, dc, 0.5, -2.0, workspace=ws); hip.sync()
        assert rel_err(read_vec(dy), oracle_vm(oracle, x, B, c, 0.5, -2.0, tout), K) <= tol


@pytest.mark.parametrize("tin,tout", [(np.float32, np.float32), (np.float16, np.float32), (np.float16, np.float16)])
def test_exact_small_integer_sums(hip, tin, tout):
    """Small integers: every partial sum is an integer below 2^11, exact in any order and in fp16."""
    rng = np.random.default_rng(7)
    M, K = 300, 120
    A = rng.integers(-2, 3, (M, K)).astype(tin); x = rng.integers(-2, 3, K).astype(tin)
    want = (A.astype(np.int64) @ x.astype(np.int64)).astype(tout)
    dA = hip.DeviceMatrix(M, K, tin, data=A); dx = vec(hip, x, False); dy = out_vec(hip, M, tout, False)
    hip.gemv(dA, dx, dy); hip.sync()
    assert np.array_equal(read_vec(dy), want)
    xr = rng.integers(-2, 3, M).astype(tin)
    want = (xr.astype(np.int64) @ A.astype(np.int64)).astype(tout)
    dxr = vec(hip, xr, False); dyr = out_vec(hip, K, tout, False)
    hip.gevm(dxr, dA, dyr); hip.sync()
    assert np.array_equal(read_vec(dyr), want)


def test_gemm_entry_routes_both_corners(hip, oracle):
    """decx_hip_gemm_* with N == 1 or M == 1 takes the vector kernels and still matches the oracle."""
    K = 3000
    for dt, orc, tol, eb in ((np.float32, oracle.gemm_f32, TOL_F32, 4), (np.float16, oracle.gemm_f16, TOL_F16, 2)):
        assert hip.plan(eb, 500, 1, K).path == hip.PATH_GEMV
        assert hip.plan(eb, 1, 500, K).path == hip.PATH_GEVM
        A = inputs(dt, 500, K, 221); b = inputs(dt, K, 1, 222); c = inputs(dt, 500, 1, 223)
        dA = hip.DeviceMatrix(500, K, dt, data=A); db = hip.DeviceMatrix(K, 1, dt, 64, b); dc = hip.DeviceMatrix(500, 1, dt, 64, c)
        dD = hip.DeviceMatrix(500, 1, dt, 64)
        hip.gemm(dA, db, dD, dc, 1.5, 0.25); hip.sync()
        assert rel_err(dD.download(), orc(A, b, c, 1.5, 0.25), K) <= tol
        a = inputs(dt, 1, K, 224); B = inputs(dt, K, 500, 225); c = inputs(dt, 1, 500, 226)
        da = hip.DeviceMatrix(1, K, dt, data=a); dB = hip.DeviceMatrix(K, 500, dt, data=B); dc = hip.DeviceMatrix(1, 500, dt, data=c)
        dD = hip.DeviceMatrix(1, 500, dt)
        hip.gemm(da, dB, dD, dc, 1.5, 0.25); hip.sync()
        assert rel_err(dD.download(), orc(a, B, c, 1.5, 0.25), K) <= tol
        hip.gemm(da, dB, dD); hip.sync()
        assert rel_err(dD.download(), orc(a, B), K) <= tol


def test_full_size_linearity_and_checksum(hip):
    """8192 x 8192: the sum over outputs equals x . (column sums) / (row sums) . x; additivity in x."""
    n = 8192
    A = synth.uniform_f32(n, n, 231); x1 = synth.uniform_f32(1, n, 232).reshape(-1); x2 = synth.uniform_f32(1, n, 233).reshape(-1)
    dA = hip.DeviceMatrix(n, n, np.float32, data=A)
    A64 = A.astype(np.float64)
    for op, check in ((hip.gemv, A64.sum(axis=0)), (hip.gevm, A64.sum(axis=1))):
        ys = []
        for x in (x1, x2, x1 + x2):
            dx = vec(hip, x, False); dy = out_vec(hip, n, np.float32, False)
            (op(dA, dx, dy) if op is hip.gemv else op(dx, dA, dy)); hip.sync()
            ys.append(read_vec(dy).astype(np.float64))
        scale = np.max(np.abs(ys[2])) * np.sqrt(n)
        assert np.max(np.abs(ys[0] + ys[1] - ys[2])) / scale <= TOL_F32
        assert abs(ys[0].sum() - float(check @ x1.astype(np.float64))) / (np.abs(check).max() * n) <= TOL_F32


def test_invalid_arguments(hip):
    L = hip.lib()
    d = hip.DeviceMatrix(4, 4, np.float32, data=np.ones((4, 4), np.float32))
    assert L.decx_hip_gevm_f32(None, d.ptr, None, d.ptr, 4, 4, 4, 1, 1, 1, 1.0, 1.0, None) == -1
    assert L.decx_hip_gevm_f32(d.ptr, d.ptr, None, d.ptr, 4, 4, 3, 1, 1, 1, 1.0, 1.0, None) == -1      # ldb < N
    assert L.decx_hip_gevm_f16(d.ptr, d.ptr, None, d.ptr, 4, 4, 4, 0, 1, 1, 1.0, 1.0, 0, None) == -1   # incx == 0
    assert L.decx_hip_gemv_f16(d.ptr, d.ptr, d.ptr, d.ptr, 4, 4, 4, 1, 0, 1, 1.0, 1.0, 1, None) == -1  # incc == 0 with c
    assert L.decx_hip_gevm_f32(d.ptr, d.ptr, None, d.ptr, 4, 0, 4, 1, 1, 1, 1.0, 1.0, None) == 0       # empty output
