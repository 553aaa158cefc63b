"""Operands beyond 4 GiB: every row offset past 2^32 bytes has to be 64-bit arithmetic in the kernels (the lane offsets
of the direct loads are 32-bit by design, relative to a tile's 64-bit base).  Inputs are small integers, so every
product and sum is exact in every precision and the expected results are closed forms; nothing of this size goes through the CPU
oracle."""
import ctypes

import numpy as np
import pytest

from decx_amd import hip

pytestmark = pytest.mark.gpu

ROWS = 70000                       # of 65536 bytes each (4.59 GB): rows from 65536 on start beyond 4 GiB
ROW_BYTES = 65536


def upload_by_panels(dm, row_values):
    """Row i of the matrix is row_values[i] in every column (uploaded 4096 rows at a time)."""
    L = hip.lib()
    step = 4096
    for r0 in range(0, dm.rows, step):
        r1 = min(dm.rows, r0 + step)
        host = np.ascontiguousarray(np.broadcast_to(row_values[r0:r1, None], (r1 - r0, dm.pitch)), dtype=dm.dtype)
        dst = ctypes.c_void_p(dm.ptr.value + r0 * dm.pitch * dm.dtype.itemsize)
        hip.check(L.decx_hip_memcpy2d_async(dst, host.nbytes, host.ctypes.data, host.nbytes, host.nbytes, 1, 0, None), "upload")
        hip.check(L.decx_hip_stream_sync(None))


@pytest.fixture(scope="module", params=[np.float32, np.float16, np.float64], ids=["fp32", "fp16", "fp64"])
def big(request):
    hip.init()
    dt = np.dtype(request.param)
    cols = ROW_BYTES // dt.itemsize
    rows = ((np.arange(ROWS) % 5) - 2).astype(dt)                     # -2 .. 2, by row
    dm = hip.DeviceMatrix(ROWS, cols, dt, cols)
    assert dm.nbytes > (1 << 32)
    upload_by_panels(dm, rows)
    yield dm, rows
    dm.free()


@pytest.mark.timeout(300)
def test_gemm_reads_rows_of_a_beyond_4_gib(big):
    A, rows = big
    dt, COLS = A.dtype, A.cols
    N = 96
    k = np.arange(COLS)[:, None]
    j = np.arange(N)[None, :]
    b = (((k + j) % 3) - 1).astype(dt)                                # -1, 0, 1
    B = hip.DeviceMatrix(COLS, N, dt, 128, data=b, pad_value=np.nan)
    D = hip.DeviceMatrix(ROWS, N, dt, 128)
    need = hip.lib().decx_hip_gemm_workspace(dt.itemsize, ROWS, N, COLS)
    W = hip.DeviceMatrix(1, max(need // 4, 1), np.float32) if need else None
    hip.gemm(A, B, D, workspace=W)
    hip.sync()
    want = rows[:, None].astype(np.float64) * b.astype(np.float64).sum(axis=0)[None, :]
    assert np.array_equal(want, want.astype(dt).astype(np.float64))   # representable: the comparison is exact
    got = D.download()
    assert np.array_equal(got.astype(np.float64), want)
    for tile in (hip.TILE_LARGE, hip.TILE_MEDIUM, hip.TILE_SMALL):
        D.upload_raw(np.full((ROWS, 128), -7.0, dt))
        hip.gemm(A, B, D, tile=tile)
        hip.sync()
        assert np.array_equal(D.download().astype(np.float64), want), tile
    for d in (B, D) + ((W,) if W else ()):
        d.free()


@pytest.mark.timeout(300)
def test_vector_kernels_read_rows_beyond_4_gib(big):
    A, rows = big
    dt, COLS = A.dtype, A.cols
    f64 = dt == np.float64                 # fp64 vectors have no entry points of their own: N = 1 / M = 1 of the GEMM entry
    # matrix x vector: y[i] = rows[i] * sum(x); x has as many -1 as +1 and a 2 in every 8th place
    xv = np.array([-1, 0, 1, 0, -1, 2, 1, 0], dt)[np.arange(COLS) % 8]
    if f64:
        x = hip.DeviceMatrix(COLS, 1, dt, 2, data=xv[:, None])
        y = hip.DeviceMatrix(ROWS, 1, dt, 2)
        hip.gemm(A, x, y)
    else:
        x = hip.DeviceMatrix(1, COLS, dt, COLS, data=xv[None, :])
        y = hip.DeviceMatrix(1, ROWS, dt, ROWS)
        hip.gemv(A, x, y)
    hip.sync()
    want_y = rows.astype(np.float64) * float(xv.astype(np.float64).sum())
    assert np.array_equal(want_y, want_y.astype(dt).astype(np.float64))
    assert np.array_equal(y.download().reshape(-1).astype(np.float64), want_y)
    # vector x matrix with the same buffer as the right operand (70000 rows): y[j] = sum_k x[k] rows[k]
    xk = ((np.arange(ROWS) % 3) - 1).astype(dt)
    x2 = hip.DeviceMatrix(1, ROWS, dt, ROWS, data=xk[None, :])
    y2 = hip.DeviceMatrix(1, COLS, dt, COLS)
    (hip.gemm if f64 else hip.gevm)(x2, A, y2)
    hip.sync()
    want = float(np.dot(xk.astype(np.float64), rows.astype(np.float64)))
    assert want == float(dt.type(want))
    assert np.array_equal(y2.download()[0].astype(np.float64), np.full(COLS, want))
    need = hip.lib().decx_hip_gemm_workspace(dt.itemsize, 1, COLS, ROWS)
    if need:
        W = hip.DeviceMatrix(1, need // 4, np.float32)
        y2.upload_raw(np.full((1, COLS), -7.0, dt))
        (hip.gemm if f64 else hip.gevm)(x2, A, y2, workspace=W)
        hip.sync()
        assert np.array_equal(y2.download()[0].astype(np.float64), np.full(COLS, want))
        W.free()
    for d in (x, y, x2, y2):
        d.free()


@pytest.mark.timeout(300)
def test_gemm_writes_rows_of_d_beyond_4_gib():
    hip.init()
    M, N, K = 40000, 30016, 32                                        # D: 4.8 GB
    a = np.broadcast_to((np.arange(M) % 3).astype(np.float32)[:, None], (M, K))
    b = np.broadcast_to(((np.arange(N) % 5) - 2).astype(np.float32)[None, :], (K, N))
    A = hip.DeviceMatrix(M, K, np.float32, K, data=a)
    B = hip.DeviceMatrix(K, N, np.float32, N, data=b)
    D = hip.DeviceMatrix(M, N, np.float32, N)
    assert D.nbytes > (1 << 32)
    hip.gemm(A, B, D)
    hip.sync()
    L = hip.lib()
    want_cols = K * ((np.arange(N) % 5) - 2).astype(np.float64)
    for r0 in (0, 35000, M - 2048):                                   # bands of rows on both sides of 4 GiB
        host = np.empty((2048, N), np.float32)
        src = ctypes.c_void_p(D.ptr.value + r0 * N * 4)
        hip.check(L.decx_hip_memcpy2d_async(host.ctypes.data, host.nbytes, src, host.nbytes, host.nbytes, 1, 1, None), "download")
        hip.check(L.decx_hip_stream_sync(None))
        want = (np.arange(r0, r0 + 2048) % 3).astype(np.float64)[:, None] * want_cols[None, :]
        assert np.array_equal(host.astype(np.float64), want), r0
    for d in (A, B, D):
        d.free()
