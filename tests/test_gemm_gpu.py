"""Parity of the HIP GEMM path (through the C ABI) against the CPU oracle.

Bar: max|d| / (max|ref| * sqrt(K)) <= 1e-5 for fp32 and <= 2e-3 for fp16; bit-exact where
the mathematics makes the answer exactly representable (identity, small-integer products).
"""
import glob
import os

import numpy as np
import pytest

from decx_amd import synth

pytestmark = pytest.mark.gpu

GOLD = os.path.join(os.path.dirname(__file__), "golden")
TOL_F32 = 1e-5
TOL_F16 = 2e-3


@pytest.fixture(scope="module")
def hip():
    from decx_amd import hip as h
    h.init()                    # raises if the library or the GPU is missing: no fallback
    return h


def rel_err(got, ref, K):
    ref = ref.astype(np.float64)
    scale = max(float(np.max(np.abs(ref))), 1e-30) * np.sqrt(max(K, 1))
    return float(np.max(np.abs(got.astype(np.float64) - ref))) / scale


def device_pitch(cols, dtype):
    """The reference's device pitch rule: rows padded to 128 bytes
    (srcs/modules/core/classes/GPU_Matrix.cu:35-61)."""
    per = 128 // np.dtype(dtype).itemsize
    return (cols + per - 1) // per * per


def run(hip, A, B, C=None, alpha=1.0, beta=1.0, tile=-1, force_edge=False, pitches=None, offsets=(0, 0, 0, 0)):
    """Uploads with NaN-poisoned padding, runs, checks the padding of D is untouched."""
    dt = A.dtype
    M, K = A.shape
    N = B.shape[1]
    pa, pb, pc, pd = pitches or (device_pitch(K, dt), device_pitch(N, dt), device_pitch(N, dt), device_pitch(N, dt))
    dA = hip.DeviceMatrix(M, K, dt, pa, A, pad_value=np.nan, offset_elems=offsets[0])
    dB = hip.DeviceMatrix(K, N, dt, pb, B, pad_value=np.nan, offset_elems=offsets[1])
    dC = hip.DeviceMatrix(M, N, dt, pc, C, pad_value=np.nan, offset_elems=offsets[2]) if C is not None else None
    sentinel = np.full((M, pd), -12345.0, dt)
    dD = hip.DeviceMatrix(M, N, dt, pd, offset_elems=offsets[3])
    dD.upload_raw(sentinel)
    hip.gemm(dA, dB, dD, dC, alpha, beta, tile=tile, force_edge=force_edge)
    hip.sync()
    raw = dD.download_raw()
    assert np.all(raw[:, N:] == dt.type(-12345.0)), "padding columns of D were written"
    out = raw[:, :N].copy()
    assert not np.isnan(out).any(), "NaN leaked from pitch padding into the result"
    for d in (dA, dB, dC, dD):
        if d is not None:
            d.free()
    return out


# ------------------------------------------------------------------ golden fixtures

@pytest.mark.parametrize("path", sorted(glob.glob(os.path.join(GOLD, "*_f32_*.npz"))))
def test_golden_f32(hip, path):
    g = np.load(path)
    M, N, K = int(g["M"]), int(g["N"]), int(g["K"])
    A = synth.uniform_f32(M, K, int(g["seed_a"])); B = synth.uniform_f32(K, N, int(g["seed_b"]))
    C = None; alpha = beta = 1.0
    if "with_c" in g.files and bool(g["with_c"]):
        C = synth.uniform_f32(M, N, int(g["seed_c"]))
        if not np.isnan(g["alpha"]):
            alpha, beta = float(g["alpha"]), float(g["beta"])
    for tile in (-1, 0, 1, 2):
        got = run(hip, A, B, C, alpha, beta, tile=tile)
        assert rel_err(got, g["D"], K) <= TOL_F32, (path, tile)


@pytest.mark.parametrize("path", sorted(glob.glob(os.path.join(GOLD, "orc_f16_*.npz"))))
def test_golden_f16(hip, path):
    g = np.load(path)
    K = int(g["K"])
    A = g["A"].view(np.float16); B = g["B"].view(np.float16)
    C = g["C"].view(np.float16) if bool(g["with_c"]) else None
    for tile in (-1, 0, 1, 2):
        got = run(hip, A, B, C, float(g["alpha"]), float(g["beta"]), tile=tile)
        assert rel_err(got, g["D"].view(np.float16), K) <= TOL_F16, (path, tile)


# ------------------------------------------------------------------ the benchmark configurations, full or sampled

def sample_rows(M, count, seed):
    rng = np.random.default_rng(seed)
    rows = set(rng.choice(M, size=min(count, M), replace=False).tolist())
    rows.update([0, M - 1])                       # first and last row always
    return np.array(sorted(rows), np.uint32)


def test_config1_f32_1024_cubed(hip, oracle):
    M = N = K = 1024
    sa, sb, _ = synth.seeds(1)
    A = synth.uniform_f32(M, K, sa); B = synth.uniform_f32(K, N, sb)
    ref = oracle.gemm_f32(A, B)
    for tile in (-1, 0, 1, 2):
        assert rel_err(run(hip, A, B, tile=tile), ref, K) <= TOL_F32, tile


def test_config2_f32_ragged_with_and_without_c(hip, oracle):
    M, N, K = 1000, 1500, 777
    sa, sb, sc = synth.seeds(2)
    A = synth.uniform_f32(M, K, sa); B = synth.uniform_f32(K, N, sb); C = synth.uniform_f32(M, N, sc)
    ref_ab = oracle.gemm_f32(A, B)
    ref_abc = oracle.gemm_f32(A, B, C)                 # the CPU entry point's D = A.B + C
    ref_axpby = oracle.gemm_f32(A, B, C, 1.0, 1.0)     # the GPU entry point with alpha = beta = 1
    for tile in (-1, 0, 1, 2):
        assert rel_err(run(hip, A, B, tile=tile), ref_ab, K) <= TOL_F32
        got = run(hip, A, B, C, 1.0, 1.0, tile=tile)
        assert rel_err(got, ref_abc, K) <= TOL_F32
        assert rel_err(got, ref_axpby, K) <= TOL_F32
    got = run(hip, A, B, C, -0.75, 2.5)
    assert rel_err(got, oracle.gemm_f32(A, B, C, -0.75, 2.5), K) <= TOL_F32


def test_config3_f16_4096_cubed_sampled(hip, oracle):
    M = N = K = 4096
    sa, sb, _ = synth.seeds(3)
    A = synth.normal_half(M, K, sa); B = synth.normal_half(K, N, sb)
    rows = sample_rows(M, 96, 3)
    ref = oracle.gemm_f16(A, B, rows=rows)
    got = run(hip, A, B)
    assert rel_err(got[rows], ref, K) <= TOL_F16
    # size-independent property: scaling A by 2 (exact in binary16) scales D by exactly 2
    got2 = run(hip, (A * np.float16(2)).astype(np.float16), B)
    assert np.array_equal(got2[rows], (got[rows] * np.float16(2)).astype(np.float16))


def test_config4_f32_8192_cubed_sampled(hip, oracle):
    M = N = K = 8192
    sa, sb, _ = synth.seeds(4)
    A = synth.uniform_f32(M, K, sa); B = synth.uniform_f32(K, N, sb)
    rows = sample_rows(M, 64, 4)
    ref = oracle.gemm_f32(A, B, rows=rows)
    got = run(hip, A, B)
    assert rel_err(got[rows], ref, K) <= TOL_F32
    # column checksum: (1^T A) B == 1^T (A B), in float64 on the host
    colsum = A.astype(np.float64).sum(axis=0) @ B.astype(np.float64)
    assert np.max(np.abs(got.astype(np.float64).sum(axis=0) - colsum)) / np.max(np.abs(colsum)) < 1e-5


def test_config5a_f32_tall_skinny_sampled(hip, oracle):
    M, N, K = 65536, 256, 1024
    sa, sb, _ = synth.seeds(5)
    A = synth.uniform_f32(M, K, sa); B = synth.uniform_f32(K, N, sb)
    rows = sample_rows(M, 512, 5)
    ref = oracle.gemm_f32(A, B, rows=rows)
    got = run(hip, A, B)
    assert rel_err(got[rows], ref, K) <= TOL_F32


def test_config5b_f32_gemv(hip, oracle):
    M, N, K = 8192, 1, 8192
    sa, sb, sc = synth.seeds(6)
    A = synth.uniform_f32(M, K, sa); B = synth.uniform_f32(K, N, sb); C = synth.uniform_f32(M, N, sc)
    assert hip.plan(4, M, N, K).path == hip.PATH_GEMV
    assert rel_err(run(hip, A, B), oracle.gemm_f32(A, B), K) <= TOL_F32
    assert rel_err(run(hip, A, B, C, 0.5, -2.0), oracle.gemm_f32(A, B, C, 0.5, -2.0), K) <= TOL_F32
    # the columns stored dense, as de::GPU_Matrix keeps a single column: the same sums
    dense = (device_pitch(K, np.float32), 1, 1, 1)
    assert np.array_equal(run(hip, A, B, pitches=dense), run(hip, A, B))
    assert np.array_equal(run(hip, A, B, C, 0.5, -2.0, pitches=dense), run(hip, A, B, C, 0.5, -2.0))
    # and the same column through the tiled kernel
    assert rel_err(run(hip, A, B, tile=2), oracle.gemm_f32(A, B), K) <= TOL_F32


# ------------------------------------------------------------------ edge cases

SHAPES = [(1, 1, 1), (1, 7, 3), (7, 1, 3), (3, 5, 1), (31, 33, 17), (64, 64, 16), (65, 63, 15), (129, 257, 100),
          (255, 256, 257), (300, 20, 40), (20, 300, 1025), (2, 2, 4097)]


@pytest.mark.parametrize("M,N,K", SHAPES)
@pytest.mark.parametrize("tile", [0, 1, 2])
def test_f32_ragged_shapes_every_tile(hip, oracle, M, N, K, tile):
    A = synth.uniform_f32(M, K, 101); B = synth.uniform_f32(K, N, 102); C = synth.uniform_f32(M, N, 103)
    assert rel_err(run(hip, A, B, tile=tile), oracle.gemm_f32(A, B), K) <= TOL_F32
    assert rel_err(run(hip, A, B, C, 1.5, -0.5, tile=tile), oracle.gemm_f32(A, B, C, 1.5, -0.5), K) <= TOL_F32


@pytest.mark.parametrize("K", [2, 5, 8, 15, 16, 17, 31, 32, 33, 47, 48, 63, 64, 65, 101, 130])
@pytest.mark.parametrize("tile", [0, 1, 2])
def test_f32_every_k_remainder(hip, oracle, K, tile):
    """K around the slab depths (16 and 32): full slabs only, a partial last slab only, both; the pitch
    padding next to the last k holds NaN, so a product that reads past K shows."""
    M, N = 70, 91
    A = synth.uniform_f32(M, K, 161); B = synth.uniform_f32(K, N, 162); C = synth.uniform_f32(M, N, 163)
    assert rel_err(run(hip, A, B, tile=tile), oracle.gemm_f32(A, B), K) <= TOL_F32
    assert rel_err(run(hip, A, B, C, -1.0, 0.5, tile=tile), oracle.gemm_f32(A, B, C, -1.0, 0.5), K) <= TOL_F32


@pytest.mark.parametrize("M,N", [(70, 5), (300, 20), (1000, 32), (129, 31), (4100, 24)])
@pytest.mark.parametrize("K", [1, 31, 32, 33, 64, 100, 777])
def test_f32_outputs_of_at_most_32_columns(hip, oracle, M, N, K):
    """At most 32 columns: the smallest tile class runs as 128 x 32 (B rows of 128 bytes, k rows r and r + 4 stored
    side by side).  Planner's choice and the forced smallest class, every K remainder around the slab depth."""
    A = synth.uniform_f32(M, K, 211); B = synth.uniform_f32(K, N, 212); C = synth.uniform_f32(M, N, 213)
    plan = hip.plan(4, M, N, K)
    assert (plan.tile_m, plan.tile_n) == (128, 32)
    for tile in (-1, 2):
        assert rel_err(run(hip, A, B, tile=tile), oracle.gemm_f32(A, B), K) <= TOL_F32
        assert rel_err(run(hip, A, B, C, 1.5, -0.5, tile=tile), oracle.gemm_f32(A, B, C, 1.5, -0.5), K) <= TOL_F32


def test_f32_large_ragged_sampled(hip, oracle):
    """A ragged problem large enough for several rounds of workgroups per CU, planner's choice of tile."""
    M, N, K = 3001, 2903, 3107
    A = synth.uniform_f32(M, K, 171); B = synth.uniform_f32(K, N, 172)
    rows = sample_rows(M, 192, 7)
    got = run(hip, A, B)
    assert rel_err(got[rows], oracle.gemm_f32(A, B, rows=rows), K) <= TOL_F32
    colsum = A.astype(np.float64).sum(axis=0) @ B.astype(np.float64)       # checksum over all rows
    assert np.max(np.abs(got.astype(np.float64).sum(axis=0) - colsum)) / np.max(np.abs(colsum)) < 1e-5


@pytest.mark.parametrize("M,N,K", SHAPES + [(193, 385, 130), (500, 390, 200)])
@pytest.mark.parametrize("tile", [0, 1, 2, 3, 4, 5])
def test_f16_ragged_shapes_every_tile(hip, oracle, M, N, K, tile):
    A = synth.normal_half(M, K, 111); B = synth.normal_half(K, N, 112); C = synth.normal_half(M, N, 113)
    assert rel_err(run(hip, A, B, tile=tile), oracle.gemm_f16(A, B), K) <= TOL_F16
    assert rel_err(run(hip, A, B, C, 1.5, -0.5, tile=tile), oracle.gemm_f16(A, B, C, 1.5, -0.5), K) <= TOL_F16


@pytest.mark.parametrize("dtype", [np.float32, np.float16])
def test_unaligned_pitches_and_bases(hip, oracle, dtype):
    """Pitches that are not multiples of 16 bytes and bases off by one element: the kernels
    must fall back to element loads, never to misaligned vector loads."""
    M, N, K = 70, 90, 50
    if dtype == np.float32:
        A = synth.uniform_f32(M, K, 121); B = synth.uniform_f32(K, N, 122); C = synth.uniform_f32(M, N, 123)
        ref = oracle.gemm_f32(A, B, C, 2.0, 1.0); tol = TOL_F32
    else:
        A = synth.normal_half(M, K, 121); B = synth.normal_half(K, N, 122); C = synth.normal_half(M, N, 123)
        ref = oracle.gemm_f16(A, B, C, 2.0, 1.0); tol = TOL_F16
    for tile in (0, 1, 2):
        got = run(hip, A, B, C, 2.0, 1.0, tile=tile, pitches=(K + 1, N + 3, N + 5, N + 1), offsets=(1, 3, 1, 1))
        assert rel_err(got, ref, K) <= tol


@pytest.mark.parametrize("dtype", [np.float32, np.float16])
def test_row_pitch_of_16_mib_takes_the_register_staged_kernels(hip, oracle, dtype):
    """The direct-load kernels address a tile with 32-bit lane offsets, which 256 rows of a 16 MiB
    pitch overflow: such operands must be routed to the kernels with full 64-bit addresses."""
    M, N, K = 3, 40, 72
    pitch_a = (1 << 24) // np.dtype(dtype).itemsize + 64
    if dtype == np.float32:
        A = synth.uniform_f32(M, K, 141); B = synth.uniform_f32(K, N, 142)
        ref = oracle.gemm_f32(A, B); tol = TOL_F32
    else:
        A = synth.normal_half(M, K, 141); B = synth.normal_half(K, N, 142)
        ref = oracle.gemm_f16(A, B); tol = TOL_F16
    pn = device_pitch(N, dtype)
    for tile in (0, 2):
        assert rel_err(run(hip, A, B, tile=tile, pitches=(pitch_a, pn, pn, pn)), ref, K) <= tol


@pytest.mark.parametrize("M,N,K", [(300, 300, 8192), (64, 64, 4099), (130, 70, 2500), (512, 512, 1024), (33, 1000, 3000), (4100, 20, 4099)])
def test_f32_split_k_through_a_workspace(hip, oracle, M, N, K):
    """Few output tiles and a long K: with a workspace the product is split along K and the partial products are added
    in a fixed order.  Parity with the oracle, identical results from run to run, C / alpha / beta, untouched padding,
    and a workspace that is too small simply means no split."""
    A = synth.uniform_f32(M, K, 151); B = synth.uniform_f32(K, N, 152); C = synth.uniform_f32(M, N, 153)
    need = hip.lib().decx_hip_gemm_f32_workspace(M, N, K)
    assert need > 0 and need % 16 == 0
    ws = hip.DeviceMatrix(1, need // 4, np.float32)
    ws.upload_raw(np.full((1, ws.pitch), np.nan, np.float32))            # partial products never read what they did not write
    pa, pn = device_pitch(K, np.float32), device_pitch(N, np.float32)

    def product(c, alpha, beta, workspace):
        dA = hip.DeviceMatrix(M, K, np.float32, pa, A, pad_value=np.nan); dB = hip.DeviceMatrix(K, N, np.float32, pn, B, pad_value=np.nan)
        dC = hip.DeviceMatrix(M, N, np.float32, pn, c, pad_value=np.nan) if c is not None else None
        dD = hip.DeviceMatrix(M, N, np.float32, pn)
        dD.upload_raw(np.full((M, pn), -12345.0, np.float32))
        hip.gemm(dA, dB, dD, dC, alpha, beta, workspace=workspace)
        hip.sync()
        raw = dD.download_raw()
        for d in (dA, dB, dC, dD):
            if d is not None:
                d.free()
        assert np.all(raw[:, N:] == np.float32(-12345.0))
        return raw[:, :N].copy()

    first = product(None, 1.0, 1.0, ws)
    assert rel_err(first, oracle.gemm_f32(A, B), K) <= TOL_F32
    assert np.array_equal(first, product(None, 1.0, 1.0, ws))             # fixed summation order
    assert rel_err(product(C, 1.5, -0.5, ws), oracle.gemm_f32(A, B, C, 1.5, -0.5), K) <= TOL_F32
    plain = product(None, 1.0, 1.0, None)
    assert rel_err(plain, oracle.gemm_f32(A, B), K) <= TOL_F32
    small = hip.DeviceMatrix(1, 64, np.float32)
    assert np.array_equal(product(None, 1.0, 1.0, small), plain)          # too small: the plain kernel runs
    for d in (ws, small):
        d.free()


@pytest.mark.parametrize("M,N,K", [(300, 300, 8192), (70, 130, 4099), (512, 384, 2048)])
def test_f16_split_k_through_a_workspace(hip, oracle, M, N, K):
    """fp16 products keep their partial products in fp32 and round once after the sum."""
    A = synth.normal_half(M, K, 161); B = synth.normal_half(K, N, 162); C = synth.normal_half(M, N, 163)
    need = hip.lib().decx_hip_gemm_workspace(2, M, N, K)
    assert need > 0
    ws = hip.DeviceMatrix(1, need // 4, np.float32)
    ws.upload_raw(np.full((1, ws.pitch), np.nan, np.float32))
    pa, pn = device_pitch(K, np.float16), device_pitch(N, np.float16)

    def product(c, alpha, beta, workspace):
        dA = hip.DeviceMatrix(M, K, np.float16, pa, A, pad_value=np.nan); dB = hip.DeviceMatrix(K, N, np.float16, pn, B, pad_value=np.nan)
        dC = hip.DeviceMatrix(M, N, np.float16, pn, c, pad_value=np.nan) if c is not None else None
        dD = hip.DeviceMatrix(M, N, np.float16, pn)
        dD.upload_raw(np.full((M, pn), -12345.0, np.float16))
        hip.gemm(dA, dB, dD, dC, alpha, beta, workspace=workspace)
        hip.sync()
        raw = dD.download_raw()
        for d in (dA, dB, dC, dD):
            if d is not None:
                d.free()
        assert np.all(raw[:, N:] == np.float16(-12345.0))
        return raw[:, :N].copy()

    first = product(None, 1.0, 1.0, ws)
    assert rel_err(first, oracle.gemm_f16(A, B), K) <= TOL_F16
    assert np.array_equal(first.view(np.uint16), product(None, 1.0, 1.0, ws).view(np.uint16))
    assert rel_err(product(C, 1.5, -0.5, ws), oracle.gemm_f16(A, B, C, 1.5, -0.5), K) <= TOL_F16
    assert rel_err(product(None, 1.0, 1.0, None), oracle.gemm_f16(A, B), K) <= TOL_F16
    ws.free()


@pytest.mark.parametrize("dtype,M,N,K,tile,splits,whole", [
    (np.float32, 1280, 1024, 4096, 64, 4, 256),     # 320 tiles of 64 x 64, 1.25 per CU: a whole one per CU, the other 64 on 4 ranges
    (np.float32, 1536, 1536, 1536, 64, 4, 512),     # 2.25 per CU: two whole per CU and a quarter of another
    (np.float32, 1664, 2048, 2048, 64, 4, 768),     # 3.25 per CU
    (np.float32, 1100, 1100, 1100, 64, 3, 256),     # ragged output, K not a multiple of the range, 68 split tiles on 204 workgroups
    (np.float32, 900, 700, 4100, 64, 3, 0),         # fewer tiles than CUs: all of them on 3 ranges
    (np.float16, 1280, 1024, 6144, 128, 3, 0),      # 80 tiles of 128 x 128 on 3 ranges
    (np.float16, 768, 768, 8200, 128, 4, 0),
    (np.float16, 2560, 2048, 4100, 128, 4, 256),    # 320 tiles of 128 x 128: a whole one per CU, 64 on 4 ranges
])
def test_split_k_for_a_few_hundred_tiles(hip, oracle, dtype, M, N, K, tile, splits, whole):
    """Outputs of a few hundred small tiles and a long K: with a workspace the product runs on the tile shape that
    splits best, on the planned number of ranges.  Parity on sampled rows, a column checksum over the whole output
    against the product without a workspace, identical results from run to run, untouched padding."""
    f16 = dtype == np.float16
    A = synth.normal_half(M, K, 191) if f16 else synth.uniform_f32(M, K, 191)
    B = synth.normal_half(K, N, 192) if f16 else synth.uniform_f32(K, N, 192)
    esz = dtype().itemsize
    plan = hip.plan(esz, M, N, K)
    assert (plan.tile_m, plan.tile_n, plan.k_splits, plan.whole_tiles) == (tile, tile, splits, whole)
    need = hip.lib().decx_hip_gemm_workspace(esz, M, N, K)
    assert need == (-(-M // tile) * -(-N // tile) - whole) * splits * tile * tile * 4      # a slot per workgroup of a split tile
    ws = hip.DeviceMatrix(1, need // 4, np.float32)
    ws.upload_raw(np.full((1, ws.pitch), np.nan, np.float32))
    pa, pn = device_pitch(K, dtype), device_pitch(N, dtype)
    dA = hip.DeviceMatrix(M, K, dtype, pa, A, pad_value=np.nan); dB = hip.DeviceMatrix(K, N, dtype, pn, B, pad_value=np.nan)

    def product(workspace):
        dD = hip.DeviceMatrix(M, N, dtype, pn)
        dD.upload_raw(np.full((M, pn), -12345.0, dtype))
        hip.gemm(dA, dB, dD, workspace=workspace)
        hip.sync()
        raw = dD.download_raw()
        dD.free()
        assert np.all(raw[:, N:] == dtype(-12345.0))
        return raw[:, :N].copy()

    split = product(ws)
    rows = sample_rows(M, 48, 9)
    ref = (oracle.gemm_f16 if f16 else oracle.gemm_f32)(A, B, rows=rows)
    assert rel_err(split[rows], ref, K) <= (TOL_F16 if f16 else TOL_F32)
    assert np.array_equal(split.view(np.uint8), product(ws).view(np.uint8))
    whole = product(None)
    col_a = split.astype(np.float64).sum(axis=0); col_b = whole.astype(np.float64).sum(axis=0)
    assert np.max(np.abs(col_a - col_b)) <= (2e-2 if f16 else 1e-4) * np.max(np.abs(col_b))
    for d in (dA, dB, ws):
        d.free()


@pytest.mark.parametrize("dtype,M,N,K,whole", [(np.float32, 1000, 1500, 777, 256), (np.float32, 1536, 1400, 1000, 512), (np.float64, 1000, 1500, 777, 256),
                                              (np.float64, 1100, 1030, 2100, 256)])
def test_whole_tiles_that_share_their_cus_with_split_ones(hip, oracle, dtype, M, N, K, whole):
    """A few more tiles than a whole number per CU: the first ones of the grid stay whole and the others are cut along K
    so that all workgroups are resident together (the split ones at a raised wave priority where K is short).  Every
    form of the epilogue on both kinds of tile: A.B, alpha A.B + beta C and C aliased to D; all rows against the
    oracle, identical from run to run, padding untouched."""
    f64 = dtype == np.float64
    esz = 8 if f64 else 4
    plan = hip.plan(esz, M, N, K)
    assert plan.whole_tiles == whole and plan.k_splits > 1 and plan.grid == whole + (plan.grid - whole) // plan.k_splits * plan.k_splits
    rng = np.random.default_rng(77)
    A = rng.uniform(-1, 1, (M, K)).astype(dtype); B = rng.uniform(-1, 1, (K, N)).astype(dtype); C = rng.uniform(-1, 1, (M, N)).astype(dtype)
    need = hip.lib().decx_hip_gemm_workspace(esz, M, N, K)
    ws = hip.DeviceMatrix(1, need // 4, np.float32)
    ws.upload_raw(np.full((1, ws.pitch), np.nan, np.float32))
    pa, pn = device_pitch(K, dtype), device_pitch(N, dtype)
    dA = hip.DeviceMatrix(M, K, dtype, pa, A, pad_value=np.nan); dB = hip.DeviceMatrix(K, N, dtype, pn, B, pad_value=np.nan)
    dC = hip.DeviceMatrix(M, N, dtype, pn, C, pad_value=np.nan)
    rows = sample_rows(M, 96, 5)
    ref_ab = (oracle.gemm_f64 if f64 else oracle.gemm_f32)(A, B, rows=rows).astype(np.float64)
    tol = 1e-14 if f64 else TOL_F32

    def product(c, alpha, beta, alias=False):
        dD = hip.DeviceMatrix(M, N, dtype, pn)
        raw0 = np.full((M, pn), -12345.0, dtype)
        if alias:
            raw0[:, :N] = C
        dD.upload_raw(raw0)
        hip.gemm(dA, dB, dD, C=dD if alias else c, alpha=alpha, beta=beta, workspace=ws)
        hip.sync()
        raw = dD.download_raw()
        dD.free()
        assert np.all(raw[:, N:] == dtype(-12345.0))
        return raw[:, :N].copy()

    ab = product(None, 1.0, 1.0)
    assert rel_err(ab[rows], ref_ab, K) <= tol
    assert np.array_equal(ab.view(np.uint8), product(None, 1.0, 1.0).view(np.uint8))
    want = 0.5 * ref_ab - 2.0 * C[rows].astype(np.float64)
    for alias in (False, True):
        got = product(dC, 0.5, -2.0, alias)
        assert np.max(np.abs(got[rows].astype(np.float64) - want)) <= tol * np.sqrt(K) * np.max(np.abs(want)), alias
        # beyond the sampled rows: every element is alpha x (the product above) + beta x C, rounded once more at most
        full = 0.5 * ab.astype(np.float64) - 2.0 * C.astype(np.float64)
        assert np.max(np.abs(got.astype(np.float64) - full)) <= (1e-14 if f64 else 4e-6) * np.max(np.abs(full))
    for d in (dA, dB, dC, ws):
        d.free()


def test_f32_split_k_is_planned_only_where_it_pays(hip):
    L = hip.lib()
    assert L.decx_hip_gemm_f32_workspace(8192, 8192, 8192) == 0           # enough tiles
    assert L.decx_hip_gemm_f32_workspace(300, 300, 400) == 0              # K too short to cut
    assert L.decx_hip_gemm_f32_workspace(1024, 1024, 1024) == 0           # a tile per CU, K too short to pay for the exchange
    assert L.decx_hip_gemm_f32_workspace(1, 8192, 8192) == 0              # a row vector is dense already
    assert L.decx_hip_gemm_f32_workspace(0, 5, 5000) == 0


@pytest.mark.parametrize("dtype", [np.float32, np.float16])
@pytest.mark.parametrize("M,K", [(2048, 4096), (1030, 8200), (70, 16390), (3100, 3080)])
def test_column_operand_gathered_through_a_workspace(hip, oracle, dtype, M, K):
    """N = 1: B is the single column of a pitched K x 1 matrix.  With a workspace it is copied once into a dense
    vector in front of the matrix-vector kernel; the result is the one the strided path gives, bit for bit (same
    kernel, same order), and a workspace that is too small means the strided path."""
    f16 = dtype == np.float16
    A = synth.normal_half(M, K, 171) if f16 else synth.uniform_f32(M, K, 171)
    B = synth.normal_half(K, 1, 172) if f16 else synth.uniform_f32(K, 1, 172)
    C = synth.normal_half(M, 1, 173) if f16 else synth.uniform_f32(M, 1, 173)
    need = hip.lib().decx_hip_gemm_workspace(dtype().itemsize, M, 1, K)
    assert need >= K * dtype().itemsize and need % 16 == 0
    assert hip.lib().decx_hip_gemm_workspace(dtype().itemsize, 512, 1, 1024) == 0      # too small to pay
    ws = hip.DeviceMatrix(1, need // 4, np.float32)
    ws.upload_raw(np.full((1, ws.pitch), np.nan, np.float32))
    pa, p1 = device_pitch(K, dtype), device_pitch(1, dtype)
    ref = oracle.gemm_f16 if f16 else oracle.gemm_f32
    tol = TOL_F16 if f16 else TOL_F32

    def product(c, alpha, beta, workspace):
        dA = hip.DeviceMatrix(M, K, dtype, pa, A, pad_value=np.nan); dB = hip.DeviceMatrix(K, 1, dtype, p1, B, pad_value=np.nan)
        dC = hip.DeviceMatrix(M, 1, dtype, p1, c, pad_value=np.nan) if c is not None else None
        dD = hip.DeviceMatrix(M, 1, dtype, p1)
        dD.upload_raw(np.full((M, p1), -12345.0, dtype))
        hip.gemm(dA, dB, dD, dC, alpha, beta, workspace=workspace)
        hip.sync()
        raw = dD.download_raw()
        for d in (dA, dB, dC, dD):
            if d is not None:
                d.free()
        assert np.all(raw[:, 1:] == dtype(-12345.0))
        return raw[:, :1].copy()

    gathered = product(None, 1.0, 1.0, ws)
    assert rel_err(gathered, ref(A, B), K) <= tol
    strided = product(None, 1.0, 1.0, None)
    assert np.array_equal(gathered.view(np.uint8), strided.view(np.uint8))
    assert rel_err(product(C, 1.5, -0.5, ws), ref(A, B, C, 1.5, -0.5), K) <= tol
    small = hip.DeviceMatrix(1, 64, np.float32)
    assert np.array_equal(product(None, 1.0, 1.0, small).view(np.uint8), strided.view(np.uint8))
    for d in (ws, small):
        d.free()


@pytest.mark.parametrize("dtype", [np.float32, np.float16])
@pytest.mark.parametrize("K,N", [(8192, 2048), (20000, 70), (16500, 7), (33000, 513)])
def test_row_operand_few_columns_split_through_a_workspace(hip, oracle, dtype, K, N):
    """M = 1 with few columns and a long K: with a workspace, ranges of K go to workgroups of their own and the last
    workgroup of a column group to finish adds their partial sums in range order.  Parity, identical results from run to run,
    C / alpha / beta, untouched padding; a workspace that is too small means the single-kernel path."""
    f16 = dtype == np.float16
    A = synth.normal_half(1, K, 181) if f16 else synth.uniform_f32(1, K, 181)
    B = synth.normal_half(K, N, 182) if f16 else synth.uniform_f32(K, N, 182)
    C = synth.normal_half(1, N, 183) if f16 else synth.uniform_f32(1, N, 183)
    need = hip.lib().decx_hip_gemm_workspace(dtype().itemsize, 1, N, K)
    assert need > 0 and need % 16 == 0
    assert hip.plan(dtype().itemsize, 1, N, K).k_splits > 1
    assert hip.lib().decx_hip_gemm_workspace(dtype().itemsize, 1, 512, 8192) == 0       # too little to share out
    assert hip.lib().decx_hip_gemm_workspace(4, 1, 8192, 8192) == 0                     # fp32: a column group per CU already
    ws = hip.DeviceMatrix(1, need // 4, np.float32)
    ws.upload_raw(np.full((1, ws.pitch), np.nan, np.float32))
    pk, pn = device_pitch(K, dtype), device_pitch(N, dtype)
    ref = oracle.gemm_f16 if f16 else oracle.gemm_f32
    tol = TOL_F16 if f16 else TOL_F32

    def product(c, alpha, beta, workspace):
        dA = hip.DeviceMatrix(1, K, dtype, pk, A, pad_value=np.nan); dB = hip.DeviceMatrix(K, N, dtype, pn, B, pad_value=np.nan)
        dC = hip.DeviceMatrix(1, N, dtype, pn, c, pad_value=np.nan) if c is not None else None
        dD = hip.DeviceMatrix(1, N, dtype, pn)
        dD.upload_raw(np.full((1, pn), -12345.0, dtype))
        hip.gemm(dA, dB, dD, dC, alpha, beta, workspace=workspace)
        hip.sync()
        raw = dD.download_raw()
        for d in (dA, dB, dC, dD):
            if d is not None:
                d.free()
        assert np.all(raw[:, N:] == dtype(-12345.0))
        return raw[:, :N].copy()

    first = product(None, 1.0, 1.0, ws)
    assert rel_err(first, ref(A, B), K) <= tol
    assert np.array_equal(first.view(np.uint8), product(None, 1.0, 1.0, ws).view(np.uint8))      # fixed summation order
    assert rel_err(product(C, 1.5, -0.5, ws), ref(A, B, C, 1.5, -0.5), K) <= tol
    plain = product(None, 1.0, 1.0, None)
    assert rel_err(plain, ref(A, B), K) <= tol
    small = hip.DeviceMatrix(1, 64, np.float32)
    assert np.array_equal(product(None, 1.0, 1.0, small).view(np.uint8), plain.view(np.uint8))
    for d in (ws, small):
        d.free()


@pytest.mark.parametrize("tile", [0, 1, 2])
def test_forced_edge_variant_equals_fast_variant(hip, tile):
    """On tile-multiple shapes the predicated kernel and the unpredicated one run the same
    arithmetic in the same order: bit-identical."""
    M, N, K = 512, 512, 256
    A = synth.uniform_f32(M, K, 131); B = synth.uniform_f32(K, N, 132)
    assert np.array_equal(run(hip, A, B, tile=tile), run(hip, A, B, tile=tile, force_edge=True))
    Ah = synth.normal_half(M, K, 133); Bh = synth.normal_half(K, N, 134)
    assert np.array_equal(run(hip, Ah, Bh, tile=tile).view(np.uint16),
                          run(hip, Ah, Bh, tile=tile, force_edge=True).view(np.uint16))


@pytest.mark.parametrize("dtype", [np.float32, np.float16])
def test_exact_closed_forms(hip, dtype):
    n = 200
    rng = np.random.default_rng(5)
    X = rng.integers(-8, 9, (n, 150)).astype(dtype)
    eye = np.eye(n, dtype=dtype)
    assert np.array_equal(run(hip, eye, X), X)                       # I . X == X, bit for bit
    Y = rng.integers(-8, 9, (150, n)).astype(dtype)
    assert np.array_equal(run(hip, Y, eye), Y)
    K = 1000                                                         # ones . ones == K (K < 2^11 for half)
    assert np.all(run(hip, np.ones((9, K), dtype), np.ones((K, 11), dtype)) == dtype(K))
    a = rng.integers(-3, 4, (130, 96)).astype(dtype); b = rng.integers(-3, 4, (96, 140)).astype(dtype)
    assert np.array_equal(run(hip, a, b), (a.astype(np.int64) @ b.astype(np.int64)).astype(dtype))


def test_reference_sample_known_answer(hip):
    """samples/Matrix_Multiplication/MatMul.cpp:16-40 with W=1013, H=1077, L=1005."""
    W, H, L = 1013, 1077, 1005
    A = np.tile(np.arange(L, dtype=np.float32), (H, 1))
    B = np.tile(np.arange(L, dtype=np.float32)[:, None], (1, W))
    got = run(hip, A, B)
    assert np.max(np.abs(got.astype(np.float64) - 337853530.0)) / 337853530.0 < 4e-6


def test_linearity_at_full_size(hip):
    """(A1 + A2) . B == A1 . B + A2 . B up to rounding, at the fp32 headline size's tile shape."""
    M = N = 2048; K = 1024
    A1 = synth.uniform_f32(M, K, 141); A2 = synth.uniform_f32(M, K, 142); B = synth.uniform_f32(K, N, 143)
    lhs = run(hip, A1 + A2, B)
    rhs = run(hip, A1, B).astype(np.float64) + run(hip, A2, B).astype(np.float64)
    assert np.max(np.abs(lhs - rhs)) / (np.max(np.abs(rhs)) * np.sqrt(K)) <= TOL_F32


def test_c_may_alias_d(hip, oracle):
    M, N, K = 100, 150, 77
    A = synth.uniform_f32(M, K, 151); B = synth.uniform_f32(K, N, 152); C = synth.uniform_f32(M, N, 153)
    dA = hip.DeviceMatrix(M, K, np.float32, data=A); dB = hip.DeviceMatrix(K, N, np.float32, data=B)
    dD = hip.DeviceMatrix(M, N, np.float32, data=C)
    hip.gemm(dA, dB, dD, dD, 1.0, 1.0)
    hip.sync()
    assert rel_err(dD.download(), oracle.gemm_f32(A, B, C, 1.0, 1.0), K) <= TOL_F32


@pytest.mark.parametrize("dtype,tile", [(d, t) for d in (np.float32, np.float16, np.float64) for t in (0, 1, 2)] +
                         [(np.float16, t) for t in (3, 4, 5)])
def test_c_term_on_interior_and_edge_tiles_of_every_tile(hip, oracle, dtype, tile):
    """alpha A.B + beta C on an output that holds interior tiles, tiles on the right and lower edges and the corner tile of
    every tile class, with C apart from D and with C = D (the epilogues ask for the C values of several rows ahead of
    their use; every element is read before it is overwritten)."""
    M, N, K = 650, 420, 130
    f64 = dtype == np.float64
    rng = np.random.default_rng(4242 + tile)
    A = rng.uniform(-1, 1, (M, K)).astype(dtype); B = rng.uniform(-1, 1, (K, N)).astype(dtype); C = rng.uniform(-1, 1, (M, N)).astype(dtype)
    ref = {np.float32: oracle.gemm_f32, np.float16: oracle.gemm_f16, np.float64: oracle.gemm_f64}[dtype](A, B, C, 0.75, -1.25)
    tol = {np.float32: TOL_F32, np.float16: TOL_F16, np.float64: 1e-14}[dtype]
    pk, pn = device_pitch(K, dtype), device_pitch(N, dtype)
    dA = hip.DeviceMatrix(M, K, dtype, pk, A, pad_value=np.nan); dB = hip.DeviceMatrix(K, N, dtype, pn, B, pad_value=np.nan)
    dC = hip.DeviceMatrix(M, N, dtype, pn, C, pad_value=np.nan)
    for alias in (False, True):
        dD = hip.DeviceMatrix(M, N, dtype, pn)
        raw0 = np.full((M, pn), -12345.0, dtype)
        if alias:
            raw0[:, :N] = C
        dD.upload_raw(raw0)
        hip.gemm(dA, dB, dD, dD if alias else dC, 0.75, -1.25, tile=tile)
        hip.sync()
        raw = dD.download_raw()
        dD.free()
        assert np.all(raw[:, N:] == dtype(-12345.0)), "padding columns of D were written"
        assert rel_err(raw[:, :N], ref, K) <= tol, alias
    for d in (dA, dB, dC):
        d.free()


def test_empty_and_invalid_arguments(hip):
    L = hip.lib()
    d = hip.DeviceMatrix(4, 4, np.float32, data=np.ones((4, 4), np.float32))
    p = d.ptr
    assert L.decx_hip_gemm_f32(p, p, None, p, 0, 4, 4, 4, 4, 0, 4, 1.0, 1.0, None) == 0      # empty: nothing to do
    assert L.decx_hip_gemm_f32(p, p, None, p, 4, 0, 4, 4, 4, 0, 4, 1.0, 1.0, None) == 0
    assert L.decx_hip_gemm_f32(None, p, None, p, 4, 4, 4, 4, 4, 0, 4, 1.0, 1.0, None) == -1   # null operand
    assert L.decx_hip_gemm_f32(p, p, None, p, 4, 4, 4, 3, 4, 0, 4, 1.0, 1.0, None) == -1      # lda < K
    assert L.decx_hip_gemm_f32(p, p, p, p, 4, 4, 4, 4, 4, 3, 4, 1.0, 1.0, None) == -1         # ldc < N
    assert L.decx_hip_gemm_f32_tile(p, p, None, p, 4, 4, 4, 4, 4, 0, 4, 1.0, 1.0, None, 9, 0) == -1
    hip.sync()
    assert np.all(d.download() == 1.0)
    # K == 0: the product is empty, D = 0 (or beta * C)
    out = hip.DeviceMatrix(4, 4, np.float32, data=np.full((4, 4), 7, np.float32))
    assert L.decx_hip_gemm_f32(p, p, None, out.ptr, 4, 4, 0, 4, 4, 0, 4, 1.0, 1.0, None) == 0
    hip.sync()
    assert np.all(out.download() == 0.0)
    assert L.decx_hip_gemm_f32(p, p, d.ptr, out.ptr, 4, 4, 0, 4, 4, 4, 4, 1.0, 3.0, None) == 0
    hip.sync()
    assert np.all(out.download() == 3.0)


def test_stream_and_events(hip):
    import ctypes
    L = hip.lib()
    s = ctypes.c_void_p()
    assert L.decx_hip_stream_create(ctypes.byref(s)) == 0
    A = synth.uniform_f32(256, 256, 161)
    dA = hip.DeviceMatrix(256, 256, np.float32, data=A)
    dI = hip.DeviceMatrix(256, 256, np.float32, data=np.eye(256, dtype=np.float32))
    dD = hip.DeviceMatrix(256, 256, np.float32)
    t = hip.Timer()
    t.start(s)
    hip.gemm(dA, dI, dD, stream=s)
    ms = t.stop(s)
    hip.sync(s)
    assert ms > 0 and np.array_equal(dD.download(), A)
    assert L.decx_hip_stream_destroy(s) == 0


@pytest.mark.parametrize("dtype,M,N,K", [
    (np.float32, 300, 300, 8192), (np.float32, 1280, 1024, 8192), (np.float32, 1000, 1500, 777),
    (np.float16, 300, 300, 8192), (np.float16, 1280, 1024, 6144), (np.float16, 640, 640, 8192),
    (np.float64, 300, 300, 8192), (np.float64, 1280, 1024, 2048),
    # more than 8 ranges: groups of four are added first, then the group sums
    (np.float32, 100, 120, 20000), (np.float16, 128, 128, 16384), (np.float16, 70, 130, 40000), (np.float64, 100, 120, 4096),
    # more tiles than fit the chip at once: the full rounds stay whole, the tiles of the ragged last round are split
    (np.float32, 2112, 2112, 1024), (np.float64, 1536, 1400, 1536),
])
def test_split_k_slots_carry_nothing_from_launch_to_launch(hip, oracle, dtype, M, N, K):
    """The workgroups of a tile meet in the workspace (slots written and read at device scope, a counter per tile
    that ends every launch at zero).  Two input sets take turns on the same workspace: a slot, a cache line or a
    counter left over from the launch before would show as a result that differs from the set's first one."""
    esz = np.dtype(dtype).itemsize
    need = hip.lib().decx_hip_gemm_workspace(esz, M, N, K)
    if need == 0 or hip.plan(esz, M, N, K).k_splits < 2:
        pytest.skip("the planner does not split this shape")
    if K >= 16384 or (M, N) == (100, 120):
        assert hip.plan(esz, M, N, K).k_splits > 8
    if M >= 1536:
        plan = hip.plan(esz, M, N, K)
        assert plan.whole_tiles > 0 and plan.grid == plan.whole_tiles + (-(-M // 64) * -(-N // 64) - plan.whole_tiles) * plan.k_splits
    ws = hip.DeviceMatrix(1, need // 4, np.float32)
    pa, pn = device_pitch(K, dtype), device_pitch(N, dtype)
    make = {2: synth.normal_half, 4: synth.uniform_f32, 8: synth.uniform_f64}[esz]
    ref = {2: oracle.gemm_f16, 4: oracle.gemm_f32, 8: oracle.gemm_f64}[esz]
    tol = {2: TOL_F16, 4: TOL_F32, 8: 1e-14}[esz]
    bits = {2: np.uint16, 4: np.uint32, 8: np.uint64}[esz]
    sets = []
    for s in range(2):
        A = make(M, K, 700 + s); B = make(K, N, 710 + s)
        sets.append((A, B, hip.DeviceMatrix(M, K, dtype, pa, A), hip.DeviceMatrix(K, N, dtype, pn, B)))
    dD = hip.DeviceMatrix(M, N, dtype, pn)
    first = [None, None]
    for it in range(60):
        A, B, dA, dB = sets[it % 2]
        hip.gemm(dA, dB, dD, workspace=ws)
        if it % 2 == 1 or it < 2 or it % 7 == 0:             # most launches follow each other without a host round trip
            hip.sync()
            got = dD.download()
            if first[it % 2] is None:
                first[it % 2] = got
                rows = np.arange(0, M, max(1, M // 24), dtype=np.uint32)
                assert rel_err(got[rows], ref(A, B, rows=rows), K) <= tol
            else:
                assert np.array_equal(got.view(bits), first[it % 2].view(bits)), "launch %d" % it
    for d in [ws, dD] + [x for t in sets for x in t[2:]]:
        d.free()


@pytest.mark.parametrize("dtype,M,N,K", [(np.float32, 1000, 1500, 777), (np.float16, 640, 640, 8192), (np.float64, 1536, 1400, 1536)])
def test_split_k_on_two_streams_at_once(hip, oracle, dtype, M, N, K):
    """Every launch takes its own window of tile counters, so products that split K may run side by side on two streams
    (each with a workspace of its own): the results are those of the same products run alone, bit for bit."""
    import ctypes
    esz = np.dtype(dtype).itemsize
    need = hip.lib().decx_hip_gemm_workspace(esz, M, N, K)
    if need == 0 or hip.plan(esz, M, N, K).k_splits < 2:
        pytest.skip("the planner does not split this shape")
    L = hip.lib()
    pa, pn = device_pitch(K, dtype), device_pitch(N, dtype)
    make = {2: synth.normal_half, 4: synth.uniform_f32, 8: synth.uniform_f64}[esz]
    bits = {2: np.uint16, 4: np.uint32, 8: np.uint64}[esz]
    lanes = []
    for s in range(2):
        st = ctypes.c_void_p()
        assert L.decx_hip_stream_create(ctypes.byref(st)) == 0
        A = make(M, K, 900 + s); B = make(K, N, 910 + s)
        lanes.append(dict(stream=st, A=hip.DeviceMatrix(M, K, dtype, pa, A), B=hip.DeviceMatrix(K, N, dtype, pn, B),
                          D=hip.DeviceMatrix(M, N, dtype, pn), ws=hip.DeviceMatrix(1, need // 4, np.float32)))
    alone = []
    for ln in lanes:                                          # one after the other, on the default stream
        hip.gemm(ln["A"], ln["B"], ln["D"], workspace=ln["ws"])
        hip.sync()
        alone.append(ln["D"].download())
    for rep in range(5):
        for ln in lanes:
            ln["D"].upload_raw(np.full((M, pn), 3, dtype))
        for it in range(12):                                  # launches of the two streams interleave on the chip
            for ln in lanes:
                hip.gemm(ln["A"], ln["B"], ln["D"], workspace=ln["ws"], stream=ln["stream"])
        for ln, want in zip(lanes, alone):
            hip.sync(ln["stream"])
            assert np.array_equal(ln["D"].download().view(bits), want.view(bits)), "repetition %d" % rep
    for ln in lanes:
        assert L.decx_hip_stream_destroy(ln["stream"]) == 0
        for k in ("A", "B", "D", "ws"):
            ln[k].free()


@pytest.mark.parametrize("M,N,K,tile_m,tile_n", [(3000, 3000, 3000, 192, 192), (8192, 4608, 256, 256, 192), (4608, 4608, 512, 192, 256)])
def test_f16_tiles_between_the_two_largest_are_planned_and_right(hip, oracle, M, N, K, tile_m, tile_n):
    """Outputs that 256 x 256 tiles cut into an awkward number of pieces for the CUs take a tile of 192 rows or columns:
    the plan says so, the result holds on sampled rows (first and last tile rows included), bit-equal to the forced
    tile, and a column checksum covers every element."""
    p = hip.plan(2, M, N, K)
    assert (p.tile_m, p.tile_n) == (tile_m, tile_n) and p.k_splits == 1
    A = synth.normal_half(M, K, 171); B = synth.normal_half(K, N, 172)
    got = run(hip, A, B)
    rows = np.unique(np.concatenate([[0, 1, tile_m - 1, tile_m, M - 2, M - 1], sample_rows(M, 40, 9)])).astype(np.uint32)
    assert rel_err(got[rows], oracle.gemm_f16(A, B, rows=rows), K) <= TOL_F16
    # ones . (A B) = (ones . A) B in float64, against the sum of the rounded outputs: rounding errors average out
    want = (A.astype(np.float64).sum(axis=0) @ B.astype(np.float64))
    have = got.astype(np.float64).sum(axis=0)
    assert float(np.max(np.abs(have - want))) <= 2e-3 * float(np.max(np.abs(want))) + 0.05 * np.sqrt(M)
    forced = {(192, 192): 3, (192, 256): 4, (256, 192): 5}[(tile_m, tile_n)]
    assert np.array_equal(run(hip, A, B, tile=forced).view(np.uint16), got.view(np.uint16))


@pytest.mark.parametrize("M,N,K,with_c", [(4300, 4352, 3000, False), (4352, 4352, 4096, True)])
def test_f16_last_round_of_the_largest_tiles_split_along_k(hip, oracle, M, N, K, with_c):
    """More 256 x 256 tiles than CUs: the full rounds stay whole, the few tiles of the last round are cut along K and
    summed in range order inside the launch.  The plan says so; sampled rows (from whole and from split tiles) hold
    against the oracle, a column checksum covers every element, two runs agree bit for bit, D's padding stays."""
    p = hip.plan(2, M, N, K)
    tiles = -(-M // 256) * -(-N // 256)
    assert (p.tile_m, p.tile_n) == (256, 256) and p.k_splits > 1 and p.whole_tiles == tiles // 256 * 256
    assert p.grid == p.whole_tiles + (tiles - p.whole_tiles) * p.k_splits
    need = hip.lib().decx_hip_gemm_workspace(2, M, N, K)
    assert need == (tiles - p.whole_tiles) * p.k_splits * 256 * 256 * 4
    A = synth.normal_half(M, K, 181); B = synth.normal_half(K, N, 182)
    C = synth.normal_half(M, N, 183) if with_c else None
    pk, pn = device_pitch(K, np.float16), device_pitch(N, np.float16)
    dA = hip.DeviceMatrix(M, K, np.float16, pk, A, pad_value=np.nan); dB = hip.DeviceMatrix(K, N, np.float16, pn, B, pad_value=np.nan)
    dC = hip.DeviceMatrix(M, N, np.float16, pn, C, pad_value=np.nan) if with_c else None
    ws = hip.DeviceMatrix(1, need // 4, np.float32)
    ws.upload_raw(np.full((1, ws.pitch), np.nan, np.float32))
    outs = []
    for _ in range(2):
        dD = hip.DeviceMatrix(M, N, np.float16, pn)
        dD.upload_raw(np.full((M, pn), -12345.0, np.float16))
        hip.gemm(dA, dB, dD, dC, 0.5 if with_c else 1.0, -2.0 if with_c else 1.0, workspace=ws)
        hip.sync()
        raw = dD.download_raw()
        assert np.all(raw[:, N:] == np.float16(-12345.0))
        outs.append(raw[:, :N].copy())
        dD.free()
    assert np.array_equal(outs[0].view(np.uint16), outs[1].view(np.uint16))
    got = outs[0]
    rows = np.unique(np.concatenate([[0, 255, 256, M - 257, M - 256, M - 2, M - 1], sample_rows(M, 40, 19)])).astype(np.uint32)
    ref = oracle.gemm_f16(A, B, C, 0.5, -2.0, rows=rows) if with_c else oracle.gemm_f16(A, B, rows=rows)
    assert rel_err(got[rows], ref, K) <= TOL_F16
    want = A.astype(np.float64).sum(axis=0) @ B.astype(np.float64)
    if with_c:
        want = 0.5 * want - 2.0 * C.astype(np.float64).sum(axis=0)
    have = got.astype(np.float64).sum(axis=0)
    assert float(np.max(np.abs(have - want))) <= 2e-3 * float(np.max(np.abs(want))) + 0.05 * np.sqrt(M)
    for d in (dA, dB, dC, ws):
        if d is not None:
            d.free()
