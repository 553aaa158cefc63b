"""Seeded random shapes through the planner's own picks (with a workspace, so that split plans run too): every product
against the CPU oracle on sampled rows, pitch padding untouched, a second run bit-equal to the first.  The shape
classes are drawn so that the plans the fixed-shape tests name one by one all come up here as the planner meets them:
fp16 tiles of 192 rows or columns, the last round of the largest fp16 tiles split along K, whole tiles in front of
split ones, two-level sums."""
import numpy as np
import pytest

from decx_amd import synth

pytestmark = pytest.mark.gpu

BAR = {2: 2e-3, 4: 1e-5, 8: 1e-14}
SAMPLED_ROWS = 16


@pytest.fixture(scope="module")
def hip():
    from decx_amd import hip as h
    h.init()
    return h


def draw_shape(rng, cls):
    r = lambda lo, hi: int(rng.integers(lo, hi))
    if cls == 0:
        return 2, r(4100, 6200), r(4100, 6200), r(800, 4500)        # more 256 x 256 fp16 tiles than CUs
    if cls == 1:
        return 2, r(1500, 4200), r(1500, 4200), r(64, 3000)         # fp16 tiles between the two largest
    if cls == 2:
        return 2, r(100, 2500), r(100, 2500), r(32, 9000)
    if cls == 3:
        return 2, r(2000, 9000), r(150, 800), r(200, 6000)
    if cls == 4:
        return 4, r(300, 3500), r(300, 3500), r(100, 5000)
    return 8, r(300, 2500), r(300, 2500), r(100, 4000)


def make(dt, rows, cols, seed):
    if dt == np.float16:
        return synth.normal_half(rows, cols, seed)
    return synth.uniform_f32(rows, cols, seed) if dt == np.float32 else synth.uniform_f64(rows, cols, seed)


def test_planner_picks_on_random_shapes_match_the_oracle(hip, oracle):
    rng = np.random.default_rng(0x5EED)
    plans = set()
    for case in range(60):
        esz, M, N, K = draw_shape(rng, case % 6)
        if rng.random() < 0.5:
            M, N = N, M
        dt = {2: np.float16, 4: np.float32, 8: np.float64}[esz]
        per16 = 16 // esz
        pitch = lambda c: (c + int(rng.integers(0, 40)) + per16 - 1) // per16 * per16
        with_c = bool(rng.random() < 0.5)
        alpha, beta = (float(rng.uniform(-2, 2)), float(rng.uniform(-2, 2))) if with_c else (1.0, 1.0)
        if esz == 2:                                             # the scalars travel as halves through the public API; here as given
            alpha, beta = float(np.float32(alpha)), float(np.float32(beta))
        A = make(dt, M, K, 0x9000 + 3 * case); B = make(dt, K, N, 0x9001 + 3 * case)
        C = make(dt, M, N, 0x9002 + 3 * case) if with_c else None
        dA = hip.DeviceMatrix(M, K, dt, pitch(K), A, pad_value=np.nan)
        dB = hip.DeviceMatrix(K, N, dt, pitch(N), B, pad_value=np.nan)
        dC = hip.DeviceMatrix(M, N, dt, pitch(N), C, pad_value=np.nan) if with_c else None
        pd = pitch(N)
        dD = hip.DeviceMatrix(M, N, dt, pd)
        need = int(hip.lib().decx_hip_gemm_workspace(esz, M, N, K))
        ws = hip.DeviceMatrix(1, max(need // 4, 4), np.float32)
        ws.upload_raw(np.full((1, ws.pitch), np.nan, np.float32))
        p = hip.plan(esz, M, N, K)
        plans.add((esz, p.tile_m, p.tile_n, p.k_splits > 1, p.k_splits > 8, p.whole_tiles > 0))
        print("case", case, np.dtype(dt).name, (M, N, K), "C" if with_c else "-", "plan", (p.tile_m, p.tile_n), p.k_splits,
              p.whole_tiles, flush=True)
        runs = []
        for _ in range(2):
            dD.upload_raw(np.full((M, pd), -7.0, dt))
            hip.gemm(dA, dB, dD, dC, alpha, beta, workspace=ws)
            hip.sync()
            runs.append(dD.download_raw())
        raw = runs[0]
        assert np.array_equal(runs[0].view(np.uint8), runs[1].view(np.uint8)), "two runs of one product differ"
        assert np.all(raw[:, N:] == dt(-7.0)), "padding columns of D were written"
        rows = np.sort(rng.choice(M, min(M, SAMPLED_ROWS), replace=False)).astype(np.uint32)
        fn = {2: oracle.gemm_f16, 4: oracle.gemm_f32, 8: oracle.gemm_f64}[esz]
        ref = (fn(A, B, C, alpha, beta, rows=rows) if with_c else fn(A, B, rows=rows)).astype(np.float64)
        got = raw[rows, :N].astype(np.float64)
        assert not np.isnan(got).any()
        err = float(np.max(np.abs(got - ref))) / (max(float(np.max(np.abs(ref))), 1e-30) * np.sqrt(K))
        assert err <= BAR[esz], (case, M, N, K, err)
        for d in (dA, dB, dC, dD, ws):
            if d is not None:
                d.free()
    kinds = {(e, tm, tn) for e, tm, tn, *_ in plans}
    assert {(2, 256, 256), (2, 128, 128), (4, 64, 64), (8, 64, 64)} <= kinds, kinds
    assert any(e == 2 and (tm, tn) in ((192, 192), (192, 256), (256, 192)) for e, tm, tn in kinds), kinds
    assert any(e == 2 and tm == 256 and split and whole for e, tm, tn, split, two, whole in plans), plans     # last round split
    assert any(split and whole for e, tm, tn, split, two, whole in plans if e == 4), plans
    assert any(split for e, tm, tn, split, two, whole in plans if e == 8), plans
