"""decx_hip_gemm_f32_static (the entry point that allocates nothing: its split-K / gather workspace is a device array
inside the library) against decx_hip_gemm_f32_ws with a caller-allocated workspace, through the C ABI, bit for bit.

The static array keeps what the previous call left in it, so the cases run back to back, largest first: a call
that relied on a cleared workspace, or read beyond what it wrote itself, would pick up the bigger product's
partial sums.  The ws result itself is checked against the CPU oracle."""
import ctypes

import numpy as np
import pytest

from decx_amd import synth

pytestmark = pytest.mark.gpu

STATIC_BYTES = 16 << 20          # DECX_HIP_STATIC_WORKSPACE_BYTES
E_TOO_LARGE = -4


@pytest.fixture(scope="module")
def hip():
    from decx_amd import hip as h
    h.init()
    return h


def pitch32(cols):
    return (cols + 31) // 32 * 32


def both(hip, M, N, K, seed, with_c, alpha=1.0, beta=1.0, offset_a=0):
    """(result of _static, result of _ws, host A, B, C) on NaN-padded device matrices of the reference's pitches.
    Device memory the runtime reports free must be the same before and after the _static call (its second one: see below)."""
    L = hip.lib()
    A = synth.uniform_f32(M, K, seed); B = synth.uniform_f32(K, N, seed + 1)
    C = synth.uniform_f32(M, N, seed + 2) if with_c else None
    dA = hip.DeviceMatrix(M, K, np.float32, pitch32(K), A, pad_value=np.nan, offset_elems=offset_a)
    dB = hip.DeviceMatrix(K, N, np.float32, pitch32(N), B, pad_value=np.nan)
    dC = hip.DeviceMatrix(M, N, np.float32, pitch32(N), C, pad_value=np.nan) if with_c else None
    need = L.decx_hip_gemm_f32_workspace(M, N, K)
    ws = hip.DeviceMatrix(1, max(need // 4, 4), np.float32)
    outs = []
    for static in (True, False):
        dD = hip.DeviceMatrix(M, N, np.float32, pitch32(N))
        dD.upload_raw(np.full((M, pitch32(N)), -777.0, np.float32))
        args = [dA.ptr, dB.ptr, dC.ptr if with_c else None, dD.ptr, M, N, K, dA.pitch, dB.pitch,
                dC.pitch if with_c else 0, dD.pitch, alpha, beta]
        print("no-alloc case", (M, N, K), "C" if with_c else "-", "static" if static else "ws", "need", need, flush=True)
        if static:
            # The first launch of a kernel in a process lets the runtime load its code, for which it may take device
            # memory of its own: one call in front, then the call that is held to "free memory unchanged".
            hip.check(L.decx_hip_gemm_f32_static(*args, None), "gemm")
            hip.sync()
            dD.upload_raw(np.full((M, pitch32(N)), -777.0, np.float32))
            hip.sync()
            free_before = hip.mem_free_bytes()
            rc = L.decx_hip_gemm_f32_static(*args, None)
            hip.sync()
            assert hip.mem_free_bytes() == free_before, "the call changed the amount of free device memory"
        else:
            rc = L.decx_hip_gemm_f32_ws(*args, ws.ptr, need, None)
        hip.check(rc, "gemm")
        hip.sync()
        raw = dD.download_raw()
        assert np.all(raw[:, N:] == np.float32(-777.0)), "padding columns of D were written"
        outs.append(raw[:, :N].copy())
        dD.free()
    for d in (dA, dB, dC, ws):
        if d is not None:
            d.free()
    return outs[0], outs[1], A, B, C, need


def test_static_workspace_matches_the_allocated_one_call_after_call(hip, oracle):
    # (M, N, K, C term): split K over 5, 10, 16 ranges, then the dense copy of a pitched x, then a product that needs
    # no workspace at all.  Each smaller than the one before, so stale partial sums of the bigger call lie beyond.
    cases = [(640, 640, 8192, True), (300, 300, 8192, False), (100, 120, 4096, True), (8192, 1, 8192, False),
             (200, 136, 120, True)]
    used_split = 0
    for i, (M, N, K, with_c) in enumerate(cases):
        got, want, A, B, C, need = both(hip, M, N, K, 0x5700 + 16 * i, with_c, alpha=0.75 if with_c else 1.0,
                                        beta=-1.25 if with_c else 1.0)
        assert need <= STATIC_BYTES
        used_split += hip.plan(4, M, N, K).k_splits > 1
        assert not np.isnan(want).any()
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), (M, N, K)
        if M * N * K <= 300 * 300 * 8192:                       # the ws path itself against the oracle
            ref = oracle.gemm_f32(A, B, C, 0.75, -1.25) if with_c else oracle.gemm_f32(A, B)
            err = float(np.max(np.abs(got.astype(np.float64) - ref))) / (float(np.max(np.abs(ref))) * np.sqrt(K))
            assert err <= 1e-5, err
    assert used_split >= 3                                      # the cases do go through the workspace


def test_static_workspace_rejects_what_does_not_fit(hip):
    L = hip.lib()
    M, N, K = 480, 864, 4096                                    # 112 tiles on 16 ranges: 28 MiB of partial products
    need = L.decx_hip_gemm_f32_workspace(M, N, K)
    assert need > STATIC_BYTES, "pick another shape: this one fits the static workspace now"
    dA = hip.DeviceMatrix(M, K, np.float32, K, synth.uniform_f32(M, K, 1))
    dB = hip.DeviceMatrix(K, N, np.float32, N, synth.uniform_f32(K, N, 2))
    dD = hip.DeviceMatrix(M, N, np.float32, N)
    dD.upload_raw(np.full((M, N), 3.5, np.float32))
    rc = L.decx_hip_gemm_f32_static(dA.ptr, dB.ptr, None, dD.ptr, M, N, K, K, N, 0, N, 1.0, 1.0, None)
    hip.sync()
    assert rc == E_TOO_LARGE
    assert b"workspace" in L.decx_hip_error_string(rc)
    assert np.all(dD.download_raw() == np.float32(3.5)), "a rejected call must launch nothing"
    for d in (dA, dB, dD):
        d.free()


def test_static_workspace_takes_what_the_workspace_form_would_not_split(hip, oracle):
    """Operands the workspace form would not split (a base that is not 16-byte aligned: the register-staged kernel
    runs) are no business of the static array, however much the shape's query says: not refused, same bits."""
    M, N, K = 480, 864, 4096
    assert hip.lib().decx_hip_gemm_f32_workspace(M, N, K) > STATIC_BYTES
    got, want, A, B, _, _ = both(hip, M, N, K, 0x5800, False, offset_a=1)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    ref = oracle.gemm_f32(A, B, rows=np.arange(0, M, 37, dtype=np.uint32))
    err = float(np.max(np.abs(got[::37].astype(np.float64) - ref))) / (float(np.max(np.abs(ref))) * np.sqrt(K))
    assert err <= 1e-5, err


def test_static_workspace_reads_a_long_column_in_place(hip):
    """N == 1 with a column longer than the static array holds: the workspace form copies it into a dense vector
    first, the static one reads it where it lies; the sums are the same."""
    M, K = 64, (STATIC_BYTES // 4) + 4096
    assert hip.lib().decx_hip_gemm_f32_workspace(M, 1, K) > STATIC_BYTES
    got, want, A, B, _, _ = both(hip, M, 1, K, 0x5820, False)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    ref = A.astype(np.float64) @ B.astype(np.float64)
    assert float(np.max(np.abs(got - ref))) / (float(np.max(np.abs(ref))) * np.sqrt(K)) <= 1e-5


def test_static_workspace_allocates_nothing_between_two_streams(hip):
    """Split launches from two streams carry events (a window goes to another stream only behind a completed one): they
    come from the pool decx_hip_init made, so the amount of free device memory does not move here either."""
    L = hip.lib()
    M, N, K = 300, 300, 8192
    A = synth.uniform_f32(M, K, 0x5900); B = synth.uniform_f32(K, N, 0x5901)
    dA = hip.DeviceMatrix(M, K, np.float32, pitch32(K), A); dB = hip.DeviceMatrix(K, N, np.float32, pitch32(N), B)
    dD1 = hip.DeviceMatrix(M, N, np.float32, pitch32(N)); dD2 = hip.DeviceMatrix(M, N, np.float32, pitch32(N))
    need = L.decx_hip_gemm_f32_workspace(M, N, K)
    ws = hip.DeviceMatrix(1, need // 4, np.float32)
    s1, s2 = hip.Stream(), hip.Stream()

    def round_of_two():
        hip.check(L.decx_hip_gemm_f32_ws(dA.ptr, dB.ptr, None, dD2.ptr, M, N, K, dA.pitch, dB.pitch, 0, dD2.pitch, 1.0, 1.0,
                                         ws.ptr, need, s2.handle), "gemm")
        hip.check(L.decx_hip_gemm_f32_static(dA.ptr, dB.ptr, None, dD1.ptr, M, N, K, dA.pitch, dB.pitch, 0, dD1.pitch, 1.0, 1.0,
                                             s1.handle), "gemm")

    round_of_two(); s1.sync(); s2.sync()
    want = dD1.download()
    assert np.array_equal(want.view(np.uint32), dD2.download().view(np.uint32))
    before = hip.split_counter_stats()
    free_before = hip.mem_free_bytes()
    print("no-alloc, two streams: 60 rounds", flush=True)
    for _ in range(60):
        round_of_two()
    s1.sync(); s2.sync()
    assert hip.mem_free_bytes() == free_before, "the calls changed the amount of free device memory"
    after = hip.split_counter_stats()
    assert after["events"] - before["events"] >= 100            # nearly every launch recorded one
    assert np.array_equal(dD1.download().view(np.uint32), want.view(np.uint32))
    assert np.array_equal(dD2.download().view(np.uint32), want.view(np.uint32))
    for s in (s1, s2):
        s.destroy()
    for d in (dA, dB, dD1, dD2, ws):
        d.free()
