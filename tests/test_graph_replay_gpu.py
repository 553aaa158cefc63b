"""Split products recorded into a HIP graph: every replay must give the bits of the same call made outside a graph,
with other split launches and host synchronisations between the replays.  A recorded split launch keeps a window of
the counter array that launches outside graphs never get (the upper half), so a replay meets its counters at zero
whenever it runs.  The graph calls themselves go to the HIP runtime the library is linked against."""
import ctypes

import numpy as np
import pytest

from decx_amd import synth

pytestmark = pytest.mark.gpu

CAPTURE_MODE_GLOBAL = 0


@pytest.fixture(scope="module")
def hip():
    from decx_amd import hip as h
    h.init()
    return h


@pytest.fixture(scope="module")
def runtime():
    rt = ctypes.CDLL("libamdhip64.so.7")
    vp = ctypes.c_void_p
    rt.hipStreamBeginCapture.argtypes = [vp, ctypes.c_int]
    rt.hipStreamEndCapture.argtypes = [vp, ctypes.POINTER(vp)]
    rt.hipGraphInstantiate.argtypes = [ctypes.POINTER(vp), vp, ctypes.POINTER(vp), ctypes.c_char_p, ctypes.c_size_t]
    rt.hipGraphLaunch.argtypes = [vp, vp]
    rt.hipGraphExecDestroy.argtypes = [vp]
    rt.hipGraphDestroy.argtypes = [vp]
    for f in (rt.hipStreamBeginCapture, rt.hipStreamEndCapture, rt.hipGraphInstantiate, rt.hipGraphLaunch,
              rt.hipGraphExecDestroy, rt.hipGraphDestroy):
        f.restype = ctypes.c_int
    return rt


def pitch32(cols):
    return (cols + 31) // 32 * 32


class Product:
    def __init__(self, hip, M, N, K, seed, with_c):
        self.hip, self.M, self.N, self.K = hip, M, N, K
        self.A = synth.uniform_f32(M, K, seed); self.B = synth.uniform_f32(K, N, seed + 1)
        self.C = synth.uniform_f32(M, N, seed + 2) if with_c else None
        self.dA = hip.DeviceMatrix(M, K, np.float32, pitch32(K), self.A)
        self.dB = hip.DeviceMatrix(K, N, np.float32, pitch32(N), self.B)
        self.dC = hip.DeviceMatrix(M, N, np.float32, pitch32(N), self.C) if with_c else None
        self.dD = hip.DeviceMatrix(M, N, np.float32, pitch32(N))
        self.need = int(hip.lib().decx_hip_gemm_f32_workspace(M, N, K))
        assert self.need > 0 and hip.plan(4, M, N, K).k_splits > 1
        self.ws = hip.DeviceMatrix(1, self.need // 4, np.float32)

    def args(self):
        return [self.dA.ptr, self.dB.ptr, self.dC.ptr if self.dC else None, self.dD.ptr, self.M, self.N, self.K,
                self.dA.pitch, self.dB.pitch, self.dC.pitch if self.dC else 0, self.dD.pitch, 0.75, -1.25]

    def launch(self, stream, static):
        L = self.hip.lib()
        if static:
            rc = L.decx_hip_gemm_f32_static(*self.args(), stream)
        else:
            rc = L.decx_hip_gemm_f32_ws(*self.args(), self.ws.ptr, self.need, stream)
        self.hip.check(rc, "gemm")

    def poison(self):
        self.dD.upload_raw(np.full((self.M, pitch32(self.N)), -3.0, np.float32))

    def free(self):
        for d in (self.dA, self.dB, self.dC, self.dD, self.ws):
            if d is not None:
                d.free()


@pytest.mark.parametrize("static", [True, False], ids=["static workspace", "caller's workspace"])
def test_a_recorded_split_product_replays_to_the_same_bits(hip, runtime, oracle, static):
    stream = hip.Stream()
    prod = Product(hip, 300, 300, 8192, 0x7100, True)            # 25 tiles on 10 ranges each
    other = Product(hip, 1000, 1500, 777, 0x7200, False)         # launches outside the graph, between the replays
    prod.poison(); hip.sync()
    prod.launch(stream.handle, static); stream.sync()
    want = prod.dD.download()
    ref = oracle.gemm_f32(prod.A, prod.B, prod.C, 0.75, -1.25)
    assert float(np.max(np.abs(want.astype(np.float64) - ref))) / (float(np.max(np.abs(ref))) * np.sqrt(prod.K)) <= 1e-5
    other.poison(); hip.sync()
    other.launch(None, False); hip.sync()
    want_other = other.dD.download()

    before = hip.split_counter_stats()
    graph, graph_exec = ctypes.c_void_p(), ctypes.c_void_p()
    print("recording", "decx_hip_gemm_f32_static" if static else "decx_hip_gemm_f32_ws", flush=True)
    assert runtime.hipStreamBeginCapture(stream.handle, CAPTURE_MODE_GLOBAL) == 0
    try:
        prod.launch(stream.handle, static)
    finally:
        ended = runtime.hipStreamEndCapture(stream.handle, ctypes.byref(graph))
    assert ended == 0 and graph.value
    after = hip.split_counter_stats()
    assert after["reserved"] > before["reserved"], "the recorded launch ran unsplit"
    assert after["ring"] == before["ring"]
    assert runtime.hipGraphInstantiate(ctypes.byref(graph_exec), graph, None, None, 0) == 0

    for replay in range(6):
        prod.poison(); other.poison(); hip.sync()
        # eager split launches on another stream while and before the replay runs, enough of them to go round the ring
        for _ in range(40 if replay % 2 else 3):
            other.launch(None, False)
        print("replay", replay, flush=True)
        assert runtime.hipGraphLaunch(graph_exec, stream.handle) == 0
        if replay >= 3:                                          # two replays back to back on the one stream
            assert runtime.hipGraphLaunch(graph_exec, stream.handle) == 0
        other.launch(None, False)
        stream.sync(); hip.sync()
        got = prod.dD.download()
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), replay
        assert np.array_equal(other.dD.download().view(np.uint32), want_other.view(np.uint32)), replay
    # and outside the graph again
    prod.poison(); hip.sync()
    prod.launch(stream.handle, static); stream.sync()
    assert np.array_equal(prod.dD.download().view(np.uint32), want.view(np.uint32))
    assert runtime.hipGraphExecDestroy(graph_exec) == 0
    assert runtime.hipGraphDestroy(graph) == 0
    stream.destroy()
    prod.free(); other.free()
