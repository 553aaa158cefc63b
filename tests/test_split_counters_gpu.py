"""The windows of the split-K counter array on a real GPU: enough split launches to walk the array round more than
once, on one stream and on two, must leave every product bit-equal to the same product run alone; and a launch whose
window still belongs to an unfinished launch of ANOTHER stream must run unsplit instead (correct, not racing).
The bookkeeping itself is tested on the CPU (tests/test_counter_ring.py)."""
import numpy as np
import pytest

from decx_amd import synth

pytestmark = pytest.mark.gpu

TOL_F32 = 1e-5


@pytest.fixture(scope="module")
def hip():
    from decx_amd import hip as h
    h.init()
    return h


def pitch32(cols):
    return (cols + 31) // 32 * 32


class Product:
    """Operands, output and workspace of one split product, resident on the device."""

    def __init__(self, hip, M, N, K, seed):
        self.hip, self.M, self.N, self.K = hip, M, N, K
        self.A = synth.uniform_f32(M, K, seed); self.B = synth.uniform_f32(K, N, seed + 1)
        self.dA = hip.DeviceMatrix(M, K, np.float32, pitch32(K), self.A)
        self.dB = hip.DeviceMatrix(K, N, np.float32, pitch32(N), self.B)
        self.dD = hip.DeviceMatrix(M, N, np.float32, pitch32(N))
        self.need = int(hip.lib().decx_hip_gemm_f32_workspace(M, N, K))
        assert self.need > 0 and hip.plan(4, M, N, K).k_splits > 1
        self.ws = hip.DeviceMatrix(1, self.need // 4, np.float32)

    def launch(self, stream=None, split=True):
        self.hip.gemm(self.dA, self.dB, self.dD, stream=stream, workspace=self.ws if split else None)

    def alone(self, split=True):
        self.hip.sync()
        self.dD.upload_raw(np.full((self.M, pitch32(self.N)), -3.0, np.float32))
        self.launch(None, split)
        self.hip.sync()
        return self.dD.download()

    def free(self):
        for d in (self.dA, self.dB, self.dD, self.ws):
            d.free()


def counters_per_launch(hip, M, N, K):
    p = hip.plan(4, M, N, K)
    tiles = -(-M // p.tile_m) * -(-N // p.tile_n) - p.whole_tiles
    per_tile = 1 if p.k_splits <= 8 else 1 + -(-p.k_splits // 4)
    return tiles * per_tile


def test_one_stream_walks_the_array_round(hip, oracle):
    M, N, K = 1000, 1500, 777                                   # 128 split tiles on two ranges beside 256 whole ones
    prod = Product(hip, M, N, K, 0x6100)
    want = prod.alone()
    ref = oracle.gemm_f32(prod.A, prod.B)
    assert float(np.max(np.abs(want.astype(np.float64) - ref))) / (float(np.max(np.abs(ref))) * np.sqrt(K)) <= TOL_F32
    per = counters_per_launch(hip, M, N, K)
    before = hip.split_counter_stats()
    launches = 2 * (before["ring"] // per) + 50
    print("one stream:", launches, "launches of", per, "counters", flush=True)
    for i in range(launches):
        prod.launch()
        if i % 197 == 0:
            hip.sync()
            assert np.array_equal(prod.dD.download().view(np.uint32), want.view(np.uint32)), i
    hip.sync()
    after = hip.split_counter_stats()
    assert after["wraps"] - before["wraps"] >= 2
    assert after["refused"] == before["refused"]                # one stream runs its launches in order: never refused
    assert np.array_equal(prod.dD.download().view(np.uint32), want.view(np.uint32))
    prod.free()


def test_two_streams_walk_the_array_round(hip):
    shapes = [(1000, 1500, 777), (300, 300, 8192)]
    prods = [Product(hip, *s, 0x6200 + 16 * i) for i, s in enumerate(shapes)]
    want = [p.alone() for p in prods]
    plain = [p.alone(split=False) for p in prods]
    streams = [hip.Stream(), hip.Stream()]
    per = sum(counters_per_launch(hip, *s) for s in shapes)
    before = hip.split_counter_stats()
    rounds = 2 * (before["ring"] // per) + 20
    print("two streams:", rounds, "rounds of", per, "counters", flush=True)
    for i in range(rounds):
        for p, s in zip(prods, streams):
            p.launch(s.handle)
        if i % 101 == 0:                                        # let the host look in now and then; mostly the queues stay full
            for s in streams:
                s.sync()
            for p, w, u in zip(prods, want, plain):
                got = p.dD.download().view(np.uint32)
                assert np.array_equal(got, w.view(np.uint32)) or np.array_equal(got, u.view(np.uint32)), i
    for s in streams:
        s.sync()
    after = hip.split_counter_stats()
    assert after["wraps"] - before["wraps"] >= 2
    assert after["events"] - before["events"] >= rounds          # more than one stream: every split launch carries an event
    # whatever happened on the way, the counters are all zero again: the products run alone come out as before
    for p, w in zip(prods, want):
        assert np.array_equal(p.alone().view(np.uint32), w.view(np.uint32))
    for s in streams:
        s.destroy()
    for p in prods:
        p.free()


def test_a_window_of_a_busy_stream_is_not_handed_out(hip, oracle):
    """Stream A queues a long product and a split one behind it; stream B then launches split products until its
    windows come round to the one A's launch holds.  A has not finished: B's launch there runs unsplit."""
    big = 6144
    dX = hip.DeviceMatrix(big, big, np.float32, big, synth.uniform_f32(big, big, 0x6301))
    dY = hip.DeviceMatrix(big, big, np.float32, big)
    a = Product(hip, 300, 300, 8192, 0x6310)
    b = Product(hip, 1000, 1500, 777, 0x6320)
    want_a, want_b, plain_b = a.alone(), b.alone(), b.alone(split=False)
    assert not np.array_equal(want_b, plain_b)                  # (the two orders of summation differ in some bit)
    sa, sb = hip.Stream(), hip.Stream()
    per_b = counters_per_launch(hip, 1000, 1500, 777)
    before = hip.split_counter_stats()
    launches = before["ring"] // per_b + 8
    print("busy stream: 24 products of", big, "cubed on A, then", launches, "split launches on B", flush=True)
    for _ in range(24):                                         # about 70 ms of work in front of A's split launch
        hip.gemm(dX, dX, dY, stream=sa.handle)
    a.launch(sa.handle)
    for _ in range(launches):
        b.launch(sb.handle)
    sb.sync()
    refused = hip.split_counter_stats()["refused"] - before["refused"]
    got_b = b.dD.download()
    sa.sync()
    got_a = a.dD.download()
    assert refused >= 1, "B came round to A's window while A was busy and must have been refused"
    assert np.array_equal(got_a.view(np.uint32), want_a.view(np.uint32))
    assert np.array_equal(got_b.view(np.uint32), want_b.view(np.uint32)) or np.array_equal(got_b.view(np.uint32), plain_b.view(np.uint32))
    ref = oracle.gemm_f32(b.A, b.B)
    assert float(np.max(np.abs(got_b.astype(np.float64) - ref))) / (float(np.max(np.abs(ref))) * np.sqrt(777)) <= TOL_F32
    # A is done now: B's next launch gets its window again
    mid = hip.split_counter_stats()["refused"]
    b.launch(sb.handle)
    sb.sync()
    assert hip.split_counter_stats()["refused"] == mid
    assert np.array_equal(b.dD.download().view(np.uint32), want_b.view(np.uint32))
    for s in (sa, sb):
        s.destroy()
    for d in (dX, dY):
        d.free()
    a.free(); b.free()


def test_host_threads_with_streams_of_their_own(hip):
    """Four host threads launch split products at the same time, each on its own stream, workspace and output: the
    windows are handed out under the library's lock, and whatever a thread gets (a window, or a refusal while another
    stream's launch still holds it) its product has the bits of the split or of the unsplit form."""
    import threading
    shapes = [(1000, 1500, 777), (300, 300, 8192), (640, 640, 4096), (100, 120, 4096)]
    prods = [Product(hip, *s, 0x6500 + 16 * i) for i, s in enumerate(shapes)]
    want = [p.alone() for p in prods]
    plain = [p.alone(split=False) for p in prods]
    streams = [hip.Stream() for _ in prods]
    before = hip.split_counter_stats()
    wrong = []

    def work(i):
        p, s = prods[i], streams[i]
        try:
            for n in range(400):
                p.launch(s.handle)
                if n % 80 == 79:
                    s.sync()
                    got = p.dD.download().view(np.uint32)
                    if not (np.array_equal(got, want[i].view(np.uint32)) or np.array_equal(got, plain[i].view(np.uint32))):
                        wrong.append((i, n))
        except Exception as e:                                   # noqa: BLE001 -- reported by the main thread
            wrong.append((i, repr(e)))

    print("four host threads, 400 split launches each", flush=True)
    threads = [threading.Thread(target=work, args=(i,)) for i in range(len(prods))]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    for s in streams:
        s.sync()
    assert not wrong, wrong
    after = hip.split_counter_stats()
    assert after["taken"] + after["refused"] - before["taken"] - before["refused"] == 400 * len(prods)
    assert after["taken"] - before["taken"] >= 400              # most launches do get their window
    for p, w in zip(prods, want):                               # all counters are back at zero
        assert np.array_equal(p.alone().view(np.uint32), w.view(np.uint32))
    for s in streams:
        s.destroy()
    for p in prods:
        p.free()


def test_reset_puts_the_counters_back(hip):
    p = Product(hip, 300, 300, 8192, 0x6400)
    want = p.alone()
    hip.check(hip.lib().decx_hip_reset_split_counters(), "reset")
    assert np.array_equal(p.alone().view(np.uint32), want.view(np.uint32))
    p.free()
