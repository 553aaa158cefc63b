"""The measurement aids of include/decx_hip_profiling.h do what the figures built on them assume: the calibration copy
copies every byte (whole 2 MiB blocks in its fast form and the remainder behind them), and the calibration read writes
nothing."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def hip():
    from decx_amd import hip as h
    h.init()
    return h


def test_calibration_copy_copies_every_byte(hip):
    rng = np.random.default_rng(0xCA11)
    for n_bytes in (5 * (1 << 20) + 48, 2 << 20, 4096):            # two blocks and a remainder; one block; a remainder only
        words = n_bytes // 4
        data = rng.integers(0, 2 ** 32, (1, words), dtype=np.uint32)
        src = hip.DeviceMatrix(1, words, np.uint32, words, data)
        dst = hip.DeviceMatrix(1, words + 8, np.uint32)
        dst.upload_raw(np.full((1, words + 8), 0xDEADBEEF, np.uint32))
        hip.check(hip.lib().decx_hip_calibration_copy(dst.ptr, src.ptr, n_bytes, None), "copy")
        hip.sync()
        got = dst.download_raw()
        assert np.array_equal(got[0, :words], data[0]), n_bytes
        assert np.all(got[0, words:] == 0xDEADBEEF), "the copy wrote beyond its size"
        src.free(); dst.free()


def test_calibration_read_stores_nothing(hip):
    n_bytes = 8 << 20
    src = hip.DeviceMatrix(1, n_bytes // 4, np.uint32)
    hip.check(hip.lib().decx_hip_memset_async(src.ptr, 1, n_bytes, None))
    sink_words = n_bytes // 2048
    sink = hip.DeviceMatrix(1, sink_words, np.uint32)
    sink.upload_raw(np.full((1, sink_words), 0x12345678, np.uint32))
    hip.check(hip.lib().decx_hip_calibration_read(src.ptr, n_bytes, sink.ptr, sink_words, None), "read")
    hip.sync()
    assert np.all(sink.download_raw() == 0x12345678)
    # sizes it does not take: not whole blocks, a sink too small
    assert hip.lib().decx_hip_calibration_read(src.ptr, n_bytes - 16, sink.ptr, sink_words, None) == -1
    assert hip.lib().decx_hip_calibration_read(src.ptr, n_bytes, sink.ptr, sink_words - 1, None) == -1
    src.free(); sink.free()
