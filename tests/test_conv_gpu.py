"""Parity of the implicit-GEMM convolution (through the C ABI) against the CPU oracle.
Bar: max|d| / (max|ref| * sqrt(KH * KW * C)) <= 1e-5 (fp32); bit-exact on small-integer data."""
import numpy as np
import pytest

from decx_amd import synth

pytestmark = pytest.mark.gpu
TOL = 1e-5


@pytest.fixture(scope="module")
def hip():
    from decx_amd import hip as h
    h.init()
    return h


def rel_err(got, ref, K):
    ref = ref.astype(np.float64)
    return float(np.max(np.abs(got.astype(np.float64) - ref))) / (max(float(np.max(np.abs(ref))), 1e-30) * np.sqrt(K))


def data(W, H, C, OC, KW, KH, seed):
    image = synth.uniform_f32(H, W * C, seed).reshape(H, W, C)
    kernels = synth.uniform_f32(OC, KH * KW * C, seed + 1).reshape(OC, KH, KW, C)
    return image, kernels


CASES = [  # W, H, C, OC, KW, KH, sx, sy
    (9, 7, 3, 2, 3, 3, 1, 1), (16, 12, 4, 5, 3, 5, 1, 1), (20, 17, 5, 3, 4, 2, 2, 1), (23, 19, 8, 7, 5, 3, 1, 2),
    (31, 29, 1, 1, 7, 7, 3, 2), (8, 8, 16, 33, 1, 1, 1, 1), (10, 11, 2, 4, 3, 3, 2, 2),
    (64, 48, 16, 64, 3, 3, 1, 1), (57, 43, 13, 70, 3, 3, 1, 1), (130, 70, 32, 96, 5, 5, 2, 2), (40, 40, 64, 300, 3, 3, 1, 1),
    (33, 9, 24, 16, 11, 1, 1, 1), (12, 40, 12, 16, 1, 9, 1, 3),
    # shallow patches, few kernels, a short channel pitch: the lane-per-pixel kernel (several workgroups, a partial last one)
    (640, 480, 3, 16, 3, 3, 1, 1), (200, 150, 4, 32, 5, 5, 2, 1), (333, 77, 7, 5, 2, 3, 1, 2), (1030, 9, 1, 29, 3, 3, 1, 1),
]


@pytest.mark.parametrize("W,H,C,OC,KW,KH,sx,sy", CASES)
@pytest.mark.parametrize("extend", [False, True])
def test_conv2d_against_oracle(hip, oracle, W, H, C, OC, KW, KH, sx, sy, extend):
    image, kernels = data(W, H, C, OC, KW, KH, 500 + W)
    ref = oracle.conv2d_f32(image, kernels, sx, sy, extend)
    got, raw = hip.conv2d(image, kernels, sx, sy, extend)
    assert got.shape == ref.shape
    assert not np.isnan(got).any(), "NaN leaked from the row padding of the image"
    assert rel_err(got, ref, KW * KH * C) <= TOL
    oh, ow = ref.shape[:2]
    assert np.all(raw[:oh, ow:, :] == np.float32(-555.0)), "padding columns of dst were written"
    assert np.all(raw[:oh, :ow, OC:] == np.float32(-555.0)), "padding channels of dst were written"


def test_conv2d_exact_on_small_integers(hip, oracle):
    rng = np.random.default_rng(9)
    image = rng.integers(-3, 4, (37, 41, 6)).astype(np.float32)
    kernels = rng.integers(-2, 3, (10, 3, 3, 6)).astype(np.float32)
    for extend in (False, True):
        got, _ = hip.conv2d(image, kernels, extend=extend)
        assert np.array_equal(got, oracle.conv2d_f32(image, kernels, extend=extend))
    shift = np.zeros((6, 3, 3, 6), np.float32)
    for c in range(6):
        shift[c, 1, 2, c] = 1                                  # picks one row down, two columns right: no flip
    got, _ = hip.conv2d(image, shift)
    assert np.array_equal(got, image[1:36, 2:41, :])


def test_conv2d_large_sampled(hip, oracle):
    """256 x 256 x 112 image, 256 kernels of 3 x 3: 64 516 x 256 x 1008, the tall-skinny GEMM shape."""
    W = H = 256; C = 112; OC = 256
    image, kernels = data(W, H, C, OC, 3, 3, 700)
    got, _ = hip.conv2d(image, kernels)
    rows = [0, 1, 100, 253]
    ref = oracle.conv2d_f32(image[:5], kernels)                # first output rows from the first image rows
    assert rel_err(got[:3], ref, 9 * C) <= TOL
    ref_tail = oracle.conv2d_f32(image[-3:], kernels)
    assert rel_err(got[-1:], ref_tail, 9 * C) <= TOL
    # checksum over all pixels: sum_out(oc) = sum over windows, in float64
    win = sum(image[kh:kh + 254, kw:kw + 254].astype(np.float64).sum(axis=(0, 1))[None, :] * kernels[:, kh, kw, :].astype(np.float64)
              for kh in range(3) for kw in range(3)).sum(axis=1)
    assert np.max(np.abs(got.astype(np.float64).sum(axis=(0, 1)) - win)) / np.max(np.abs(win)) < 1e-5


def test_conv2d_invalid_arguments(hip):
    L = hip.lib()
    d = hip.DeviceMatrix(8, 64, np.float32, data=np.zeros((8, 64), np.float32))
    ok = [d.ptr, d.ptr, d.ptr, 2, 2, 4, 3, 3, 4, 8, 1, 1, 4, 4, 8, None]
    assert L.decx_hip_conv2d_f32(*ok) == 0
    for idx, bad in ((0, None), (8, 3), (12, 3), (13, 3), (9, 3), (10, 0), (14, 1)):
        args = list(ok); args[idx] = bad
        assert L.decx_hip_conv2d_f32(*args) == -1, idx
    assert L.decx_hip_conv2d_f32(d.ptr, d.ptr, d.ptr, 0, 2, 4, 3, 3, 4, 8, 1, 1, 4, 4, 8, None) == 0      # empty output
    # the same call with the number of channels that exist: 1 .. the channel pitch
    withdepth = lambda depth: L.decx_hip_conv2d_f32_depth(d.ptr, d.ptr, d.ptr, 2, 2, 4, 3, 3, depth, 4, 8, 1, 1, 4, 4, 8, None)
    assert withdepth(3) == 0 and withdepth(4) == 0 and withdepth(0) == -1 and withdepth(5) == -1


@pytest.mark.parametrize("OC", [4, 8, 12, 16, 20, 24, 28, 32, 3, 6, 10, 30])
@pytest.mark.parametrize("W,H", [(70, 50), (259, 21), (64, 9)])
def test_every_store_path_of_the_lane_per_pixel_kernel(hip, oracle, OC, W, H):
    """3 x 3 over RGB.  A multiple of four kernels from 8 up: a wavefront lays its 64 pixels out in LDS and stores whole
    cache lines (here with image rows that end inside a wavefront: 68, 257 and 62 output pixels per row, the destination's
    rows are longer, and the last wavefront has idle lanes); 4 kernels: one piece per lane; any other number: the last
    piece element by element, the channels beyond the kernels untouched.  Bit-exact: the kernel runs the oracle's chain."""
    image, kernels = data(W, H, 3, OC, 3, 3, 7000 + OC + W)
    ref = oracle.conv2d_f32(image, kernels, 1, 1, False)
    got, raw = hip.conv2d(image, kernels, 1, 1, False)
    assert got.shape == ref.shape == (H - 2, W - 2, OC)
    assert np.array_equal(got.view(np.uint32), ref.view(np.uint32))
    oh, ow = ref.shape[:2]
    assert np.all(raw[:oh, ow:, :] == np.float32(-555.0)), "padding columns of dst were written"
    assert np.all(raw[:oh, :ow, OC:] == np.float32(-555.0)), "padding channels of dst were written"
    assert np.all(raw[oh:] == np.float32(-555.0)), "rows beyond the output were written"


@pytest.mark.parametrize("C", [1, 2, 3])
@pytest.mark.parametrize("extend", [False, True])
def test_padding_channel_of_grey_and_rgb_images_is_never_read_into_a_result(hip, oracle, C, extend):
    """Channel pitch 4 with 1 to 3 real channels and few kernels: the lane-per-pixel kernel leaves the padding
    channels out of its arithmetic, so NaN in them must not reach the output (the GEMM form would multiply them by
    zero weights: NaN)."""
    W, H, OC, KW, KH = 96, 40, 8, 3, 3
    image, kernels = data(W, H, C, OC, KW, KH, 900 + C)
    ref = oracle.conv2d_f32(image, kernels, 1, 1, extend)
    got, _ = hip.conv2d(image, kernels, 1, 1, extend, channel_pad_value=np.nan)
    assert np.isfinite(got).all(), "a padding channel reached the result"
    assert rel_err(got, ref, KW * KH * C) <= TOL
