"""Pins oracle/conv_oracle.c without the GPU: an independent float64 formulation, scipy's correlate2d on
single-channel cases, and closed forms chosen so that a flipped kernel, swapped strides, a wrong
extension offset or a wrong output size fails one of them."""
import numpy as np
import pytest
from scipy.signal import correlate2d


def windows_f64(image, kernels, sx, sy, extend):
    """Independent restatement in float64: zero-extend, take strided windows, contract with einsum."""
    H, W, C = image.shape
    OC, KH, KW, _ = kernels.shape
    img = image.astype(np.float64)
    if extend:
        OW, OH = W // sx, H // sy
        need_w = (OW - 1) * sx + KW if OW else 0
        need_h = (OH - 1) * sy + KH if OH else 0
        padded = np.zeros((max(need_h, H + KH // 2), max(need_w, W + KW // 2), C))
        padded[KH // 2:KH // 2 + H, KW // 2:KW // 2 + W] = img
        img = padded
    else:
        OW, OH = (W - KW + 1) // sx, (H - KH + 1) // sy
    out = np.zeros((OH, OW, OC))
    for kh in range(KH):
        for kw in range(KW):
            patch = img[kh:kh + (OH - 1) * sy + 1:sy, kw:kw + (OW - 1) * sx + 1:sx]      # [OH][OW][C]
            out += np.einsum("yxc,oc->yxo", patch, kernels[:, kh, kw, :].astype(np.float64))
    return out


CASES = [(9, 7, 3, 2, 3, 3, 1, 1), (16, 12, 4, 5, 3, 5, 1, 1), (20, 17, 5, 3, 4, 2, 2, 1), (23, 19, 8, 7, 5, 3, 1, 2),
         (31, 29, 1, 1, 7, 7, 3, 2), (8, 8, 16, 33, 1, 1, 1, 1), (10, 11, 2, 4, 3, 3, 2, 2)]


@pytest.mark.parametrize("W,H,C,OC,KW,KH,sx,sy", CASES)
@pytest.mark.parametrize("extend", [False, True])
def test_against_independent_float64(oracle, W, H, C, OC, KW, KH, sx, sy, extend):
    rng = np.random.default_rng(W * 100 + H)
    image = rng.uniform(-1, 1, (H, W, C)).astype(np.float32)
    kernels = rng.uniform(-1, 1, (OC, KH, KW, C)).astype(np.float32)
    got = oracle.conv2d_f32(image, kernels, sx, sy, extend)
    want = windows_f64(image, kernels, sx, sy, extend)
    assert got.shape == want.shape
    assert oracle.conv2d_out_dims(W, H, KW, KH, sx, sy, extend) == (want.shape[1], want.shape[0])
    assert np.max(np.abs(got - want)) <= 1e-6 * np.sqrt(KW * KH * C) * max(1.0, np.max(np.abs(want)))


@pytest.mark.parametrize("KW,KH", [(3, 3), (5, 3), (2, 4)])
def test_single_channel_equals_scipy_correlate(oracle, KW, KH):
    rng = np.random.default_rng(11)
    image = rng.integers(-4, 5, (13, 17, 1)).astype(np.float32)
    kernel = rng.integers(-3, 4, (1, KH, KW, 1)).astype(np.float32)
    got = oracle.conv2d_f32(image, kernel)[:, :, 0]
    assert np.array_equal(got, correlate2d(image[:, :, 0], kernel[0, :, :, 0], mode="valid"))   # small integers: exact
    # zero extension, stride 1: scipy's zero-filled full correlation, cropped at the window origin
    full = correlate2d(image[:, :, 0], kernel[0, :, :, 0], mode="full")
    y0, x0 = KH - 1 - KH // 2, KW - 1 - KW // 2
    got_e = oracle.conv2d_f32(image, kernel, extend=True)[:, :, 0]
    assert np.array_equal(got_e, full[y0:y0 + 13, x0:x0 + 17])


def test_closed_forms(oracle):
    H, W, C = 12, 15, 3
    ones = np.ones((H, W, C), np.float32)
    box = np.ones((2, 3, 5, C), np.float32)
    out = oracle.conv2d_f32(ones, box)                       # every window holds KH * KW * C ones
    assert out.shape == (H - 2, W - 4, 2) and np.all(out == 3 * 5 * C)
    ext = oracle.conv2d_f32(ones, box, extend=True)          # at the corner only part of the window is inside
    assert ext.shape == (H, W, 2) and ext[0, 0, 0] == (3 - 1) * (5 - 2) * C and ext[5, 7, 1] == 3 * 5 * C
    rng = np.random.default_rng(3)
    image = rng.integers(-9, 10, (H, W, C)).astype(np.float32)
    shift = np.zeros((C, 3, 3, C), np.float32)               # output channel c picks channel c one row down, two columns right
    for c in range(C):
        shift[c, 1, 2, c] = 1
    out = oracle.conv2d_f32(image, shift)
    assert np.array_equal(out, image[1:H - 1, 2:W, :])       # a flipped kernel would pick [1, 0] instead
    strided = oracle.conv2d_f32(image, shift, sx=2, sy=3)
    assert np.array_equal(strided, image[1:H - 1, 2:W, :][::3, ::2][:(H - 2) // 3, :(W - 2) // 2])
