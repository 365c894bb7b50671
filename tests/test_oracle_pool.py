"""Pins for the oracle's pooling: max against torch on integer-valued floats and brute
force, avg against an exact rational evaluation (nearest-even of sum / divisor) and the
reference test's own bound (test_quantization.py:634-639: |int8 - fp32 pooling| <= 2)."""
from fractions import Fraction

import numpy as np
import pytest
import torch

from oracle import qref


def brute(x, kernel, stride, pad, OH, OW, avg, include_pad):
    N, C, H, W = x.shape
    out = np.zeros((N, C, OH, OW), dtype=np.int64)
    lo, hi = (0, 255) if x.dtype == np.uint8 else (-128, 127)
    for oh in range(OH):
        for ow in range(OW):
            hs, ws = oh * stride[0] - pad[0], ow * stride[1] - pad[1]
            he, we = min(hs + kernel[0], H + pad[0]), min(ws + kernel[1], W + pad[1])
            size = (he - hs) * (we - ws)
            hs, ws, he, we = max(hs, 0), max(ws, 0), min(he, H), min(we, W)
            if not include_pad:
                size = (he - hs) * (we - ws)
            win = x[:, :, hs:he, ws:we].astype(np.int64).reshape(N, C, -1)
            for n in range(N):
                for c in range(C):
                    if not avg:
                        out[n, c, oh, ow] = win[n, c].max() if win.shape[2] else lo
                    else:
                        q = Fraction(int(win[n, c].sum()), size)
                        fl = q.numerator // q.denominator
                        rem = q - fl
                        r = fl + (1 if rem > Fraction(1, 2) or
                                  (rem == Fraction(1, 2) and fl % 2 == 1) else 0)
                        out[n, c, oh, ow] = min(max(r, lo), hi)
    return out


@pytest.mark.parametrize("dtype", [np.int8, np.uint8])
@pytest.mark.parametrize("kernel,stride,pad,conv", [((3, 3), (2, 2), (0, 0), "valid"),
                                                    ((3, 3), (2, 2), (1, 1), "valid"),
                                                    ((3, 3), (2, 2), (0, 0), "full"),
                                                    ((2, 3), (1, 2), (1, 0), "full"),
                                                    ((5, 5), (3, 3), (2, 2), "valid")])
@pytest.mark.parametrize("pool_type", ["max", "avg"])
def test_pool_matches_brute_force(dtype, kernel, stride, pad, conv, pool_type):
    rng = np.random.default_rng(11)
    lo, hi = (0, 256) if dtype == np.uint8 else (-128, 128)
    x = rng.integers(lo, hi, (2, 3, 13, 10)).astype(dtype)
    for include_pad in (True, False):
        out, mn, mx = qref.quantized_pooling(x, -3.0, 5.0, kernel, pool_type, stride, pad,
                                             convention=conv, count_include_pad=include_pad)
        OH, OW = out.shape[2:]
        want = brute(x, kernel, stride, pad, OH, OW, pool_type == "avg", include_pad)
        np.testing.assert_array_equal(out.astype(np.int64), want)
        assert out.dtype == dtype and (mn, mx) == (np.float32(-3.0), np.float32(5.0))


def test_max_pool_matches_torch_and_reference_test_shapes():
    rng = np.random.default_rng(5)
    x = rng.integers(-127, 128, (3, 4, 56, 56)).astype(np.int8)
    out, _, _ = qref.quantized_pooling(x, -127.0, 127.0, (3, 3), "max", (2, 2), (0, 0))
    want = torch.nn.functional.max_pool2d(torch.from_numpy(x).float(), 3, 2).numpy()
    assert out.shape == (3, 4, 27, 27)
    np.testing.assert_array_equal(out.astype(np.float32), want)
    out, _, _ = qref.quantized_pooling(x, -127.0, 127.0, (3, 3), "max", (2, 2), (0, 0),
                                       convention="full")
    want = torch.nn.functional.max_pool2d(torch.from_numpy(x).float(), 3, 2,
                                          ceil_mode=True).numpy()
    assert out.shape == (3, 4, 28, 28)
    np.testing.assert_array_equal(out.astype(np.float32), want)
    out, _, _ = qref.quantized_pooling(x, -127.0, 127.0, (3, 3), "max", (2, 2), (0, 0),
                                       global_pool=True)
    np.testing.assert_array_equal(out[:, :, 0, 0], x.reshape(3, 4, -1).max(axis=2))


def test_avg_pool_within_the_reference_tests_bound():
    rng = np.random.default_rng(6)
    for dtype, lo in ((np.int8, -127), (np.uint8, 0)):
        x = rng.integers(lo, 128, (3, 512, 7, 7)).astype(dtype)
        for gp in (False, True):
            out, _, _ = qref.quantized_pooling(x, -127.0, 127.0, (7, 7), "avg", (1, 1), (0, 0),
                                               global_pool=gp)
            want = torch.nn.functional.avg_pool2d(torch.from_numpy(x).float(), 7, 1).numpy()
            assert out.shape == (3, 512, 1, 1)
            assert np.abs(out.astype(np.float32) - want).max() <= 0.5 + 1e-6


def test_avg_ties_round_to_even_and_saturate():
    x = np.array([[[[1, 2], [3, 4]]]], dtype=np.int8)       # 10/4 = 2.5 -> 2
    assert qref.quantized_pooling(x, -1, 1, (2, 2), "avg")[0].item() == 2
    x = np.array([[[[3, 4], [3, 4]]]], dtype=np.int8)       # 14/4 = 3.5 -> 4
    assert qref.quantized_pooling(x, -1, 1, (2, 2), "avg")[0].item() == 4
    x = np.array([[[[-1, -2], [-3, -4]]]], dtype=np.int8)   # -2.5 -> -2
    assert qref.quantized_pooling(x, -1, 1, (2, 2), "avg")[0].item() == -2
    x = np.full((1, 1, 2, 2), -128, dtype=np.int8)
    assert qref.quantized_pooling(x, -1, 1, (2, 2), "avg")[0].item() == -128
    # padding counts in the divisor: 4 taps of 100 over a 3x3 window -> 400/9 = 44.4
    x = np.full((1, 1, 2, 2), 100, dtype=np.int8)
    out = qref.quantized_pooling(x, -1, 1, (3, 3), "avg", (1, 1), (1, 1))[0]
    assert out.shape == (1, 1, 2, 2) and (out == 44).all()
    out = qref.quantized_pooling(x, -1, 1, (3, 3), "avg", (1, 1), (1, 1),
                                 count_include_pad=False)[0]
    assert (out == 100).all()


def test_flatten():
    x = np.arange(2 * 3 * 4, dtype=np.int8).reshape(2, 3, 4)
    out, mn, mx = qref.quantized_flatten(x, -2.0, 3.0)
    assert out.shape == (2, 12) and (out.ravel() == x.ravel()).all()
    assert (mn, mx) == (np.float32(-2.0), np.float32(3.0))
