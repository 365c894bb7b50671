"""Pins the cast half of the CPU oracle (oracle/mxq_oracle.c) without a GPU:
hand-derived known answers, the numpy baselines of the reference's own tests, an
exact-rational model of every rounding step, and algebraic invariants."""
import numpy as np
import pytest

import oracle
from tests import exact_f32 as ex


def test_known_answers_int8():
    # range (-1, 1): scale = 127; q = trunc(sign * min(|x|*127 + 0.5, 127))
    x = np.array([0.0, 0.5, -0.5, 1.0, -1.0, 2.0, -2.0, 1 / 254, 0.0039, 0.00394, -0.9999, 0.3,
                  -0.7], np.float32)
    q, mn, mx = oracle.quantize_v2(x, "int8", -1.0, 1.0)
    assert q.tolist() == [0, 64, -64, 127, -127, 127, -127, 1, 0, 1, -127, 38, -89]
    assert (mn, mx) == (-1.0, 1.0)
    # the range is max(|min|, |max|), whichever side is larger
    q, mn, mx = oracle.quantize_v2(np.array([1.0, -2.0], np.float32), "int8", -2.0, 0.5)
    assert q.tolist() == [64, -127] and (mn, mx) == (-2.0, 2.0)
    # never -128
    q, _, _ = oracle.quantize_v2(np.array([-1e30], np.float32), "int8", -1.0, 1.0)
    assert q.tolist() == [-127]


def test_known_answers_uint8_and_auto():
    q, mn, mx = oracle.quantize_v2(np.array([0.3, -1.0, 1.0, 0.0], np.float32), "uint8", -1.0, 1.0)
    # s = 127.5: (0.3+1)*127.5 + .5 = 166.25 ; 0 ; 255.5 -> 255 ; 128.0
    assert q.tolist() == [166, 0, 255, 128] and (mn, mx) == (-1.0, 1.0)
    q, _, _ = oracle.quantize_v2(np.array([0.5], np.float32), "auto", 0.0, 1.0)
    assert q.dtype == np.uint8 and q.tolist() == [128]
    q, _, _ = oracle.quantize_v2(np.array([0.5], np.float32), "auto", -0.1, 1.0)
    assert q.dtype == np.int8 and q.tolist() == [64]
    q, _, _ = oracle.quantize_v2(np.array([0.5], np.float32), "auto")
    assert q.dtype == np.int8


def test_known_answers_requantize_dequantize_range():
    mn, mx = oracle.range_for_multiplication(-1.0, 1.0, -0.08, 0.08)
    assert mx == np.float32(10651.54) and mn == -mx
    acc = np.array([1, -1, 10 ** 6, -10 ** 6, np.iinfo(np.int32).min], np.int32)
    q, rmn, rmx = oracle.requantize(acc, mn, mx, -4.0, 4.0)
    # 1e6 * (10651.54 / 2^31) = 4.96 -> 4.96*31.75 + .5 = 157.98 -> saturates
    assert q.tolist() == [0, 0, 127, -127, -127] and (rmn, rmx) == (-4.0, 4.0)
    y = oracle.dequantize(np.array([64, -127], np.int8), -1.0, 1.0)
    assert y[0] == np.float32(64) * (np.float32(1) / np.float32(127)) and y[1] == -1.0
    assert oracle.dequantize(np.array([-127], np.int8), -4.0, 3.0)[0] == -4.0
    y = oracle.dequantize(np.array([0, 255, 51], np.uint8), -1.0, 1.0)
    assert y[0] == -1.0 and abs(y[1] - 1.0) < 1e-6 and abs(y[2] - (-0.6)) < 1e-6
    # MinAbs(INT32_MIN, INT32_MAX) as floats is 2^31: int32 min maps to -range exactly
    f = ex.i32_to_float(np.iinfo(np.int32).min, -3.0, 3.0)
    assert f == -3


def test_reference_numpy_baselines():
    """The baselines the reference's tests compare against
    (tests/python/quantization/test_quantization.py:66-102, 104-143, 146-235), with
    the reference's tolerance of one level."""
    rng = np.random.default_rng(0)
    data = rng.uniform(-1.0, 1.0, size=(7, 5, 9, 3)).astype(np.float32)
    lo, hi = data.min(), data.max()
    q, mn, mx = oracle.quantize(data, lo, hi, "int8")
    real_range = np.maximum(np.abs(lo), np.abs(hi))
    base = (np.sign(data) * np.minimum(np.abs(data) * (127.0 / real_range) + 0.5, 127.0)
            ).astype(np.int8)
    assert np.abs(q.astype(int) - base.astype(int)).max() <= 1
    assert mn == -real_range and mx == real_range

    qd = rng.uniform(-127, 127, size=(4, 3, 8, 6)).astype(np.int8)
    y = oracle.dequantize(qd, -128.0, 128.0)
    np.testing.assert_allclose(y, qd * (128 / 127.0), rtol=1e-6)

    for shape, calib in [((3, 4, 10, 10), None), ((32, 3, 23, 23), (-134.349, 523.43)),
                         ((3, 4, 10, 10), (-1050.0, 1040.0))]:
        qi = rng.uniform(-1000.0, 1000.0, size=shape).astype(np.int32)

        def to_float(x):
            return x.astype("float32") * (1020.0 / float(np.iinfo("int32").max))
        rr = (max(abs(calib[0]), abs(calib[1])) if calib else
              max(abs(to_float(qi.min())), abs(to_float(qi.max()))))
        f = to_float(qi)
        base = (np.sign(f) * np.minimum(np.abs(f) * (127.0 / float(rr)) + 0.5, 127)).astype("int8")
        kw = {} if calib is None else dict(min_calib_range=calib[0], max_calib_range=calib[1])
        q, mn, mx = oracle.requantize(qi, -1010.0, 1020.0, **kw)
        assert np.abs(q.astype(int) - base.astype(int)).max() <= 1
        np.testing.assert_allclose([mn, mx], [-rr, rr], rtol=1e-6)


def _interesting_floats(rng, n, scale):
    x = (rng.standard_normal(n) * scale).astype(np.float32)
    # half-level ties and their float neighbours are where a wrong rounding shows
    ties = ((np.arange(-130, 131) + 0.5) * (scale * 4 / 127.0)).astype(np.float32)
    return np.concatenate([x, ties, np.nextafter(ties, np.float32(np.inf)),
                           np.nextafter(ties, np.float32(-np.inf)),
                           np.array([0.0, -0.0, 1e-30, -1e-30, 1e30, -1e30], np.float32)])


@pytest.mark.parametrize("lo,hi", [(-1.0, 1.0), (-4.0, 3.1), (-0.37, 2.9), (-50.0, 50.0),
                                   (-1e-3, 7e-4), (0.0, 6.0)])
def test_quantize_int8_matches_exact_rational_model(lo, hi):
    rng = np.random.default_rng(1)
    x = _interesting_floats(rng, 300, max(abs(lo), abs(hi)) / 4)
    q, mn, mx = oracle.quantize_v2(x, "int8", lo, hi)
    for xi, qi in zip(x, q):
        want, wmn, wmx = ex.quantize_int8(xi, np.float32(lo), np.float32(hi))
        assert int(qi) == want, (float(xi), lo, hi)
    assert (ex.f(mn), ex.f(mx)) == (wmn, wmx)


@pytest.mark.parametrize("lo,hi", [(-1.0, 1.0), (0.0, 6.0), (-0.37, 2.9), (-50.0, 47.5)])
def test_quantize_uint8_matches_exact_rational_model(lo, hi):
    rng = np.random.default_rng(2)
    x = rng.uniform(lo, hi, size=400).astype(np.float32)
    levels = (lo + (np.arange(0, 256) + 0.5) * ((hi - lo) / 255.0)).astype(np.float32)
    x = np.clip(np.concatenate([x, levels, np.nextafter(levels, np.float32(np.inf))]),
                np.float32(lo), np.float32(hi))
    q, mn, mx = oracle.quantize_v2(x, "uint8", lo, hi)
    for xi, qi in zip(x, q):
        assert int(qi) == ex.quantize_uint8(xi, np.float32(lo), np.float32(hi)), float(xi)
    assert (mn, mx) == (np.float32(lo), np.float32(hi))


def test_requantize_matches_exact_rational_model():
    rng = np.random.default_rng(3)
    q32 = np.concatenate([rng.integers(-2 ** 31, 2 ** 31 - 1, size=300, dtype=np.int64),
                          rng.integers(-5000, 5000, size=100),
                          [0, 1, -1, 2 ** 24, 2 ** 24 + 1, 2 ** 24 + 3, -2 ** 24 - 1, 2 ** 31 - 1,
                           -2 ** 31]]).astype(np.int32)
    for (imin, imax, calib) in [(-10651.54, 10651.54, (-4.0, 4.0)), (-3.7, 4.1, (-0.3, 0.25)),
                                (-1.0, 1.0, None)]:
        kw = {} if calib is None else dict(min_calib_range=calib[0], max_calib_range=calib[1])
        q, mn, mx = oracle.requantize(q32, imin, imax, **kw)
        if calib is None:
            rr = max(abs(ex.i32_to_float(q32.min(), np.float32(imin), np.float32(imax))),
                     abs(ex.i32_to_float(q32.max(), np.float32(imin), np.float32(imax))))
            assert ex.f(mx) == rr and ex.f(mn) == -rr
            rr = mx
        else:
            rr = np.float32(max(abs(np.float32(calib[0])), abs(np.float32(calib[1]))))
            assert mx == rr and mn == -rr
        for a, b in zip(q32, q):
            assert int(b) == ex.requantize(a, np.float32(imin), np.float32(imax), rr), int(a)


def test_dequantize_matches_exact_rational_model():
    q = np.arange(-128, 128).astype(np.int8)
    for lo, hi in [(-1.0, 1.0), (-2.73, 2.5), (-1e-3, 5e-4)]:
        y = oracle.dequantize(q, lo, hi)
        for a, b in zip(q, y):
            assert ex.f(b) == ex.dequantize_int8(a, np.float32(lo), np.float32(hi))
    u = np.arange(0, 256).astype(np.uint8)
    for lo, hi in [(0.0, 6.0), (-0.61, 3.3)]:
        y = oracle.dequantize(u, lo, hi)
        for a, b in zip(u, y):
            assert ex.f(b) == ex.dequantize_uint8(a, np.float32(lo), np.float32(hi))


def test_range_and_bias_match_exact_rational_model():
    rng = np.random.default_rng(4)
    for _ in range(50):
        a, b, c = (float(np.float32(abs(v)) + np.float32(1e-3))
                   for v in rng.standard_normal(3) * [2.0, 0.1, 0.5])
        mn, mx = oracle.range_for_multiplication(-a, a * 0.9, -b * 0.7, b)
        assert ex.f(mx) == ex.range_for_multiplication(np.float32(-a), np.float32(a * 0.9),
                                                       np.float32(-b * 0.7), np.float32(b))
        assert mn == -mx
        bias = rng.integers(-127, 128, size=40).astype(np.int8)
        b32 = oracle.bias_i8_to_i32(bias, mn, mx, -c, c * 0.8)
        for x, y in zip(bias, b32):
            assert int(y) == ex.bias_i8_to_i32(x, mn, mx, np.float32(-c), np.float32(c * 0.8))
    # zero output range -> zero bias (the reference's guard)
    assert oracle.bias_i8_to_i32(np.array([5], np.int8), 0.0, 0.0, -1.0, 1.0).tolist() == [0]


def test_invariants():
    rng = np.random.default_rng(5)
    x = (rng.standard_normal(20000) * 3).astype(np.float32)
    q, mn, mx = oracle.quantize_v2(x, "int8")
    assert mx == np.abs(x).max() and mn == -mx
    assert np.abs(q.astype(int)).max() == 127 and q.min() >= -127
    q2, _, _ = oracle.quantize_v2(-x, "int8")
    np.testing.assert_array_equal(q2, -q)                       # odd symmetry
    order = np.argsort(x, kind="stable")
    assert (np.diff(q[order].astype(int)) >= 0).all()            # monotone
    y = oracle.dequantize(q, mn, mx)
    assert np.abs(y - x).max() <= float(mx) / 254 * (1 + 1e-5)   # half-level error bound
    # calibrated with the observed range == uncalibrated
    q3, _, _ = oracle.quantize_v2(x, "int8", float(mn), float(mx))
    np.testing.assert_array_equal(q3, q)
    # relu commutes with requantize
    acc = rng.integers(-2 ** 20, 2 ** 20, size=5000).astype(np.int32)
    r1 = oracle.relu_i8(oracle.requantize(acc, -9.0, 9.0, -0.002, 0.002)[0])
    r2 = oracle.requantize(np.maximum(acc, 0), -9.0, 9.0, -0.002, 0.002)[0]
    np.testing.assert_array_equal(r1, r2)


def test_minmax():
    rng = np.random.default_rng(6)
    for n in (1, 2, 17, 100003):
        x = rng.standard_normal(n).astype(np.float32)
        assert oracle.minmax_f32(x) == (x.min(), x.max())
        i = rng.integers(-2 ** 31, 2 ** 31 - 1, size=n, dtype=np.int64).astype(np.int32)
        assert oracle.minmax_i32(i) == (int(i.min()), int(i.max()))
    x = rng.standard_normal(1000).astype(np.float32)
    x[123] = np.nan  # red::minimum / red::maximum propagate NaN (mshadow/base.h:1054-1115)
    mn, mx = oracle.minmax_f32(x)
    assert np.isnan(mn) and np.isnan(mx)


def test_exact_model_self_check():
    """The rational model itself: fl32 agrees with numpy's correctly rounded conversion
    and with textbook cases."""
    from fractions import Fraction
    assert ex.fl32(Fraction(1, 3)) == Fraction(float(np.float32(1 / 3)))
    assert ex.fl32(Fraction(2 ** 24 + 1)) == 2 ** 24          # tie -> even
    assert ex.fl32(Fraction(2 ** 24 + 3)) == 2 ** 24 + 4
    assert ex.fl32(Fraction(16777217, 2 ** 24)) == 1            # 1 + 2^-24 ties to even
    rng = np.random.default_rng(7)
    for v in rng.standard_normal(200) * 10.0 ** rng.integers(-20, 20, size=200):
        assert ex.fl32(Fraction(float(v))) == Fraction(float(np.float32(v)))
