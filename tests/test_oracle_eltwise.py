"""Pins for the oracle's quantized elemwise_add and concat.  The element rounding of both
operators lives inside oneDNN in the reference (parity unpinned for that step); what these
tests pin is everything around it: the scale derivation (against the reference test's own
bound, tests/python/quantization/test_quantization.py:375-433, which a swapped or mis-ranged
scale fails), the stated rule itself (exact rational evaluation), saturation, the type
rules and the cases the scales make exact."""
from fractions import Fraction

import numpy as np
import pytest

from oracle import qref

F = np.float32


def low_high(dtype):
    return (0.0, 255.0) if dtype == np.uint8 else (-127.0, 127.0)


def integers(rng, dtype, shape):
    lo, hi = low_high(dtype)
    return rng.uniform(lo, hi, size=shape).astype(np.int32).astype(dtype)


def round_half_even(q):
    fl = q.numerator // q.denominator
    rem = q - fl
    return fl + (1 if rem > Fraction(1, 2) or (rem == Fraction(1, 2) and fl % 2 == 1) else 0)


@pytest.mark.parametrize("shape,ta,tb", [((4, 6), np.uint8, np.int8),
                                         ((13, 74, 52), np.uint8, np.uint8),
                                         ((3, 4, 56, 56), np.int8, np.uint8),
                                         ((32, 56, 64, 11), np.int8, np.int8)])
def test_reference_elemwise_add_test(shape, ta, tb):
    """check_quantized_elemwise_add: integer-valued operands whose ranges are the types'
    (low, high); the dequantized int32 sum is within 2 of the float sum."""
    rng = np.random.default_rng(3)
    a, b = integers(rng, ta, shape), integers(rng, tb, shape)
    (alo, ahi), (blo, bhi) = low_high(ta), low_high(tb)
    out, mn, mx = qref.quantized_elemwise_add(a, b, alo, ahi, blo, bhi)
    assert out.dtype == np.int32 and out.shape == a.shape
    assert mx == F(ahi) + F(bhi) and mn == -mx
    back = out.astype(np.float32) * mx / F(0x7fffffff)
    want = a.astype(np.float32) + b.astype(np.float32)
    assert np.abs(back - want).max() <= 2
    # and much tighter than the reference asks wherever no uint8 operand was halved
    if ta == tb:
        exact = (a.astype(np.float64) * ahi / (127.5 if ta == np.int8 else 255.5) +
                 b.astype(np.float64) * bhi / (127.5 if tb == np.int8 else 255.5))
        assert np.abs(out.astype(np.float64) * float(mx) / 2147483647.0 - exact).max() < 1e-3


@pytest.mark.parametrize("ta,tb", [(np.int8, np.int8), (np.uint8, np.uint8),
                                   (np.int8, np.uint8), (np.uint8, np.int8)])
@pytest.mark.parametrize("calib", [None, (-3.0, 2.5), (-0.4, 0.7)])
def test_add_rule_exactly(ta, tb, calib):
    """out = saturate(nearest-even(float(a') * s0 + float(b') * s1)) with each binary32
    operation rounded on its own, evaluated in rationals from independently derived scales."""
    rng = np.random.default_rng(5)
    a = rng.integers(*((0, 256) if ta == np.uint8 else (-128, 128)), 4000).astype(ta)
    b = rng.integers(*((0, 256) if tb == np.uint8 else (-128, 128)), 4000).astype(tb)
    amin, amax, bmin, bmax = -1.3, 0.9, -0.2, 2.2
    kw = {} if calib is None else {"min_calib_range": calib[0], "max_calib_range": calib[1]}
    out, mn, mx = qref.quantized_elemwise_add(a, b, amin, amax, bmin, bmax, **kw)
    ra, rb = (F(255.5) if ta == np.uint8 else F(127.5)), (F(255.5) if tb == np.uint8 else F(127.5))
    a_abs, b_abs = max(abs(F(amin)), abs(F(amax))), max(abs(F(bmin)), abs(F(bmax)))
    if calib is None:
        out_range, omax = 2147483647.0, F(a_abs + b_abs)
        omin, lo, hi = -omax, -2 ** 31, 2147483520
        assert out.dtype == np.int32
    else:
        same = ta == tb
        unsigned_out = same and ta == np.uint8
        out_range = 255.5 if unsigned_out else 127.5
        omin, omax = F(calib[0]), F(calib[1])
        lo, hi = (0, 255) if unsigned_out else (-128, 127)
        assert out.dtype == (np.uint8 if unsigned_out else np.int8)
    assert (mn, mx) == (omin, omax)
    out_scale = F(out_range / float(max(abs(omin), abs(omax))))
    s0, s1 = F(out_scale / F(ra / a_abs)), F(out_scale / F(rb / b_abs))
    halve_a, halve_b = ta == np.uint8 and tb == np.int8, tb == np.uint8 and ta == np.int8
    if halve_a:
        s0 = F(s0 * F(2))
    if halve_b:
        s1 = F(s1 * F(2))
    for i in range(a.size):
        x, y = int(a[i]), int(b[i])
        if halve_a:
            x = min(round_half_even(Fraction(x, 2)), 127)
        if halve_b:
            y = min(round_half_even(Fraction(y, 2)), 127)
        # each product and the sum rounded to binary32 (numpy rounds correctly)
        t = F(F(x) * s0) + F(F(y) * s1)
        q = Fraction(float(F(t)))
        q = min(max(q, Fraction(lo)), Fraction(hi))
        assert int(out[i]) == round_half_even(q), (i, x, y)


def test_add_saturates_and_zero_is_exact():
    a = np.array([127, -127, 0, 127, -128], np.int8)
    b = np.array([127, -127, 0, -127, -128], np.int8)
    out, mn, mx = qref.quantized_elemwise_add(a, b, -1.0, 1.0, -1.0, 1.0, -0.5, 0.5)
    np.testing.assert_array_equal(out, np.array([127, -128, 0, 0, -128], np.int8))
    u = np.array([255, 0, 200], np.uint8)
    out, _, _ = qref.quantized_elemwise_add(u, u, 0.0, 1.0, 0.0, 1.0, 0.0, 1.0)
    np.testing.assert_array_equal(out, np.array([255, 0, 255], np.uint8))


def test_add_equal_ranges_is_the_integer_sum_rescaled():
    """With A = B and the calibrated range 2A, s0 = s1 = 1/2 up to one rounding: the int8
    result is nearest-even((a + b) / 2) except where the scale's rounding tips a tie."""
    rng = np.random.default_rng(9)
    a = rng.integers(-127, 128, 20000).astype(np.int8)
    b = rng.integers(-127, 128, 20000).astype(np.int8)
    out, _, _ = qref.quantized_elemwise_add(a, b, -2.0, 2.0, -2.0, 2.0, -4.0, 4.0)
    s = a.astype(np.int32) + b.astype(np.int32)
    even = s % 2 == 0
    np.testing.assert_array_equal(out[even].astype(np.int32), s[even] // 2)
    assert np.abs(out.astype(np.float64) - s / 2.0).max() <= 0.5


def test_add_rejects_bad_operands():
    a = np.zeros(4, np.int8)
    with pytest.raises(TypeError):
        qref.quantized_elemwise_add(a.astype(np.int32), a, -1, 1, -1, 1)
    with pytest.raises(ValueError):
        qref.quantized_elemwise_add(a, np.zeros(5, np.int8), -1, 1, -1, 1)


# ---- concat ------------------------------------------------------------------------------

def test_concat_of_equal_scales_is_a_byte_copy():
    rng = np.random.default_rng(2)
    xs = [rng.integers(-128, 128, (2, c, 3, 5)).astype(np.int8) for c in (4, 1, 7)]
    out, mn, mx = qref.quantized_concat(xs, [-1.5] * 3, [1.5] * 3, dim=1)
    np.testing.assert_array_equal(out, np.concatenate(xs, axis=1))
    assert (mn, mx) == (F(-1.5), F(1.5)) and out.dtype == np.int8
    us = [rng.integers(0, 256, (3, 4)).astype(np.uint8) for _ in range(2)]
    out, mn, mx = qref.quantized_concat(us, [0.0, 0.0], [2.0, 2.0], dim=0)
    np.testing.assert_array_equal(out, np.concatenate(us, axis=0))
    assert (mn, mx) == (F(0.0), F(2.0)) and out.dtype == np.uint8


@pytest.mark.parametrize("dim", [0, 1, 2, 3])
def test_concat_rescales_to_the_widest_range(dim):
    rng = np.random.default_rng(4)
    shapes = [[2, 3, 4, 5] for _ in range(3)]
    for s, e in zip(shapes, (2, 5, 1)):
        s[dim] = e
    xs = [rng.integers(-127, 128, s).astype(np.int8) for s in shapes]
    mins, maxs = [-1.0, -0.25, -3.0], [0.5, 0.3, 4.0]
    out, mn, mx = qref.quantized_concat(xs, mins, maxs, dim=dim)
    assert (mn, mx) == (F(-3.0), F(4.0))
    # hull with zero, also when every range is one-sided
    _, mn1, mx1 = qref.quantized_concat(xs[:2], [0.5, 0.25], [1.0, 2.0], dim=dim)
    assert (mn1, mx1) == (F(0.0), F(2.0))
    # each slab holds its input's real values to half an output step
    step = 4.0 / 127.5
    start = 0
    for x, lo, hi in zip(xs, mins, maxs):
        sl = [slice(None)] * 4
        sl[dim] = slice(start, start + x.shape[dim])
        start += x.shape[dim]
        real = x.astype(np.float64) * max(abs(lo), abs(hi)) / 127.5
        got = out[tuple(sl)].astype(np.float64) * step
        assert np.abs(got - real).max() <= step / 2 + 1e-6
    # the widest input itself is copied
    sl = [slice(None)] * 4
    sl[dim] = slice(out.shape[dim] - 1, None)
    np.testing.assert_array_equal(out[tuple(sl)], xs[2])


def test_concat_rescale_rule_exactly():
    x = np.arange(-128, 128).astype(np.int8)
    out, _, _ = qref.quantized_concat([x, x], [-1.0, -2.7], [0.7, 1.0], dim=0)
    scale = F(F(127.5) / F(2.7)) / F(F(127.5) / F(1.0))
    for i in range(256):
        q = Fraction(float(F(F(int(x[i])) * F(scale))))
        assert int(out[i]) == round_half_even(min(max(q, Fraction(-128)), Fraction(127)))
    np.testing.assert_array_equal(out[256:], x)


def test_concat_type_rule_and_mixed_types():
    u = np.array([0, 1, 100, 255], np.uint8)
    s = np.array([-128, -1, 0, 127], np.int8)
    out, mn, mx = qref.quantized_concat([u, s], [0.0, -1.0], [1.0, 1.0], dim=0)
    assert out.dtype == np.int8 and (mn, mx) == (F(-1.0), F(1.0))
    # uint8 steps are 1/255.5, int8 steps 1/127.5: 255 -> 127.25 -> 127
    np.testing.assert_array_equal(out[:4], np.array([0, 0, 50, 127], np.int8))
    np.testing.assert_array_equal(out[4:], s)
    out, _, _ = qref.quantized_concat([u, u], [0.0, 0.0], [1.0, 1.0], dim=0)
    assert out.dtype == np.uint8
    with pytest.raises(TypeError):
        qref.quantized_concat([u.astype(np.int32)], [0.0], [1.0], dim=0)


# ---- quantized_npi_add (broadcasting) -------------------------------------------------------

@pytest.mark.parametrize("shape,ta,tb,broadcast", [
    ((4, 6), np.uint8, np.int8, None), ((13, 74, 52), np.uint8, np.uint8, None),
    ((4, 6), np.uint8, np.int8, "A"), ((13, 74, 52), np.uint8, np.uint8, "B"),
    ((3, 4, 56, 56), np.int8, np.uint8, "A"), ((32, 56, 64, 11), np.int8, np.int8, "B")])
def test_reference_npi_add_test(shape, ta, tb, broadcast):
    """check_quantized_npi_add (test_quantization.py:436-512): one operand may be all-ones
    shaped; the dequantized int32 sum is within 2 of the float sum."""
    rng = np.random.default_rng(7)
    sa = (1,) * len(shape) if broadcast == "A" else shape
    sb = (1,) * len(shape) if broadcast == "B" else shape
    a, b = integers(rng, ta, sa), integers(rng, tb, sb)
    (alo, ahi), (blo, bhi) = low_high(ta), low_high(tb)
    out, mn, mx = qref.quantized_npi_add(a, b, alo, ahi, blo, bhi)
    assert out.dtype == np.int32 and out.shape == shape
    assert mx == F(ahi) + F(bhi) and mn == -mx
    back = out.astype(np.float32) * mx / F(0x7fffffff)
    want = a.astype(np.float32) + b.astype(np.float32)
    assert np.abs(back - want).max() <= 2


@pytest.mark.parametrize("ta,tb", [(np.int8, np.int8), (np.uint8, np.uint8),
                                   (np.int8, np.uint8), (np.uint8, np.int8)])
@pytest.mark.parametrize("calib", [None, (-3.0, 2.5)])
def test_npi_add_rule_exactly(ta, tb, calib):
    """Different shapes: saturate(nearest-even(float(a) * s0 + float(b) * s1)) on the stretched
    operands, a uint8 operand next to an int8 one at its own scale (no halving); rationals."""
    rng = np.random.default_rng(11)
    a = rng.integers(*((0, 256) if ta == np.uint8 else (-128, 128)), (6, 1, 40)).astype(ta)
    b = rng.integers(*((0, 256) if tb == np.uint8 else (-128, 128)), (5, 1)).astype(tb)
    amin, amax, bmin, bmax = -1.3, 0.9, -0.2, 2.2
    kw = {} if calib is None else {"min_calib_range": calib[0], "max_calib_range": calib[1]}
    out, mn, mx = qref.quantized_npi_add(a, b, amin, amax, bmin, bmax, **kw)
    assert out.shape == (6, 5, 40)
    ra, rb = (F(255.5) if ta == np.uint8 else F(127.5)), (F(255.5) if tb == np.uint8 else F(127.5))
    a_abs, b_abs = max(abs(F(amin)), abs(F(amax))), max(abs(F(bmin)), abs(F(bmax)))
    if calib is None:
        out_range, omax = 2147483647.0, F(a_abs + b_abs)
        omin, lo, hi = -omax, -2 ** 31, 2147483520
        assert out.dtype == np.int32
    else:
        unsigned_out = ta == tb and ta == np.uint8
        out_range = 255.5 if unsigned_out else 127.5
        omin, omax = F(calib[0]), F(calib[1])
        lo, hi = (0, 255) if unsigned_out else (-128, 127)
        assert out.dtype == (np.uint8 if unsigned_out else np.int8)
    assert (mn, mx) == (omin, omax)
    out_scale = F(out_range / float(max(abs(omin), abs(omax))))
    s0, s1 = F(out_scale / F(ra / a_abs)), F(out_scale / F(rb / b_abs))
    for i in range(6):
        for j in range(5):
            for k in range(0, 40, 3):
                t = F(F(int(a[i, 0, k])) * s0) + F(F(int(b[j, 0])) * s1)
                q = min(max(Fraction(float(F(t))), Fraction(lo)), Fraction(hi))
                assert int(out[i, j, k]) == round_half_even(q), (i, j, k)


def test_npi_add_same_shape_is_elemwise_add_and_bad_shapes_fail():
    rng = np.random.default_rng(2)
    a, b = integers(rng, np.uint8, (3, 17)), integers(rng, np.int8, (3, 17))
    x = qref.quantized_npi_add(a, b, 0.0, 2.0, -1.0, 1.0)
    y = qref.quantized_elemwise_add(a, b, 0.0, 2.0, -1.0, 1.0)
    np.testing.assert_array_equal(x[0], y[0])
    assert x[1:] == y[1:]
    with pytest.raises(ValueError):
        qref.quantized_npi_add(a, b[:, :5], 0.0, 2.0, -1.0, 1.0)
