"""Pins for the oracle's quantized elemwise_mul, quantize_asym, embedding, transpose and
reshape.  The first two are native C++ loops in the reference
(quantized_elemwise_mul.cc:114-206, quantize_asym-inl.h:62-152): each rounding step is
evaluated here in exact rationals (tests/exact_f32.py shares no code with the C oracle),
plus hand-derived answers, the reference test's own check and closed forms.  The other three
move bytes; numpy's take / transpose / reshape are the statement of what they do."""
from fractions import Fraction

import numpy as np
import pytest

from exact_f32 import f, fl32, fl64, trunc
from oracle import qref

F = np.float32


def maxabs(a, b):
    """MaxAbs of two attribute / range values, which reach the operator as binary32."""
    return max(abs(f(F(a))), abs(f(F(b))))


def wrap8(v):
    return ((v + 128) % 256) - 128


def exact_mul(a, b, lmin, lmax, rmin, rmax, calib=None, as_float=False):
    """quantized_elemwise_mul.cc:114-199 on one pair, one rounding per written operation."""
    k = Fraction(255, 2)  # kInt8Range = 127.5f
    lhs_scale = fl32(k / maxabs(lmin, lmax))
    rhs_scale = fl32(k / maxabs(rmin, rmax))
    if as_float:
        out_scale = fl32(fl64(fl64(Fraction(1) / lhs_scale) / rhs_scale))
    elif calib is not None:
        out_data_scale = fl32(fl64(k / maxabs(*calib)))
        out_scale = fl32(fl32(out_data_scale / lhs_scale) / rhs_scale)
    else:
        out_scale = Fraction(1)
    v = fl32(Fraction(int(a) * int(b)) * out_scale)
    if as_float:
        return v
    return wrap8(trunc(v)) if calib is not None else trunc(v)


@pytest.mark.parametrize("shape", [(4, 6), (13, 74, 52), (3, 4, 56, 56)])
def test_reference_elemwise_mul_test(shape):
    """check_quantized_elemwise_mul (test_quantization.py:514-569): integer-valued operands,
    no calibration: the int32 output is the float product."""
    rng = np.random.default_rng(5)
    a = rng.uniform(-127, 127, size=shape).astype(np.int32).astype(np.int8)
    b = rng.uniform(-127, 127, size=shape).astype(np.int32).astype(np.int8)
    out, mn, mx = qref.quantized_elemwise_mul(a, b, -127.0, 127.0, -127.0, 127.0)
    assert out.dtype == np.int32 and out.shape == a.shape
    assert np.array_equal(out, a.astype(np.int32) * b.astype(np.int32))
    assert np.allclose(out.astype(np.float32), a.astype(np.float32) * b.astype(np.float32),
                       atol=1e-4)
    # QuantizationRangeForMultiplication<int8,int8,int32>: (127/127)^2 * 2^31
    assert mx == F(2147483648.0) and mn == -mx


def test_mul_known_answers():
    a = np.array([-128, 127, 5, 0, -1, 100], dtype=np.int8)
    b = np.array([-128, 2, -7, 9, -1, 100], dtype=np.int8)
    out, mn, mx = qref.quantized_elemwise_mul(a, b, -1.0, 1.0, -2.0, 2.0)
    assert out.tolist() == [16384, 254, -35, 0, 1, 10000]
    # (1/127) * (2/127) * 2^31 in binary32
    want = F(F(F(1.0) / F(127.0)) * F(F(2.0) / F(127.0))) * F(2147483648.0)
    assert mx == want and mn == -want
    # float output: scale = (1/127.5) * (2/127.5) up to the roundings
    fo = qref.quantized_elemwise_mul(a, b, -1.0, 1.0, -2.0, 2.0, enable_float_output=True)
    assert fo.dtype == np.float32
    assert np.allclose(fo, a.astype(np.float64) * b.astype(np.float64) * 2.0 / 127.5 ** 2,
                       rtol=1e-6)
    # calibrated to the full product range 1 * 2: q = trunc(a * b / 127.5)
    q, mn, mx = qref.quantized_elemwise_mul(a, b, -1.0, 1.0, -2.0, 2.0, -2.0, 2.0)
    assert q.dtype == np.int8 and (mn, mx) == (F(-2.0), F(2.0))
    assert q.tolist() == [wrap8(int(int(x) * int(y) / 127.5)) for x, y in zip(a, b)]


@pytest.mark.parametrize("ranges", [(-1.0, 1.0, -2.0, 2.0), (-0.37, 0.91, -3.3, 1.25),
                                    (0.0, 6.0, -1e-3, 5e-4)])
@pytest.mark.parametrize("mode", ["int32", "int8", "int8_narrow", "float"])
def test_mul_rule_exactly(ranges, mode):
    rng = np.random.default_rng(11)
    a = rng.integers(-128, 128, size=400, dtype=np.int8)
    b = rng.integers(-128, 128, size=400, dtype=np.int8)
    a[:4] = [-128, 127, -128, 0]
    b[:4] = [-128, 127, 127, 5]
    lmin, lmax, rmin, rmax = ranges
    full = float(max(abs(lmin), abs(lmax)) * max(abs(rmin), abs(rmax)))
    if mode == "float":
        got = qref.quantized_elemwise_mul(a, b, *ranges, enable_float_output=True)
        for i in range(a.size):
            assert f(got[i]) == exact_mul(a[i], b[i], *ranges, as_float=True)
        return
    # "int8_narrow": a calibrated range a quarter of the product's: results wrap (undefined
    # in the reference; the oracle keeps gcc's low byte)
    calib = None if mode == "int32" else ((-full, full) if mode == "int8" else
                                          (-full / 4, full / 5))
    kw = {} if calib is None else {"min_calib_range": calib[0], "max_calib_range": calib[1]}
    got, mn, mx = qref.quantized_elemwise_mul(a, b, *ranges, **kw)
    for i in range(a.size):
        assert int(got[i]) == exact_mul(a[i], b[i], *ranges, calib=calib)
    if calib is not None:
        assert (mn, mx) == (F(calib[0]), F(calib[1]))


def test_mul_type_rules():
    a = np.zeros((2, 3), dtype=np.int8)
    with pytest.raises(TypeError):
        qref.quantized_elemwise_mul(a.astype(np.uint8), a, 0, 1, 0, 1)
    with pytest.raises(ValueError):
        qref.quantized_elemwise_mul(a, a.reshape(3, 2), 0, 1, 0, 1)
    # one calibration bound alone does not calibrate (quantized_elemwise_mul.cc:76-79)
    out, _, _ = qref.quantized_elemwise_mul(a, a, -1, 1, -1, 1, min_calib_range=-1.0)
    assert out.dtype == np.int32


# ---- quantize_asym ---------------------------------------------------------------------

def exact_asym(x, lo, hi):
    lo, hi, x = f(F(lo)), f(F(hi)), f(x)
    scale = fl32(Fraction(255) / fl32(hi - lo))
    shift = fl32(Fraction(255) - fl32(hi * scale))
    t = fl32(fl32(x * scale) + shift)
    return trunc(fl64(t + Fraction(1, 2))) % 256, scale, shift


@pytest.mark.parametrize("lo,hi", [(-1.0, 3.0), (0.0, 6.0), (-0.731, 0.2089), (-50.0, 50.0)])
def test_asym_rule_exactly(lo, hi):
    rng = np.random.default_rng(2)
    x = rng.uniform(lo, hi, size=500).astype(np.float32)
    x[:6] = [lo, hi, 0.0 if lo <= 0 <= hi else lo, (lo + hi) / 2, np.nextafter(F(hi), F(lo)),
             np.nextafter(F(lo), F(hi))]
    q, scale, shift = qref.quantize_asym(x, lo, hi)
    assert q.dtype == np.uint8
    for i in range(x.size):
        want, s, sh = exact_asym(x[i], lo, hi)
        assert int(q[i]) == want
    assert f(scale) == s and f(shift) == sh


def test_asym_closed_forms():
    """min -> 0 and max -> 255 whenever scale and shift are exact; equal steps in between;
    without calibration the data's own min and max are the range."""
    x = np.array([-1.0, 0.0, 0.5, 3.0], dtype=np.float32)
    q, scale, shift = qref.quantize_asym(x)
    assert (scale, shift) == (F(63.75), F(63.75))
    assert q.tolist() == [0, 64, 96, 255]          # 63.75 + 0.5 -> 64; 95.625 + 0.5 -> 96
    assert np.array_equal(q, qref.quantize_asym(x, -1.0, 3.0)[0])
    ramp = np.arange(256, dtype=np.float32) * F(0.25) - F(16.0)
    q, scale, shift = qref.quantize_asym(ramp)
    assert scale == F(4.0) and shift == F(64.0)
    assert q.tolist() == list(range(256))
    # dequantized error at most half a step
    x = np.random.default_rng(0).uniform(-2, 5, 10000).astype(np.float32)
    q, scale, shift = qref.quantize_asym(x)
    back = (q.astype(np.float64) - float(shift)) / float(scale)
    assert np.abs(back - x).max() <= 0.5 / float(scale) + 1e-5


def test_asym_byte_inputs_and_out_of_range():
    i8 = np.array([-128, -1, 0, 127], dtype=np.int8)
    q, scale, shift = qref.quantize_asym(i8)
    assert q.tolist() == [0, 127, 128, 255] and (scale, shift) == (F(1.0), F(128.0))
    u8 = np.array([0, 7, 255], dtype=np.uint8)
    q, scale, shift = qref.quantize_asym(u8)
    assert q.tolist() == [0, 7, 255] and (scale, shift) == (F(1.0), F(0.0))
    # outside a narrower calibrated range the reference's conversion is undefined; the oracle
    # keeps the low byte of the truncated int32
    x = np.array([-2.0, 2.0], dtype=np.float32)
    q, _, _ = qref.quantize_asym(x, -1.0, 1.0)
    assert q.tolist() == [(-127) % 256, (383) % 256]   # trunc(-127.5 + 0.5), trunc(382.5 + 0.5)


# ---- embedding / transpose / reshape ------------------------------------------------------

@pytest.mark.parametrize("shape,input_dim,output_dim", [((1,), 1000, 256), ((1,), 1024, 512),
                                                        ((32,), 1000, 256), ((32,), 1024, 512),
                                                        ((4, 7), 50, 24)])
def test_reference_embedding_test(shape, input_dim, output_dim):
    """check_quantized_embedding (test_quantization.py:833-905): integer-valued float
    indices and an integer-valued table; the int8 rows are the float embedding's rows."""
    rng = np.random.default_rng(7)
    data = rng.uniform(0, input_dim, size=shape).astype(np.int32).astype(np.float32)
    weight = rng.uniform(-127, 127, size=(input_dim, output_dim)).astype(np.int32)
    w8 = weight.astype(np.int8)
    r = float(np.abs(weight).max())
    out, mn, mx = qref.quantized_embedding(data, w8, -r, r)
    assert out.dtype == np.int8 and out.shape == shape + (output_dim,)
    want = weight.astype(np.float32)[data.astype(np.int64)]
    assert np.array_equal(out.astype(np.float32), want)
    assert (mn, mx) == (F(-r), F(r))


def test_embedding_clip_and_index_types():
    w = np.arange(5 * 3, dtype=np.int8).reshape(5, 3)
    for idx in (np.array([-3, 0, 4, 5, 99], dtype=np.int32), np.array([-3, 0, 4, 5, 99], np.int64),
                np.array([-3.9, 0.9, 4.2, 5.0, 1e9], dtype=np.float32),
                np.array([-0.5, 0.99, 4.999, 5.5, 99.0], dtype=np.float64)):
        out, _, _ = qref.quantized_embedding(idx, w, -1, 1)
        assert np.array_equal(out, w[[0, 0, 4, 4, 4]])   # truncated toward zero, then clipped
    out, _, _ = qref.quantized_embedding(np.array([250, 2], dtype=np.uint8), w, -1, 1)
    assert np.array_equal(out, w[[4, 2]])


@pytest.mark.parametrize("shape,axes", [((), ()), ((2, 3), (1, 0)), ((8, 21), (1, 0)),
                                        ((7, 3, 9), (2, 1, 0)), ((5, 3, 6, 8), (2, 3, 0, 1)),
                                        ((5, 3, 6, 8), None)])
@pytest.mark.parametrize("dtype", [np.int8, np.uint8])
def test_reference_transpose_test(shape, axes, dtype):
    """check_quantized_transpose (test_quantization.py:811-830)."""
    rng = np.random.default_rng(1)
    lo, hi = (0, 255) if dtype == np.uint8 else (-127, 127)
    data = rng.uniform(lo, hi, size=shape).astype(dtype)
    out, mn, mx = qref.quantized_transpose(data, -3.5, 7.25, axes=axes)
    want = np.transpose(data.astype(np.float32), axes)
    assert out.dtype == dtype and np.array_equal(out.astype(np.float32), want)
    assert out.flags["C_CONTIGUOUS"] and (mn, mx) == (F(-3.5), F(7.25))
    # element by element: out[i0, i1, ...] = in[j] with j[axes[d]] = i[d]
    perm = tuple(reversed(range(len(shape)))) if axes is None else axes
    for idx in np.ndindex(*out.shape):
        src = [0] * len(shape)
        for d, ax in enumerate(perm):
            src[ax] = idx[d]
        assert out[idx] == data[tuple(src)]


def test_reshape_is_a_copy_with_ranges():
    d = np.arange(-60, 60, dtype=np.int8).reshape(2, 3, 4, 5)
    out, mn, mx = qref.quantized_reshape(d, -1023.343, 2343.324275, (6, 20))
    assert out.shape == (6, 20) and np.array_equal(out.ravel(), d.ravel())
    assert (mn, mx) == (F(-1023.343), F(2343.324275))


# ---- batch norm -----------------------------------------------------------------------------

def round_half_even(q):
    fl = q.numerator // q.denominator
    rem = q - fl
    return fl + (1 if rem > Fraction(1, 2) or (rem == Fraction(1, 2) and fl % 2 == 1) else 0)


def exact_bn(x, unsigned, gamma, beta, mean, var, min_data, max_data, eps, calib, relu):
    """dnnl_quantized_batch_norm.cc:66-112 for one element, one rounding per written operation;
    then the stated rule saturate(nearest-even((w / sqrtf(1 + eps)) * x + b))."""
    from math import isqrt
    max_abs_data, max_abs_out = maxabs(min_data, max_data), maxabs(*calib)
    # float(1.0 / sqrt(double(var) + eps)): the double sqrt and division through Python floats
    # (IEEE binary64, correctly rounded), then one rounding to binary32
    invstd = f(F(1.0 / np.sqrt(np.float64(F(var)) + np.float64(eps))))
    g, b_, m = f(F(gamma)), f(F(beta)), f(F(mean))
    w = fl32(fl32(fl32(g * invstd) * max_abs_data) / max_abs_out)
    b = fl32(fl32(fl32(b_ - fl32(fl32(m * g) * invstd)) * Fraction(255, 2)) / max_abs_out)
    unit = f(np.sqrt(F(1.0) + F(eps), dtype=np.float32))
    wn = fl32(w / unit)
    if unsigned:
        x = max(-128, min(127, round_half_even(fl32(Fraction(int(x)) * f(F(127.5) / F(255.5))))))
    v = fl32(fl32(Fraction(int(x)) * wn) + b)
    if relu and v < 0:
        v = Fraction(0)
    return max(-128, min(127, round_half_even(v)))


@pytest.mark.parametrize("dtype", [np.int8, np.uint8])
@pytest.mark.parametrize("relu", [False, True])
@pytest.mark.parametrize("eps", [1e-3, 2e-5])
def test_batch_norm_rule_exactly(dtype, relu, eps):
    rng = np.random.default_rng(13)
    C = 5
    lo, hi = (0, 256) if dtype == np.uint8 else (-128, 128)
    d = rng.integers(lo, hi, (3, C, 7)).astype(dtype)
    gamma = rng.uniform(0.5, 2.0, C).astype(np.float32)
    beta = rng.normal(0, 0.5, C).astype(np.float32)
    mean = rng.normal(0, 0.3, C).astype(np.float32)
    var = rng.uniform(0.3, 2.0, C).astype(np.float32)
    rd = (0.0, 3.1) if dtype == np.uint8 else (-2.7, 3.1)
    calib = (-6.5, 7.25)
    out, mn, mx = qref.quantized_batch_norm(d, gamma, beta, mean, var, rd[0], rd[1], calib[0],
                                            calib[1], eps=eps, relu=relu)
    assert out.dtype == np.int8 and (mn, mx) == (F(calib[0]), F(calib[1]))
    for idx in np.ndindex(*d.shape):
        c = idx[1]
        assert int(out[idx]) == exact_bn(d[idx], dtype == np.uint8, gamma[c], beta[c], mean[c],
                                         var[c], rd[0], rd[1], eps, calib, relu), idx


@pytest.mark.parametrize("shape,axis", [((8, 16, 4, 4), 1), ((4, 6, 5, 3), -1), ((10, 7), 1)])
def test_batch_norm_tracks_the_float_operator(shape, axis):
    """check_quantized_bn (test_quantization.py:1005-1050): the dequantized int8 result is the
    float batch norm within rtol 0.1 / atol 8 there; within 1.5 output levels + the 0.05 %
    that the library's second division by sqrt(1 + eps) costs here."""
    rng = np.random.default_rng(17)
    C = shape[axis]
    d = rng.integers(-127, 128, shape).astype(np.int8)
    gamma = rng.uniform(0.5, 2.0, C).astype(np.float32)
    beta = rng.normal(0, 0.5, C).astype(np.float32)
    mean = rng.normal(0, 0.3, C).astype(np.float32)
    var = rng.uniform(0.5, 2.0, C).astype(np.float32)
    rd = 3.0
    bshape = [1] * len(shape)
    bshape[axis] = C
    real = d.astype(np.float64) * rd / 127.5
    want = (real - mean.reshape(bshape)) / np.sqrt(var.reshape(bshape) + 1e-3) * \
        gamma.reshape(bshape) + beta.reshape(bshape)
    R = float(np.abs(want).max())
    out, mn, mx = qref.quantized_batch_norm(d, gamma, beta, mean, var, -rd, rd, -R, R, eps=1e-3,
                                            axis=axis)
    back = out.astype(np.float64) * R / 127.5
    assert np.abs(back - want).max() <= 1.5 * R / 127.5 + 1e-3 * R
    relu, _, _ = qref.quantized_batch_norm(d, gamma, beta, mean, var, -rd, rd, -R, R, eps=1e-3,
                                           axis=axis, relu=True)
    assert np.array_equal(relu, np.maximum(out, 0))
    with pytest.raises(ValueError):
        qref.quantized_batch_norm(d, gamma, beta, mean, var, -rd, rd, None, None)
