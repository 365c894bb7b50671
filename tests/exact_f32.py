"""Exact model of IEEE-754 binary32 arithmetic on Python rationals, used to pin the
oracle: every operation is computed exactly with fractions.Fraction and then rounded
once to the nearest binary32 (ties to even) by integer arithmetic.  Shares no code
with numpy's or the C compiler's float arithmetic."""
from fractions import Fraction

EMIN, EMAX, P = -126, 127, 24


def fl32(q):
    """Round the exact rational q to binary32 (ties-to-even); returns a Fraction."""
    q = Fraction(q)
    if q == 0:
        return Fraction(0)
    sign = -1 if q < 0 else 1
    a = abs(q)
    # exponent e with 2^e <= a < 2^(e+1)
    e = a.numerator.bit_length() - a.denominator.bit_length()
    if Fraction(2) ** e > a:
        e -= 1
    if Fraction(2) ** (e + 1) <= a:
        e += 1
    e = max(e, EMIN)                      # subnormals share the minimum exponent
    ulp = Fraction(2) ** (e - (P - 1))
    m = a / ulp                           # mantissa in units of ulp
    lo = m.numerator // m.denominator
    rem = m - lo
    if rem > Fraction(1, 2) or (rem == Fraction(1, 2) and lo % 2 == 1):
        lo += 1
    r = lo * ulp
    if r >= Fraction(2) ** (EMAX + 1):
        raise OverflowError("binary32 overflow")
    return sign * r


def f(x):
    """A float that is already a binary32 value -> exact Fraction."""
    return Fraction(float(x))


def trunc(q):
    return int(q)  # Fraction -> int truncates toward zero


def quantize_int8(x, lo, hi):
    """quantization_utils.h:83-89 / quantize_v2-inl.h:98-114, one rounding per operation."""
    R = max(abs(f(lo)), abs(f(hi)))
    s = fl32(Fraction(127) / R)
    x = f(x)
    t = fl32(abs(x) * s)
    u = fl32(t + Fraction(1, 2))
    v = min(u, Fraction(127))
    sign = (x > 0) - (x < 0)
    return trunc(sign * v), -R, R


def quantize_uint8(x, lo, hi):
    """quantize_v2-inl.h:66-81: double division narrowed to float, float product,
    double add, truncation."""
    lo, hi, x = f(lo), f(hi), f(x)
    d = fl32(hi - lo)
    s = fl32(fl64(Fraction(255) / d))
    t = fl32(fl32(x - lo) * s)
    u = fl64(t + Fraction(1, 2))
    return trunc(u)


def fl64(q):
    """Same rounding to binary64 (only used where the reference computes in double)."""
    q = Fraction(q)
    if q == 0:
        return q
    sign = -1 if q < 0 else 1
    a = abs(q)
    e = a.numerator.bit_length() - a.denominator.bit_length()
    if Fraction(2) ** e > a:
        e -= 1
    if Fraction(2) ** (e + 1) <= a:
        e += 1
    e = max(e, -1022)
    ulp = Fraction(2) ** (e - 52)
    m = a / ulp
    lo = m.numerator // m.denominator
    rem = m - lo
    if rem > Fraction(1, 2) or (rem == Fraction(1, 2) and lo % 2 == 1):
        lo += 1
    return sign * lo * ulp


def i32_to_float(q, lo, hi):
    """quantization_utils.h:91-97 for int32: float(q) * (MaxAbs / 2^31)."""
    R = max(abs(f(lo)), abs(f(hi)))
    scale = fl32(R / Fraction(2) ** 31)
    return fl32(fl32(Fraction(int(q))) * scale)


def requantize(q, lo, hi, real_range):
    x = i32_to_float(q, lo, hi)
    rr = abs(f(real_range))
    s = fl32(Fraction(127) / rr)
    t = fl32(abs(x) * s)
    u = fl32(t + Fraction(1, 2))
    v = min(u, Fraction(127))
    sign = (x > 0) - (x < 0)
    return trunc(sign * v)


def dequantize_int8(q, lo, hi):
    R = max(abs(f(hi)), abs(f(lo)))
    return fl32(Fraction(int(q)) * fl32(R / Fraction(127)))


def dequantize_uint8(q, lo, hi):
    lo, hi = f(lo), f(hi)
    s = fl32(fl32(hi - lo) / Fraction(255))
    return fl32(fl32(Fraction(int(q)) * s) + lo)


def range_for_multiplication(min_a, max_a, min_b, max_b):
    a = fl32(max(abs(f(min_a)), abs(f(max_a))) / Fraction(127))
    b = fl32(max(abs(f(min_b)), abs(f(max_b))) / Fraction(127))
    c = fl32(a * b)
    return fl32(c * Fraction(2) ** 31)


def bias_i8_to_i32(b, min_out, max_out, min_bias, max_bias):
    """quantized_fully_connected.cc:149-174"""
    one_out = fl32(fl64(max(abs(f(min_out)), abs(f(max_out))) / Fraction(2 ** 31 - 1)))
    one_bias = fl32(fl64(max(abs(f(min_bias)), abs(f(max_bias))) / Fraction(127)))
    if one_out == 0:
        return 0
    p = fl32(Fraction(int(b)) * one_bias)
    return trunc(fl32(p / one_out))
