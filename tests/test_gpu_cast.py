"""Parity of the HIP quantize / requantize / dequantize kernels with the CPU
oracle, through the C ABI.  Bit-exact for int8/uint8 and the range scalars;
dequantized fp32 within 1e-6 relative (it is in fact bit-exact, also asserted)."""
import numpy as np
import pytest
import torch

import oracle
from tests.data_gen import int32_uniform, int8_uniform, normal_with_outliers

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def capi():
    import mxnet_amd
    return mxnet_amd.capi


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


SIZES = [1, 3, 4, 5, 63, 64, 255, 1024, 4097, 65536 + 7, (1 << 20) + 13, 5_000_003]


@pytest.mark.parametrize("n", SIZES)
@pytest.mark.parametrize("calib", [None, (-50.0, 50.0), (-4.0, 4.0), (-0.37, 2.9)])
def test_quantize_v2_int8(capi, n, calib):
    x = normal_with_outliers(n, seed=n % 97 + 1)
    kw = {} if calib is None else dict(min_calib_range=calib[0], max_calib_range=calib[1])
    q, mn, mx = capi.quantize_v2(dev(x), "int8", **kw)
    rq, rmn, rmx = oracle.quantize_v2(x, "int8", **kw)
    assert q.dtype == torch.int8
    np.testing.assert_array_equal(q.cpu().numpy(), rq)
    assert mn.item() == rmn and mx.item() == rmx


@pytest.mark.parametrize("n", SIZES)
@pytest.mark.parametrize("calibrated", [False, True])
def test_quantize_v2_uint8(capi, n, calibrated):
    x = normal_with_outliers(n, seed=n % 89 + 2, dist="laplace")
    kw = {}
    if calibrated:
        kw = dict(min_calib_range=float(x.min()), max_calib_range=float(x.max()))
        if kw["min_calib_range"] == kw["max_calib_range"]:
            kw["max_calib_range"] += 1.0
    elif n == 1:
        pytest.skip("min == max: zero range divides by zero in the reference too")
    q, mn, mx = capi.quantize_v2(dev(x), "uint8", **kw)
    rq, rmn, rmx = oracle.quantize_v2(x, "uint8", **kw)
    assert q.dtype == torch.uint8
    np.testing.assert_array_equal(q.cpu().numpy(), rq)
    assert mn.item() == rmn and mx.item() == rmx


def test_quantize_v2_auto_and_ties(capi):
    # exact .5 ties: x = (j + 0.5)/127 * R is not always representable; use R = 127
    j = np.arange(-130, 131, dtype=np.float32)
    x = np.concatenate([j + 0.5, j - 0.5, j, np.array([0.0, -0.0], np.float32)])
    q, mn, mx = capi.quantize_v2(dev(x), "auto", min_calib_range=-127.0, max_calib_range=127.0)
    rq, rmn, rmx = oracle.quantize_v2(x, "auto", -127.0, 127.0)
    assert q.dtype == torch.int8
    np.testing.assert_array_equal(q.cpu().numpy(), rq)
    q, mn, mx = capi.quantize_v2(dev(np.abs(x)), "auto", min_calib_range=0.0,
                                 max_calib_range=130.5)
    rq, rmn, rmx = oracle.quantize_v2(np.abs(x), "auto", 0.0, 130.5)
    assert q.dtype == torch.uint8
    np.testing.assert_array_equal(q.cpu().numpy(), rq)
    assert (mn.item(), mx.item()) == (rmn, rmx)


def test_quantize_v2_nan_propagates(capi):
    x = normal_with_outliers(100_000, seed=5)
    x[77_777] = np.nan
    q, mn, mx = capi.quantize_v2(dev(x), "int8")
    assert np.isnan(mn.item()) and np.isnan(mx.item())


def test_quantize_v2_unaligned_views(capi):
    x = normal_with_outliers(100_003, seed=9)
    base = dev(x)
    for off in (1, 2, 3):
        v = base[off:]
        q, mn, mx = capi.quantize_v2(v, "int8")
        rq, rmn, rmx = oracle.quantize_v2(x[off:], "int8")
        np.testing.assert_array_equal(q.cpu().numpy(), rq)
        assert (mn.item(), mx.item()) == (rmn, rmx)


def test_quantize_v1(capi):
    x = normal_with_outliers(300_001, seed=11)
    lo, hi = np.float32(x.min()), np.float32(x.max())
    for ot in ("int8", "uint8"):
        q, mn, mx = capi.quantize(dev(x), dev(np.array([lo])), dev(np.array([hi])), ot)
        rq, rmn, rmx = oracle.quantize(x, lo, hi, ot)
        np.testing.assert_array_equal(q.cpu().numpy(), rq)
        assert (mn.item(), mx.item()) == (rmn, rmx)


@pytest.mark.parametrize("n", SIZES)
@pytest.mark.parametrize("calib", [None, (-0.3, 0.25), (-134.349, 523.43)])
def test_requantize(capi, n, calib):
    x = int32_uniform(n, seed=n % 83 + 3)
    imin, imax = np.float32(-3.7), np.float32(4.1)
    kw = {} if calib is None else dict(min_calib_range=calib[0], max_calib_range=calib[1])
    q, mn, mx = capi.requantize(dev(x), dev(np.array([imin])), dev(np.array([imax])), **kw)
    rq, rmn, rmx = oracle.requantize(x, imin, imax, **kw)
    np.testing.assert_array_equal(q.cpu().numpy(), rq)
    assert (mn.item(), mx.item()) == (rmn, rmx)


def test_requantize_reference_test_shapes(capi):
    # tests/python/quantization/test_quantization.py:146-235
    for shape, calib in [((3, 4, 10, 10), None), ((32, 3, 23, 23), None),
                         ((3, 4, 10, 10), (-1050.0, 1040.0)),
                         ((32, 3, 23, 23), (-134.349, 523.43))]:
        rng = np.random.default_rng(7)
        x = rng.uniform(-1000.0, 1000.0, size=shape).astype(np.int32)
        kw = {} if calib is None else dict(min_calib_range=calib[0], max_calib_range=calib[1])
        q, mn, mx = capi.requantize(dev(x), dev(np.array([-1010.0], np.float32)),
                                    dev(np.array([1020.0], np.float32)), **kw)
        rq, rmn, rmx = oracle.requantize(x, -1010.0, 1020.0, **kw)
        np.testing.assert_array_equal(q.cpu().numpy(), rq)
        assert (mn.item(), mx.item()) == (rmn, rmx)


def test_requantize_extremes(capi):
    x = np.array([np.iinfo(np.int32).min, np.iinfo(np.int32).max, 0, 1, -1, 1 << 24,
                  (1 << 24) + 1, -(1 << 24) - 1], np.int32)
    for calib in (None, (-4.0, 4.0)):
        kw = {} if calib is None else dict(min_calib_range=calib[0], max_calib_range=calib[1])
        q, mn, mx = capi.requantize(dev(x), dev(np.array([-10651.54], np.float32)),
                                    dev(np.array([10651.54], np.float32)), **kw)
        rq, rmn, rmx = oracle.requantize(x, -10651.54, 10651.54, **kw)
        np.testing.assert_array_equal(q.cpu().numpy(), rq)
        assert (mn.item(), mx.item()) == (rmn, rmx)


@pytest.mark.parametrize("n", SIZES)
@pytest.mark.parametrize("dtype", ["int8", "uint8"])
def test_dequantize(capi, n, dtype):
    if dtype == "int8":
        q = int8_uniform(n, seed=n % 79 + 4)
        lo, hi = np.float32(-2.73), np.float32(2.5)
    else:
        q = np.random.default_rng(n % 71 + 5).integers(0, 256, size=n, dtype=np.uint8)
        lo, hi = np.float32(-0.61), np.float32(3.3)
    y = capi.dequantize(dev(q), dev(np.array([lo])), dev(np.array([hi])))
    ry = oracle.dequantize(q, lo, hi)
    got = y.cpu().numpy()
    np.testing.assert_allclose(got, ry, rtol=1e-6, atol=0)
    np.testing.assert_array_equal(got.view(np.uint32), ry.view(np.uint32))


def test_roundtrip_properties_large(capi):
    """Size-independent properties at a large size (16M elements)."""
    n = 1 << 24
    g = torch.Generator(device="cuda").manual_seed(3)
    x = torch.randn(n, device="cuda", generator=g)
    q, mn, mx = capi.quantize_v2(x, "int8")
    r = mx.item()
    assert mn.item() == -r and r == x.abs().max().item()
    assert int(q.abs().max()) == 127 and int(q.min()) >= -127
    # odd symmetry
    q2, _, _ = capi.quantize_v2(-x, "int8")
    assert torch.equal(q2, -q)
    # dequantize(quantize(x)) is within half a level
    y = capi.dequantize(q, mn, mx)
    assert float((y - x).abs().max()) <= r / 254 * (1 + 1e-5)
    # calibrated with the observed range equals uncalibrated
    q3, _, _ = capi.quantize_v2(x, "int8", min_calib_range=-r, max_calib_range=r)
    assert torch.equal(q3, q)
    # monotone: sort order is preserved
    xs, _ = torch.sort(x[: 1 << 20])
    qs, _, _ = capi.quantize_v2(xs, "int8", min_calib_range=-r, max_calib_range=r)
    assert bool((qs[1:] >= qs[:-1]).all())


def test_empty_and_errors(capi):
    import mxnet_amd
    e = torch.empty(0, dtype=torch.float32, device="cuda")
    q, mn, mx = capi.quantize_v2(e, "int8", min_calib_range=-1.0, max_calib_range=1.0)
    assert q.numel() == 0
    lib = mxnet_amd._lib.lib
    x = torch.zeros(16, device="cuda")
    out = torch.zeros(16, dtype=torch.int8, device="cuda")
    s = torch.zeros(2, device="cuda")
    # bad out_type
    rc = lib.mxq_quantize_v2(None, x.data_ptr(), out.data_ptr(), s.data_ptr(),
                             s[1:].data_ptr(), 16, 4, 1, -1.0, 1.0, None, 0)
    assert rc == -1 and "int8 and uint8" in mxnet_amd._lib.last_error()
    # uncalibrated without a workspace
    rc = lib.mxq_quantize_v2(None, x.data_ptr(), out.data_ptr(), s.data_ptr(),
                             s[1:].data_ptr(), 16, 5, 0, 0.0, 0.0, None, 0)
    assert rc == -1 and "workspace" in mxnet_amd._lib.last_error()
    torch.cuda.synchronize()
