"""_contrib_quantized_elemwise_add and _contrib_quantized_concat on the GPU, called through
the operator host and the C ABI: the reference's operator test restated
(tests/python/quantization/test_quantization.py:375-433: the dequantized int32 sum is within
2 of the float sum) and bit-exact comparison with the oracle over the four operand type
pairs, calibrated and not, ragged and unaligned sizes, every concat axis, mixed types and
more inputs than one range launch takes."""
import ctypes

import numpy as np
import pytest
import torch

import oracle

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def contrib():
    import mxnet_amd
    return mxnet_amd.contrib


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def scalar(v):
    return dev(np.array([v], np.float32))


def host(t):
    return t.cpu().numpy()


def draw(rng, dtype, shape):
    lo, hi = (0, 256) if dtype == np.uint8 else (-128, 128)
    return rng.integers(lo, hi, shape).astype(dtype)


@pytest.mark.parametrize("shape,ta,tb", [((4, 6), np.uint8, np.int8),
                                         ((13, 74, 52), np.uint8, np.uint8),
                                         ((3, 4, 56, 56), np.int8, np.uint8),
                                         ((32, 56, 64, 11), np.int8, np.int8)])
def test_reference_quantized_elemwise_add(contrib, shape, ta, tb):
    rng = np.random.default_rng(21)
    rng_of = lambda t: (0.0, 255.0) if t == np.uint8 else (-127.0, 127.0)
    (alo, ahi), (blo, bhi) = rng_of(ta), rng_of(tb)
    a = rng.uniform(alo, ahi, size=shape).astype(np.int32).astype(ta)
    b = rng.uniform(blo, bhi, size=shape).astype(np.int32).astype(tb)
    out, mn, mx = contrib.quantized_elemwise_add(dev(a), dev(b), scalar(alo), scalar(ahi),
                                                 scalar(blo), scalar(bhi))
    assert out.dtype == torch.int32 and tuple(out.shape) == shape
    back = host(out).astype(np.float32) * host(mx)[0] / np.float32(0x7fffffff)
    assert np.abs(back - (a.astype(np.float32) + b.astype(np.float32))).max() <= 2
    ref, rmn, rmx = oracle.quantized_elemwise_add(a, b, alo, ahi, blo, bhi)
    np.testing.assert_array_equal(host(out), ref)
    assert host(mn)[0] == rmn and host(mx)[0] == rmx


@pytest.mark.parametrize("ta,tb", [(np.int8, np.int8), (np.uint8, np.uint8),
                                   (np.int8, np.uint8), (np.uint8, np.int8)])
@pytest.mark.parametrize("calib", [None, (-3.0, 2.5), (-0.4, 0.7)])
@pytest.mark.parametrize("n", [1, 3, 17, 4099, (1 << 20) + 5])
def test_elemwise_add_matches_oracle(contrib, ta, tb, calib, n):
    rng = np.random.default_rng(n)
    a, b = draw(rng, ta, n), draw(rng, tb, n)
    rngs = (-1.3, 0.9, -0.2, 2.2)
    kw = {} if calib is None else {"min_calib_range": calib[0], "max_calib_range": calib[1]}
    out, mn, mx = contrib.quantized_elemwise_add(dev(a), dev(b), *[scalar(v) for v in rngs], **kw)
    ref, rmn, rmx = oracle.quantized_elemwise_add(a, b, *rngs, **kw)
    assert host(out).dtype == ref.dtype
    np.testing.assert_array_equal(host(out), ref)
    assert host(mn)[0] == rmn and host(mx)[0] == rmx


@pytest.mark.parametrize("calibrated", [False, True])
def test_elemwise_add_unaligned_views(contrib, calibrated):
    """Operands that start 1..3 bytes into an allocation take the element-wise path."""
    rng = np.random.default_rng(8)
    base_a, base_b = draw(rng, np.int8, 5003), draw(rng, np.int8, 5003)
    kw = {"min_calib_range": -2.0, "max_calib_range": 2.0} if calibrated else {}
    da, db = dev(base_a), dev(base_b)
    for oa, ob in ((1, 0), (0, 3), (2, 2), (16, 16)):
        n = 4900
        out, _, _ = contrib.quantized_elemwise_add(da[oa:oa + n], db[ob:ob + n], scalar(-1.0),
                                                   scalar(1.0), scalar(-1.5), scalar(0.5), **kw)
        ref, _, _ = oracle.quantized_elemwise_add(base_a[oa:oa + n], base_b[ob:ob + n], -1.0,
                                                  1.0, -1.5, 0.5, **kw)
        np.testing.assert_array_equal(host(out), ref)


def test_elemwise_add_saturation_and_empty(contrib):
    a = np.array([127, -127, 0, 127, -128], np.int8)
    b = np.array([127, -127, 0, -127, -128], np.int8)
    out, _, _ = contrib.quantized_elemwise_add(dev(a), dev(b), scalar(-1.0), scalar(1.0),
                                               scalar(-1.0), scalar(1.0), min_calib_range=-0.5,
                                               max_calib_range=0.5)
    np.testing.assert_array_equal(host(out), np.array([127, -128, 0, 0, -128], np.int8))
    e = dev(np.zeros((0, 4), np.int8))
    out, mn, mx = contrib.quantized_elemwise_add(e, e, scalar(-1.0), scalar(1.0), scalar(-2.0),
                                                 scalar(1.0))
    assert tuple(out.shape) == (0, 4) and host(mx)[0] == np.float32(3.0)


def test_elemwise_add_c_abi_rejects_wrong_types():
    import mxnet_amd
    lib = mxnet_amd._lib.lib
    P = lambda t: ctypes.c_void_p(t.data_ptr())
    a = dev(np.zeros(16, np.int8))
    o = torch.empty(16, dtype=torch.int32, device="cuda")
    s = [scalar(1.0) for _ in range(6)]
    st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    I8, I32, F32 = 5, 4, 0
    # int8 output asked for without calibration
    rc = lib.mxq_quantized_elemwise_add(st, P(a), I8, P(a), I8, P(s[0]), P(s[1]), P(s[2]),
                                        P(s[3]), P(o), I8, P(s[4]), P(s[5]), 16, 0, 0.0, 0.0)
    assert rc == -1 and b"output type" in lib.mxq_last_error()
    rc = lib.mxq_quantized_elemwise_add(st, P(a), F32, P(a), I8, P(s[0]), P(s[1]), P(s[2]),
                                        P(s[3]), P(o), I32, P(s[4]), P(s[5]), 16, 0, 0.0, 0.0)
    assert rc == -1 and b"int8 or uint8" in lib.mxq_last_error()
    rc = lib.mxq_quantized_elemwise_add(st, P(a), I8, P(a), I8, None, P(s[1]), P(s[2]),
                                        P(s[3]), P(o), I32, P(s[4]), P(s[5]), 16, 0, 0.0, 0.0)
    assert rc == -1 and b"null range" in lib.mxq_last_error()


# ---- concat ------------------------------------------------------------------------------

def run_concat(contrib, xs, mins, maxs, dim):
    args = [dev(x) for x in xs]
    for lo, hi in zip(mins, maxs):
        args += [scalar(lo), scalar(hi)]
    out, mn, mx = contrib.quantized_concat(*args, num_args=len(xs), dim=dim)
    ref, rmn, rmx = oracle.quantized_concat(xs, mins, maxs, dim=dim)
    assert host(out).dtype == ref.dtype and tuple(out.shape) == ref.shape
    np.testing.assert_array_equal(host(out), ref)
    assert host(mn)[0] == rmn and host(mx)[0] == rmx
    return host(out)


@pytest.mark.parametrize("dim", [0, 1, 2, 3, -1])
@pytest.mark.parametrize("base", [(2, 3, 4, 5), (4, 16, 8, 16), (1, 64, 7, 32)])
def test_concat_matches_oracle_on_every_axis(contrib, dim, base):
    rng = np.random.default_rng(31)
    xs = []
    for extent in (base[dim], 2 * base[dim], 1):
        s = list(base)
        s[dim] = extent
        xs.append(draw(rng, np.int8, s))
    run_concat(contrib, xs, [-1.0, -0.25, -3.0], [0.5, 0.3, 4.0], dim)


def test_concat_equal_ranges_copies_bytes(contrib):
    rng = np.random.default_rng(32)
    xs = [draw(rng, np.int8, (8, c, 14, 14)) for c in (32, 64, 16)]
    out = run_concat(contrib, xs, [-2.0] * 3, [2.0] * 3, 1)
    np.testing.assert_array_equal(out, np.concatenate(xs, axis=1))
    us = [draw(rng, np.uint8, (5, 33)) for _ in range(2)]
    out = run_concat(contrib, us, [0.0, 0.0], [1.0, 1.0], 1)
    np.testing.assert_array_equal(out, np.concatenate(us, axis=1))


def test_concat_mixed_types_and_one_sided_ranges(contrib):
    rng = np.random.default_rng(33)
    u, s = draw(rng, np.uint8, (3, 40, 5)), draw(rng, np.int8, (3, 24, 5))
    run_concat(contrib, [u, s], [0.0, -1.0], [1.0, 1.0], 1)
    run_concat(contrib, [s, u, s], [-0.5, 0.0, -2.0], [0.5, 3.0, 1.0], 1)
    run_concat(contrib, [u, u], [0.5, 0.25], [1.0, 2.0], 1)   # the hull includes 0


def test_concat_many_inputs_single_input_and_empty_part(contrib):
    rng = np.random.default_rng(34)
    xs = [draw(rng, np.int8, (2, 1 + i % 3, 6)) for i in range(19)]
    mins = [-0.1 * (i + 1) for i in range(19)]
    maxs = [0.07 * (i + 2) for i in range(19)]
    run_concat(contrib, xs, mins, maxs, 1)
    run_concat(contrib, xs[:1], mins[:1], maxs[:1], 1)
    xs[1] = np.zeros((2, 0, 6), np.int8)
    run_concat(contrib, xs[:3], mins[:3], maxs[:3], 1)


def test_concat_large_rows_and_unaligned_pitch(contrib):
    rng = np.random.default_rng(35)
    # 16-byte aligned slabs (vector path) and slabs whose pitch breaks the alignment
    run_concat(contrib, [draw(rng, np.int8, (64, 256, 64)), draw(rng, np.int8, (64, 128, 64))],
               [-1.0, -2.0], [1.0, 2.0], 1)
    run_concat(contrib, [draw(rng, np.int8, (37, 48)), draw(rng, np.int8, (37, 23))],
               [-1.0, -2.0], [1.0, 2.0], 1)
    run_concat(contrib, [draw(rng, np.int8, (1 << 21,)), draw(rng, np.int8, (1 << 20,))],
               [-1.0, -2.0], [1.0, 2.0], 0)


def test_concat_c_abi_rejects_bad_arguments():
    import mxnet_amd
    lib = mxnet_amd._lib.lib
    a = dev(np.zeros((2, 4), np.int8))
    o = torch.empty((2, 8), dtype=torch.int8, device="cuda")
    lo, hi, omn, omx = (scalar(v) for v in (-1.0, 1.0, 0.0, 0.0))
    st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    ptrs = (ctypes.c_void_p * 2)(a.data_ptr(), a.data_ptr())
    mins = (ctypes.c_void_p * 2)(lo.data_ptr(), lo.data_ptr())
    maxs = (ctypes.c_void_p * 2)(hi.data_ptr(), hi.data_ptr())
    ext = (ctypes.c_int64 * 2)(4, 4)
    P = lambda t: ctypes.c_void_p(t.data_ptr())
    types = (ctypes.c_int * 2)(5, 5)
    # uint8 output although the inputs are int8
    rc = lib.mxq_quantized_concat(st, 2, ptrs, types, mins, maxs, ext, 2, 1, P(o), 3, P(omn),
                                  P(omx))
    assert rc == -1 and b"output type" in lib.mxq_last_error()
    types = (ctypes.c_int * 2)(5, 0)
    rc = lib.mxq_quantized_concat(st, 2, ptrs, types, mins, maxs, ext, 2, 1, P(o), 5, P(omn),
                                  P(omx))
    assert rc == -1 and b"int8 or uint8" in lib.mxq_last_error()
    rc = lib.mxq_quantized_concat(st, 0, ptrs, types, mins, maxs, ext, 2, 1, P(o), 5, P(omn),
                                  P(omx))
    assert rc == -1 and b"at least one" in lib.mxq_last_error()


# ---- quantized_npi_add (broadcasting) -------------------------------------------------------

BROADCAST_SHAPES = [((4, 6), (1, 1)), ((1, 1, 1), (13, 74, 52)), ((3, 4, 56, 56), (1, 4, 1, 1)),
                    ((32, 56, 64), (64,)), ((8, 1, 48), (1, 5, 1)), ((2, 3, 16, 32), (3, 1, 32)),
                    ((7, 33), (7, 1)), ((5, 1, 4, 1, 16), (1, 3, 1, 2, 16)), ((6,), ()),
                    ((0, 4), (1, 4)), ((64, 256), (64, 256)),
                    # innermost runs of 1 KiB and more: the wave-per-run kernel, ragged pieces
                    ((3, 5, 1040), (5, 1)), ((4, 2, 4112), (1, 2, 4112)), ((2, 3, 2048), (3, 1)),
                    ((2, 1, 1024), (1, 3, 1024)), ((1, 1), (3, 5136))]


@pytest.mark.parametrize("sa,sb", BROADCAST_SHAPES)
@pytest.mark.parametrize("ta,tb", [(np.int8, np.int8), (np.uint8, np.uint8),
                                   (np.int8, np.uint8), (np.uint8, np.int8)])
@pytest.mark.parametrize("calib", [None, (-3.0, 2.5)])
def test_quantized_npi_add_matches_oracle(sa, sb, ta, tb, calib):
    import mxnet_amd
    rng = np.random.default_rng(len(sa) * 7 + len(sb))
    a = rng.integers(*((0, 256) if ta == np.uint8 else (-128, 128)), sa).astype(ta)
    b = rng.integers(*((0, 256) if tb == np.uint8 else (-128, 128)), sb).astype(tb)
    amin, amax, bmin, bmax = -1.3, 0.9, -0.2, 2.2
    kw = {} if calib is None else {"min_calib_range": calib[0], "max_calib_range": calib[1]}
    f32 = lambda v: torch.tensor([v], dtype=torch.float32, device="cuda")
    dev = lambda x: torch.from_numpy(np.require(x, requirements="C")).cuda()
    out, mn, mx = mxnet_amd.contrib.quantized_npi_add(dev(a), dev(b), f32(amin), f32(amax),
                                                      f32(bmin), f32(bmax), **kw)
    ref, rmn, rmx = oracle.quantized_npi_add(a, b, amin, amax, bmin, bmax, **kw)
    assert tuple(out.shape) == ref.shape
    got = out.cpu().numpy()
    assert got.dtype == ref.dtype
    np.testing.assert_array_equal(got, ref)
    assert (mn.item(), mx.item()) == (rmn, rmx)


def test_quantized_npi_add_refuses_shapes_that_do_not_broadcast():
    import mxnet_amd
    a = torch.zeros((3, 4), dtype=torch.int8, device="cuda")
    b = torch.zeros((3, 5), dtype=torch.int8, device="cuda")
    s = torch.ones(1, device="cuda")
    with pytest.raises(mxnet_amd.operator.MXNetError, match="broadcast"):
        mxnet_amd.contrib.quantized_npi_add(a, b, s, s, s, s)
