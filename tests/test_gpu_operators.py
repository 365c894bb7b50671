"""The operators driven through the C++ operator host under the reference's names,
restating the reference's own operator tests
(tests/python/quantization/test_quantization.py:66-235, 238-371, 661-808) with
their numpy baselines and tolerances, plus bit-exact comparison with the oracle."""
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


def rand_shape_nd(rng, ndim, dim=10):
    return tuple(int(x) for x in rng.integers(1, dim + 1, size=ndim))


def test_quantize_float32_to_int8(contrib):
    # test_quantization.py:66-84 (v1 operator, ranges are inputs)
    rng = np.random.default_rng(0)
    for _ in range(5):
        shape = rand_shape_nd(rng, 4)
        data = rng.uniform(-1.0, 1.0, size=shape).astype(np.float32)
        lo, hi = data.min(), data.max()
        qdata, mn, mx = contrib.quantize(dev(data), scalar(lo), scalar(hi), out_type="int8")
        real_range = np.maximum(np.abs(lo), np.abs(hi))
        scale = 127.0 / real_range
        assert qdata.dtype == torch.int8 and mn.dtype == torch.float32
        assert mn.item() == -real_range and mx.item() == real_range
        base = (np.sign(data) * np.minimum(np.abs(data) * scale + 0.5, 127.0)).astype(np.int8)
        np.testing.assert_allclose(qdata.cpu().numpy(), base, atol=1)
        ref, rmn, rmx = oracle.quantize(data, lo, hi, "int8")
        np.testing.assert_array_equal(qdata.cpu().numpy(), ref)


def test_calibrated_quantize_v2_to_int8(contrib):
    # test_quantization.py:86-102 with fp32 data (bfloat16 input is oneDNN-only)
    rng = np.random.default_rng(1)
    shape = rand_shape_nd(rng, 4)
    data = rng.standard_normal(shape).astype(np.float32)
    lo, hi = float(data.min()), float(data.max())
    qdata, mn, mx = contrib.quantize_v2(dev(data), "int8", lo, hi)
    real_range = np.float32(max(abs(lo), abs(hi)))
    assert mn.item() == -real_range and mx.item() == real_range
    base = (np.sign(data) * np.minimum(np.abs(data) * (127.0 / real_range) + 0.5, 127.0)
            ).astype(np.int8)
    np.testing.assert_allclose(qdata.cpu().numpy(), base, atol=1)
    np.testing.assert_array_equal(qdata.cpu().numpy(), oracle.quantize_v2(data, "int8", lo, hi)[0])


def test_quantize_v2_int8_input_passthrough(contrib):
    # quantize_v2-inl.h:203-216
    q = np.random.default_rng(2).integers(-127, 128, size=(7, 9), dtype=np.int8)
    out, mn, mx = contrib.quantize_v2(dev(q), "int8")
    np.testing.assert_array_equal(out.cpu().numpy(), q)
    assert (mn.item(), mx.item()) == (-127.0, 127.0)
    out, mn, mx = contrib.quantize_v2(dev(q), "int8", -3.0, 2.0)
    assert (mn.item(), mx.item()) == (-3.0, 2.0)
    u = q.view(np.uint8)
    out, mn, mx = contrib.quantize_v2(dev(u), "auto", 0.0, 4.0)
    assert out.dtype == torch.uint8 and (mn.item(), mx.item()) == (0.0, 4.0)


def test_dequantize_int8_to_float32(contrib):
    # test_quantization.py:104-143
    rng = np.random.default_rng(3)
    real_range = 128
    shape = rand_shape_nd(rng, 4)
    q = rng.uniform(-127, 127, size=shape).astype(np.int8)
    out = contrib.dequantize(dev(q), scalar(-real_range), scalar(real_range), out_type="float32")
    assert out.dtype == torch.float32
    np.testing.assert_allclose(out.cpu().numpy(), q * (real_range / 127.0), atol=1)
    np.testing.assert_allclose(out.cpu().numpy(), oracle.dequantize(q, -real_range, real_range),
                               rtol=1e-6, atol=0)


def test_requantize_int32_to_int8(contrib):
    # test_quantization.py:146-235
    def baseline(q, lo, hi, calib):
        def to_float(x):
            return x.astype("float32") * (float(max(abs(lo), abs(hi))) / float(np.iinfo("int32").max))
        if calib is not None:
            rr = max(abs(calib[0]), abs(calib[1]))
        else:
            rr = max(abs(to_float(np.min(q))), abs(to_float(np.max(q))))
        f = to_float(q)
        out = (np.sign(f) * np.minimum(np.abs(f) * (127.0 / float(rr)) + 0.5, 127)).astype("int8")
        return out, -rr, rr

    rng = np.random.default_rng(4)
    for shape, calib in [((3, 4, 10, 10), None), ((32, 3, 23, 23), None),
                         ((3, 4, 10, 10), (-1050.0, 1040.0)),
                         ((32, 3, 23, 23), (-134.349, 523.43))]:
        q = rng.uniform(-1000.0, 1000.0, size=shape).astype(np.int32)
        kw = {} if calib is None else dict(min_calib_range=calib[0], max_calib_range=calib[1])
        out, mn, mx = contrib.requantize(dev(q), scalar(-1010.0), scalar(1020.0), **kw)
        b, bmn, bmx = baseline(q, -1010.0, 1020.0, calib)
        np.testing.assert_allclose(out.cpu().numpy(), b, atol=1)
        np.testing.assert_allclose(mn.item(), bmn, rtol=1e-5)
        np.testing.assert_allclose(mx.item(), bmx, rtol=1e-5)
        ref, rmn, rmx = oracle.requantize(q, -1010.0, 1020.0, **kw)
        np.testing.assert_array_equal(out.cpu().numpy(), ref)
        assert (mn.item(), mx.item()) == (rmn, rmx)


@pytest.mark.parametrize("data_shape,num_hidden,use_bias",
                         [((32, 512, 2, 2), 100, False), ((32, 111, 2, 2), 100, False),
                          ((32, 512, 2, 2), 100, True), ((32, 111, 2, 2), 100, True),
                          ((256, 2048, 2, 2), 800, True), ((256, 111, 2, 2), 800, True),
                          ((256, 2048, 2, 2), 800, False), ((256, 111, 2, 2), 800, False)])
def test_quantized_fc(contrib, data_shape, num_hidden, use_bias):
    # test_quantization.py:661-808: integer-valued fp32 Dense is the baseline
    rng = np.random.default_rng(5)
    data = rng.uniform(-63.0, 63.0, size=data_shape).astype(np.int32).astype(np.float32)
    K = int(np.prod(data_shape[1:]))
    weight = rng.uniform(-63.0, 63.0, size=(num_hidden, K)).astype(np.int32).astype(np.float32)
    data_range = float(np.abs(data).max())
    weight_range = float(np.abs(weight).max())
    want = data.reshape(data_shape[0], -1).astype(np.float64) @ weight.astype(np.float64).T
    args = dict(num_hidden=num_hidden, no_bias=not use_bias, flatten=True)
    bias = None
    if use_bias:
        bias = rng.uniform(-63.0, 63.0, size=(num_hidden,)).astype(np.int32).astype(np.float32)
        bias_range = float(np.abs(bias).max())
        bias_int32_rescale = (127.0 / data_range) * (127.0 / weight_range) / (127.0 / bias_range)
        want = want + (bias * bias_int32_rescale).astype(np.int32).astype(np.float64)
        out, mn, mx = contrib.quantized_fully_connected(
            dev(data.astype(np.int8)), dev(weight.astype(np.int8)), dev(bias.astype(np.int8)),
            scalar(-data_range), scalar(data_range), scalar(-weight_range), scalar(weight_range),
            scalar(-bias_range), scalar(bias_range), **args)
    else:
        out, mn, mx = contrib.quantized_fully_connected(
            dev(data.astype(np.int8)), dev(weight.astype(np.int8)), None, scalar(-data_range),
            scalar(data_range), scalar(-weight_range), scalar(weight_range), **args)
    assert out.dtype == torch.int32 and tuple(out.shape) == (data_shape[0], num_hidden)
    got = out.cpu().numpy()
    if use_bias:
        assert int((np.abs(want - got) > 2).sum()) == 0  # the reference's tolerance
    else:
        np.testing.assert_array_equal(got.astype(np.float64), want)
    ro, rmn, rmx = oracle.quantized_fully_connected(
        data.astype(np.int8), weight.astype(np.int8),
        None if bias is None else bias.astype(np.int8), -data_range, data_range, -weight_range,
        weight_range, None if bias is None else -bias_range,
        None if bias is None else bias_range)
    np.testing.assert_array_equal(got, ro)
    assert (mn.item(), mx.item()) == (rmn, rmx)


def test_quantized_fc_no_flatten(contrib):
    rng = np.random.default_rng(6)
    d = rng.integers(-127, 128, size=(4, 6, 80), dtype=np.int8)
    w = rng.integers(-127, 128, size=(24, 80), dtype=np.int8)
    out, mn, mx = contrib.quantized_fully_connected(dev(d), dev(w), None, scalar(-1), scalar(1),
                                                    scalar(-1), scalar(1), num_hidden=24,
                                                    no_bias=True, flatten=False)
    assert tuple(out.shape) == (4, 6, 24)
    ro, _, _ = oracle.quantized_fully_connected(d, w, None, -1, 1, -1, 1, flatten=False)
    np.testing.assert_array_equal(out.cpu().numpy(), ro)


@pytest.mark.parametrize("use_bias", [True, False])
def test_quantized_conv(contrib, use_bias):
    # test_quantization.py:238-371: (3,4,28,28) data, 3x3 kernel, 128 filters, pad 1
    rng = np.random.default_rng(7)
    data = rng.uniform(-127.0, 127.0, size=(3, 4, 28, 28)).astype(np.int32).astype(np.float32)
    weight = rng.uniform(-127.0, 127.0, size=(128, 4, 3, 3)).astype(np.int32).astype(np.float32)
    bias = rng.uniform(-127.0, 127.0, size=(128,)).astype(np.int32).astype(np.float32)
    want = torch.nn.functional.conv2d(torch.from_numpy(data).double(),
                                      torch.from_numpy(weight).double(),
                                      torch.from_numpy(bias).double() if use_bias else None,
                                      stride=1, padding=1).numpy()
    kw = dict(kernel=(3, 3), stride=(1, 1), dilate=(1, 1), pad=(1, 1), num_filter=128,
              no_bias=not use_bias, num_group=1, layout="NCHW")
    r = 127.0
    if use_bias:
        out, mn, mx = contrib.quantized_conv(dev(data.astype(np.int8)),
                                             dev(weight.astype(np.int8)),
                                             dev(bias.astype(np.int8)), scalar(-r), scalar(r),
                                             scalar(-r), scalar(r), scalar(-r), scalar(r), **kw)
    else:
        out, mn, mx = contrib.quantized_conv(dev(data.astype(np.int8)),
                                             dev(weight.astype(np.int8)), None, scalar(-r),
                                             scalar(r), scalar(-r), scalar(r), **kw)
    assert out.dtype == torch.int32 and tuple(out.shape) == (3, 128, 28, 28)
    got = out.cpu().numpy()
    if use_bias:
        assert int((np.abs(want - got) > 2).sum()) == 0
    else:
        np.testing.assert_allclose(got, want, atol=1)
    ro, rmn, rmx = oracle.quantized_conv(data.astype(np.int8), weight.astype(np.int8),
                                         bias.astype(np.int8) if use_bias else None, -r, r, -r, r,
                                         -r if use_bias else None, r if use_bias else None,
                                         (1, 1), (1, 1), (1, 1))
    np.testing.assert_array_equal(got, ro)
    assert (mn.item(), mx.item()) == (rmn, rmx)


@pytest.mark.parametrize("shape,filters,kernel,stride,pad", [
    ((2, 3, 64, 64), 64, (7, 7), (2, 2), (3, 3)),     # a 3-channel stem: space-to-depth route
    ((1, 3, 32, 30), 16, (3, 3), (2, 2), (1, 1)),     # the same route, odd padding
    ((2, 4, 17, 19), 24, (5, 5), (2, 2), (2, 2)),     # even padding, odd extents
    ((2, 1, 16, 16), 8, (2, 2), (2, 2), (0, 0)),      # one channel, window = stride
    ((1, 3, 15, 15), 32, (7, 7), (2, 2), (3, 3)),
    ((1, 2, 12, 14), 8, (4, 3), (2, 2), (1, 1)),      # rectangular window
    ((1, 3, 9, 9), 8, (2, 2), (2, 2), (0, 0)),        # extents disagree: plain route, 16 channels
    ((2, 3, 20, 20), 8, (3, 3), (2, 1), (1, 1)),      # stride 2 in one direction only: plain route
    ((2, 20, 9, 11), 36, (5, 3), (1, 1), (2, 1)),     # 20 channels padded to 32
    ((1, 17, 8, 8), 8, (1, 1), (1, 1), (0, 0)),
])
def test_quantized_conv_channel_counts_off_16(contrib, shape, filters, kernel, stride, pad):
    """The operator pads the channels with zeros while it brings NCHW to NHWC; the result
    is that of the unpadded convolution."""
    rng = np.random.default_rng(71)
    data = rng.integers(-127, 128, shape).astype(np.int8)
    weight = rng.integers(-127, 128, (filters, shape[1]) + kernel).astype(np.int8)
    bias = rng.integers(-127, 128, (filters,)).astype(np.int8)
    out, mn, mx = contrib.quantized_conv(dev(data), dev(weight), dev(bias), scalar(-1.0),
                                         scalar(1.0), scalar(-0.5), scalar(0.5), scalar(-2.0),
                                         scalar(2.0), kernel=kernel, stride=stride, pad=pad,
                                         num_filter=filters, no_bias=False)
    ro, rmn, rmx = oracle.quantized_conv(data, weight, bias, -1.0, 1.0, -0.5, 0.5, -2.0, 2.0,
                                         stride, pad, (1, 1))
    np.testing.assert_array_equal(out.cpu().numpy(), ro)
    assert (mn.item(), mx.item()) == (rmn, rmx)


# sizes: below one pass of the grid, the unrolled loop with a remainder and a ragged tail,
# many passes of the unrolled loop
@pytest.mark.parametrize("shape", [(5, 1000), (1, 1), (3, 1000003), (64, 28, 28, 512),
                                   ((1 << 25) + 17,)])
def test_quantized_act(contrib, shape):
    q = np.random.default_rng(8).integers(-128, 128, size=shape, dtype=np.int8)
    out, mn, mx = contrib.quantized_act(dev(q), scalar(-2.5), scalar(2.5), act_type="relu")
    np.testing.assert_array_equal(out.cpu().numpy(), np.maximum(q, 0))
    assert (mn.item(), mx.item()) == (-2.5, 2.5)


def test_chain_config1(contrib):
    """quantize_v2 -> quantized_fully_connected -> requantize -> dequantize on
    [128,1024] x [1024,1024] (the plumbing configuration), every stage vs the oracle."""
    rng = np.random.default_rng(0)
    data = rng.uniform(-1.0, 1.0, size=(128, 1024)).astype(np.float32)
    weight = (rng.standard_normal((1024, 1024)) * 0.02).astype(np.float32)
    bias = (rng.standard_normal(1024) * 0.02).astype(np.float32)
    wq, wmin, wmax = contrib.quantize(dev(weight), scalar(weight.min()), scalar(weight.max()),
                                      out_type="int8")
    bq, bmin, bmax = contrib.quantize(dev(bias), scalar(bias.min()), scalar(bias.max()),
                                      out_type="int8")
    dq, dmin, dmax = contrib.quantize_v2(dev(data), "int8", -1.0, 1.0)
    acc, omin, omax = contrib.quantized_fully_connected(dq, wq, bq, dmin, dmax, wmin, wmax, bmin,
                                                        bmax, num_hidden=1024)
    rq, rmin, rmax = contrib.requantize(acc, omin, omax)  # uncalibrated: device min/max
    out = contrib.dequantize(rq, rmin, rmax)

    wq_o, wmin_o, wmax_o = oracle.quantize(weight, weight.min(), weight.max())
    bq_o, bmin_o, bmax_o = oracle.quantize(bias, bias.min(), bias.max())
    dq_o, dmin_o, dmax_o = oracle.quantize_v2(data, "int8", -1.0, 1.0)
    acc_o, omin_o, omax_o = oracle.quantized_fully_connected(dq_o, wq_o, bq_o, dmin_o, dmax_o,
                                                             wmin_o, wmax_o, bmin_o, bmax_o)
    rq_o, rmin_o, rmax_o = oracle.requantize(acc_o, omin_o, omax_o)
    out_o = oracle.dequantize(rq_o, rmin_o, rmax_o)
    np.testing.assert_array_equal(wq.cpu().numpy(), wq_o)
    np.testing.assert_array_equal(acc.cpu().numpy(), acc_o)
    np.testing.assert_array_equal(rq.cpu().numpy(), rq_o)
    assert (rmin.item(), rmax.item()) == (rmin_o, rmax_o)
    np.testing.assert_allclose(out.cpu().numpy(), out_o, rtol=1e-6, atol=0)


def test_operator_errors(contrib):
    from mxnet_amd.operator import MXNetError
    x = torch.zeros((4, 4), device="cuda")
    with pytest.raises(MXNetError, match="out_type"):
        contrib.quantize_v2(x, out_type="int16")
    with pytest.raises(MXNetError, match="Type inconsistent"):
        contrib.requantize(x, torch.zeros(1, device="cuda"), torch.zeros(1, device="cuda"))
    with pytest.raises(MXNetError, match="uint8"):
        contrib.requantize(torch.zeros((4, 4), dtype=torch.int32, device="cuda"),
                           torch.ones(1, device="cuda"), torch.ones(1, device="cuda"),
                           out_type="uint8")
    with pytest.raises(MXNetError, match="Shape inconsistent"):
        contrib.quantized_fully_connected(
            torch.zeros((4, 16), dtype=torch.int8, device="cuda"),
            torch.zeros((8, 32), dtype=torch.int8, device="cuda"), None,
            *[torch.ones(1, device="cuda")] * 4, num_hidden=8, no_bias=True)
