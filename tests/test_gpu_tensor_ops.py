"""_contrib_quantized_elemwise_mul, _contrib_quantized_embedding, _contrib_quantized_reshape,
_contrib_quantized_transpose and _contrib_quantize_asym on the GPU, through the operator host
and the C ABI: the reference's operator tests restated
(tests/python/quantization/test_quantization.py:514-569, 811-905, 1057-1090) and bit-exact
comparison with the oracle over ragged and unaligned sizes, every output form, every index
type, permutations of 0 to 6 axes, and the reshape examples of the reference's own
documentation (src/operator/tensor/matrix_op.cc:154-196)."""
import ctypes
import itertools

import numpy as np
import pytest
import torch

import oracle

pytestmark = pytest.mark.gpu

F = np.float32


@pytest.fixture(scope="module")
def contrib():
    import mxnet_amd
    return mxnet_amd.contrib


@pytest.fixture(scope="module")
def lib():
    from mxnet_amd import _lib
    return _lib


def dev(a):
    return torch.from_numpy(np.require(a, requirements="C")).cuda()   # keeps 0-d arrays 0-d


def scalar(v):
    return dev(np.array([v], np.float32))


def host(t):
    return t.cpu().numpy()


def P(t):
    return ctypes.c_void_p(t.data_ptr())


def stream():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


# ---- elemwise_mul ---------------------------------------------------------------------------

@pytest.mark.parametrize("shape", [(4, 6), (13, 74, 52), (3, 4, 56, 56), (32, 56, 64, 11)])
def test_reference_quantized_elemwise_mul(contrib, shape):
    rng = np.random.default_rng(31)
    a = rng.uniform(-127, 127, size=shape).astype(np.int32).astype(np.int8)
    b = rng.uniform(-127, 127, size=shape).astype(np.int32).astype(np.int8)
    out, mn, mx = contrib.quantized_elemwise_mul(dev(a), dev(b), scalar(-127.0), scalar(127.0),
                                                 scalar(-127.0), scalar(127.0))
    assert out.dtype == torch.int32 and tuple(out.shape) == shape
    np.testing.assert_allclose(host(out).astype(np.float32),
                               a.astype(np.float32) * b.astype(np.float32), atol=1e-4)
    ref, rmn, rmx = oracle.quantized_elemwise_mul(a, b, -127.0, 127.0, -127.0, 127.0)
    np.testing.assert_array_equal(host(out), ref)
    assert host(mn)[0] == rmn and host(mx)[0] == rmx


@pytest.mark.parametrize("mode", ["int32", "int8", "int8_narrow", "float"])
@pytest.mark.parametrize("n", [1, 3, 17, 4099, (1 << 20) + 5])
def test_elemwise_mul_matches_oracle(contrib, mode, n):
    rng = np.random.default_rng(n)
    a = rng.integers(-128, 128, n).astype(np.int8)
    b = rng.integers(-128, 128, n).astype(np.int8)
    rngs = (-1.3, 0.9, -0.2, 2.2)
    kw = {"int32": {}, "float": {"enable_float_output": True},
          "int8": {"min_calib_range": -2.86, "max_calib_range": 2.5},
          "int8_narrow": {"min_calib_range": -0.6, "max_calib_range": 0.7}}[mode]
    got = contrib.quantized_elemwise_mul(dev(a), dev(b), *[scalar(v) for v in rngs], **kw)
    ref = oracle.quantized_elemwise_mul(a, b, *rngs, **kw)
    if mode == "float":
        assert got.dtype == torch.float32
        assert np.array_equal(host(got).view(np.uint32), ref.view(np.uint32))
        return
    out, mn, mx = got
    assert host(out).dtype == ref[0].dtype
    np.testing.assert_array_equal(host(out), ref[0])
    assert host(mn)[0] == ref[1] and host(mx)[0] == ref[2]


@pytest.mark.parametrize("out_type", [5, 4, 0])
@pytest.mark.parametrize("offset", [1, 4, 7])
def test_elemwise_mul_unaligned_pointers(lib, out_type, offset):
    """Operands that start off a 16-byte (or 4-byte) boundary take the element loop."""
    n = 5000
    rng = np.random.default_rng(offset)
    a = rng.integers(-128, 128, n + 16).astype(np.int8)
    b = rng.integers(-128, 128, n + 16).astype(np.int8)
    da, db = dev(a), dev(b)
    rngs = [scalar(v) for v in (-1.0, 2.0, -3.0, 0.5)]
    dtype = {5: torch.int8, 4: torch.int32, 0: torch.float32}[out_type]
    out = torch.zeros(n, dtype=dtype, device="cuda")
    mn, mx = scalar(0.0), scalar(0.0)
    calibrated = out_type == 5
    lib.check(lib.lib.mxq_quantized_elemwise_mul(
        stream(), ctypes.c_void_p(da.data_ptr() + offset), ctypes.c_void_p(db.data_ptr() + offset),
        *[P(r) for r in rngs], P(out), out_type, P(mn), P(mx), n, int(calibrated), -4.0, 5.5))
    kw = {"enable_float_output": True} if out_type == 0 else (
        {"min_calib_range": -4.0, "max_calib_range": 5.5} if calibrated else {})
    ref = oracle.quantized_elemwise_mul(a[offset:offset + n], b[offset:offset + n], -1.0, 2.0,
                                        -3.0, 0.5, **kw)
    ref_out = ref if out_type == 0 else ref[0]
    np.testing.assert_array_equal(host(out), ref_out)


def test_elemwise_mul_errors(lib, contrib):
    a = torch.zeros(8, dtype=torch.int8, device="cuda")
    s = scalar(1.0)
    out = torch.zeros(8, dtype=torch.int32, device="cuda")
    rc = lib.lib.mxq_quantized_elemwise_mul(stream(), P(a), P(a), P(s), P(s), P(s), P(s), P(out),
                                            4, P(s), P(s), 8, 1, -1.0, 1.0)
    assert rc != 0 and "int8 (calibrated)" in lib.last_error()
    rc = lib.lib.mxq_quantized_elemwise_mul(stream(), P(a), P(a), P(s), None, P(s), P(s), P(out),
                                            4, P(s), P(s), 8, 0, 0.0, 0.0)
    assert rc != 0 and "null range pointer" in lib.last_error()
    import mxnet_amd
    with pytest.raises(mxnet_amd.operator.MXNetError):
        contrib.quantized_elemwise_mul(a, a[:4].contiguous(), s, s, s, s)


# ---- embedding ------------------------------------------------------------------------------

@pytest.mark.parametrize("shape,input_dim,output_dim", [((1,), 1000, 256), ((1,), 1024, 512),
                                                        ((32,), 1000, 256), ((32,), 1024, 512)])
def test_reference_quantized_embedding(contrib, shape, input_dim, output_dim):
    rng = np.random.default_rng(41)
    data = rng.uniform(0, input_dim, size=shape).astype(np.int32).astype(np.float32)
    weight = rng.uniform(-127, 127, size=(input_dim, output_dim)).astype(np.int32)
    r = float(np.abs(weight).max())
    out, mn, mx = contrib.quantized_embedding(dev(data), dev(weight.astype(np.int8)), scalar(-r),
                                              scalar(r), input_dim=input_dim,
                                              output_dim=output_dim)
    assert out.dtype == torch.int8 and tuple(out.shape) == shape + (output_dim,)
    want = weight.astype(np.float32)[data.astype(np.int64)]
    np.testing.assert_array_equal(host(out).astype(np.float32), want)
    assert (host(mn)[0], host(mx)[0]) == (F(-r), F(r))


@pytest.mark.parametrize("itype", [np.float32, np.float64, np.uint8, np.int32, np.int8, np.int64])
@pytest.mark.parametrize("output_dim", [1, 3, 16, 48, 100, 768, 1040, 4096])
def test_embedding_matches_oracle(contrib, itype, output_dim):
    rng = np.random.default_rng(output_dim)
    input_dim = 300
    w = rng.integers(-128, 128, (input_dim, output_dim)).astype(np.int8)
    # indices below 0 and past the table are clipped; fractional ones truncate first
    if np.issubdtype(itype, np.floating):
        idx = rng.uniform(-20, input_dim + 20, size=(5, 37)).astype(itype)
    else:
        info = np.iinfo(itype)
        idx = rng.integers(max(info.min, -20), min(info.max, input_dim + 20) + 1,
                           size=(5, 37)).astype(itype)
    out, mn, mx = contrib.quantized_embedding(dev(idx), dev(w), scalar(-0.5), scalar(0.25),
                                              input_dim=input_dim, output_dim=output_dim)
    ref, rmn, rmx = oracle.quantized_embedding(idx, w, -0.5, 0.25)
    np.testing.assert_array_equal(host(out), ref)
    assert (host(mn)[0], host(mx)[0]) == (rmn, rmx)


def test_embedding_bert_vocabulary(contrib):
    """30522 x 768 table, 32 x 128 token ids."""
    rng = np.random.default_rng(3)
    w = rng.integers(-128, 128, (30522, 768)).astype(np.int8)
    idx = rng.integers(0, 30522, size=(32, 128)).astype(np.int32)
    out, _, _ = contrib.quantized_embedding(dev(idx), dev(w), scalar(-1.0), scalar(1.0),
                                            input_dim=30522, output_dim=768)
    np.testing.assert_array_equal(host(out), w[idx])


def test_embedding_errors(lib, contrib):
    import mxnet_amd
    w = torch.zeros((10, 4), dtype=torch.int8, device="cuda")
    idx = torch.zeros(3, dtype=torch.float16, device="cuda")
    s = scalar(1.0)
    out = torch.zeros((3, 4), dtype=torch.int8, device="cuda")
    rc = lib.lib.mxq_quantized_embedding(stream(), P(idx), 2, P(w), P(s), P(s), P(out), P(s), P(s),
                                         3, 10, 4)
    assert rc != 0 and "unsupported index type" in lib.last_error()
    with pytest.raises(mxnet_amd.operator.MXNetError):   # table shape against the attributes
        contrib.quantized_embedding(torch.zeros(3, device="cuda"), w, s, s, input_dim=11,
                                    output_dim=4)


# ---- transpose ------------------------------------------------------------------------------

@pytest.mark.parametrize("shape,axes", [((), ()), ((2, 3), (1, 0)), ((8, 21), (1, 0)),
                                        ((7, 3, 9), (2, 1, 0)), ((5, 3, 6, 8), (2, 3, 0, 1))])
@pytest.mark.parametrize("dtype", [np.int8, np.uint8])
def test_reference_quantized_transpose(contrib, shape, axes, dtype):
    rng = np.random.default_rng(51)
    lo, hi = (0, 255) if dtype == np.uint8 else (-127, 127)
    data = rng.uniform(lo, hi, size=shape).astype(dtype)
    mn_v, mx_v = float(data.min()) if data.size else 0.0, float(data.max()) if data.size else 0.0
    out, mn, mx = contrib.quantized_transpose(dev(data), scalar(mn_v), scalar(mx_v), axes=axes)
    want = np.transpose(data.astype(np.float32), axes)
    assert tuple(out.shape) == want.shape
    np.testing.assert_array_equal(host(out).astype(np.float32), want)
    assert (host(mn)[0], host(mx)[0]) == (F(mn_v), F(mx_v))


def all_perm_cases():
    cases = []
    for shape in [(6, 10), (3, 5, 7), (4, 16, 32), (2, 3, 4, 5), (2, 16, 3, 32)]:
        for axes in itertools.permutations(range(len(shape))):
            cases.append((shape, axes))
    return cases


@pytest.mark.parametrize("shape,axes", all_perm_cases())
def test_transpose_every_permutation(contrib, shape, axes):
    rng = np.random.default_rng(len(shape))
    data = rng.integers(-128, 128, shape).astype(np.int8)
    out, mn, mx = contrib.quantized_transpose(dev(data), scalar(-1.5), scalar(2.5), axes=axes)
    ref, rmn, rmx = oracle.quantized_transpose(data, -1.5, 2.5, axes)
    np.testing.assert_array_equal(host(out), ref)
    assert (host(mn)[0], host(mx)[0]) == (rmn, rmx)


@pytest.mark.parametrize("shape,axes", [
    ((32, 128, 12, 64), (0, 2, 1, 3)),      # BERT: heads to the front of the sequence axis
    ((32, 12, 128, 64), (0, 2, 1, 3)),      # and back
    ((32, 12, 128, 64), (0, 1, 3, 2)),      # keys transposed for the score product
    ((64, 256, 56, 56), (0, 2, 3, 1)),      # NCHW -> NHWC
    ((64, 56, 56, 256), (0, 3, 1, 2)),      # NHWC -> NCHW
    ((1000, 1003), (1, 0)),                 # ragged in both axes
    ((3, 1, 129, 1, 67), (4, 1, 0, 3, 2)),  # unit axes
    ((2, 3, 2, 5, 3, 4), (5, 3, 1, 4, 2, 0)),
    ((2, 9000, 17), (1, 0, 2)),             # inner run not a multiple of 16
    ((2, 3, 65536), (1, 0, 2)),             # few long rows
    ((3, 37, 19, 48), (0, 2, 1, 3)),        # runs of 48 bytes, ragged tiles of runs
    ((2, 9, 50, 16), (0, 2, 1, 3)),         # runs of 16 bytes
    ((5, 8, 9, 256), (0, 2, 1, 3)),         # runs of 256 bytes
    ((3, 13, 21, 128), (0, 2, 1, 3)),       # runs of 128 bytes, both swapped axes ragged
    ((3, 35, 9, 64), (0, 2, 1, 3)),         # runs of 64 bytes, ragged
    ((2, 33, 17, 32), (0, 2, 1, 3)),        # runs of 32 bytes, ragged
    ((9, 4, 11, 64), (2, 1, 0, 3)),         # the outermost axis swaps with the third
    ((2, 11, 3, 20, 32), (0, 3, 2, 1, 4)),  # an axis between the two that swap
    ((3, 1000, 10, 16), (2, 1, 0, 3)),      # one of the two axes too short for run tiles
    ((3, 32, 52), (0, 2, 1)),               # dword / 16-byte friendly, partial tiles
    ((3, 20, 48), (0, 2, 1)),               # output rows not a multiple of 16
    ((2, 144, 132), (0, 2, 1)),             # dword loads, 128-byte output rows, a 16-byte last tile
    ((2, 176, 160), (0, 2, 1)),             # 16-byte loads, a last tile of three pieces per row
    ((3, 5, 256, 144), (1, 0, 3, 2)),       # 16-byte loads under two permuted outer axes
    ((3, 14, 14, 256), (0, 3, 1, 2)),       # planes of 196 bytes: 16-byte loads, dword stores
    ((2, 132, 144), (0, 2, 1)),             # the same with a 4-byte last tile
    ((3, 7, 7, 256), (0, 3, 1, 2)),         # planes of 49 bytes out: the thin-extent kernel
    ((3, 256, 7, 7), (0, 2, 3, 1)),         # and in
    ((2, 3, 128, 5), (1, 0, 3, 2)),         # the same under two permuted outer axes
    ((2, 25, 384), (0, 2, 1)),
    ((128, 1), (1, 0)),
    ((2, 3, 130, 260), (1, 0, 3, 2)),
    ((0, 5, 3), (2, 0, 1)),                 # empty
    ((7,), (0,)),
    ((4, 5, 6), None),                      # default: reversed axes
])
@pytest.mark.parametrize("dtype", [np.int8, np.uint8])
def test_transpose_shapes(contrib, shape, axes, dtype):
    rng = np.random.default_rng(9)
    lo, hi = (0, 256) if dtype == np.uint8 else (-128, 128)
    data = rng.integers(lo, hi, shape).astype(dtype)
    kw = {} if axes is None else {"axes": axes}
    out, mn, mx = contrib.quantized_transpose(dev(data), scalar(-7.0), scalar(3.0), **kw)
    ref, rmn, rmx = oracle.quantized_transpose(data, -7.0, 3.0, axes)
    assert tuple(out.shape) == ref.shape
    np.testing.assert_array_equal(host(out), ref)
    assert (host(mn)[0], host(mx)[0]) == (rmn, rmx)


def test_transpose_errors(lib):
    x = torch.zeros((2, 3), dtype=torch.int8, device="cuda")
    s = scalar(1.0)
    shape = (ctypes.c_int64 * 2)(2, 3)
    bad = (ctypes.c_int * 2)(0, 0)
    rc = lib.lib.mxq_quantized_transpose(stream(), P(x), P(s), P(s), P(x), P(s), P(s), 2, shape, bad)
    assert rc != 0 and "not a permutation" in lib.last_error()
    rc = lib.lib.mxq_quantized_transpose(stream(), P(x), P(s), P(s), P(x), P(s), P(s), 9, shape, None)
    assert rc != 0 and "at most 8 axes" in lib.last_error()


# ---- reshape --------------------------------------------------------------------------------

# src/operator/tensor/matrix_op.cc:154-196: the examples of the Reshape documentation
RESHAPE_DOC_EXAMPLES = [
    ((2, 3, 4), (4, 0, 2), False, (4, 3, 2)), ((2, 3, 4), (2, 0, 0), False, (2, 3, 4)),
    ((2, 3, 4), (6, 1, -1), False, (6, 1, 4)), ((2, 3, 4), (3, -1, 8), False, (3, 1, 8)),
    ((2, 3, 4), (-1,), False, (24,)), ((2, 3, 4), (-2,), False, (2, 3, 4)),
    ((2, 3, 4), (2, -2), False, (2, 3, 4)), ((2, 3, 4), (-2, 1, 1), False, (2, 3, 4, 1, 1)),
    ((2, 3, 4), (-3, 4), False, (6, 4)), ((2, 3, 4, 5), (-3, -3), False, (6, 20)),
    ((2, 3, 4), (0, -3), False, (2, 12)), ((2, 3, 4), (-3, -2), False, (6, 4)),
    ((2, 3, 4), (-4, 1, 2, -2), False, (1, 2, 3, 4)),
    ((2, 3, 4), (2, -4, -1, 3, -2), False, (2, 1, 3, 4)),
    ((10, 5, 4), (-1, 0), False, (40, 5)), ((10, 5, 4), (-1, 0), True, (50, 4)),
]


@pytest.mark.parametrize("shape,newshape,reverse,expected", RESHAPE_DOC_EXAMPLES)
@pytest.mark.parametrize("dtype", [np.int8, np.uint8])
def test_quantized_reshape(contrib, shape, newshape, reverse, expected, dtype):
    """check_quantized_reshape (test_quantization.py:1076-1090) on the legacy operator: the
    bytes in order under the new shape, the ranges untouched."""
    rng = np.random.default_rng(61)
    lo, hi = (0, 256) if dtype == np.uint8 else (-128, 128)
    data = rng.integers(lo, hi, shape).astype(dtype)
    out, mn, mx = contrib.quantized_reshape(dev(data), scalar(-1023.343), scalar(2343.324275),
                                            shape=newshape, reverse=reverse)
    assert tuple(out.shape) == expected
    ref, rmn, rmx = oracle.quantized_reshape(data, -1023.343, 2343.324275, expected)
    np.testing.assert_array_equal(host(out), ref)
    assert (host(mn)[0], host(mx)[0]) == (rmn, rmx)


# ---- quantize_asym --------------------------------------------------------------------------

@pytest.mark.parametrize("calib", [None, (-1.0, 3.0), (-0.731, 0.2089), (-0.2, 0.4)])
@pytest.mark.parametrize("n", [1, 3, 17, 4099, (1 << 20) + 5])
def test_quantize_asym_matches_oracle(contrib, calib, n):
    rng = np.random.default_rng(n)
    x = rng.uniform(-1.0, 3.0, n).astype(np.float32) if calib != (-0.731, 0.2089) else \
        rng.uniform(-0.731, 0.2089, n).astype(np.float32)
    kw = {} if calib is None else {"min_calib_range": calib[0], "max_calib_range": calib[1]}
    q, scale, shift = contrib.quantize_asym(dev(x), **kw)
    ref, rscale, rshift = oracle.quantize_asym(x, *(calib or ()))
    assert q.dtype == torch.uint8
    np.testing.assert_array_equal(host(q), ref)     # (-0.2, 0.4) clips: low bytes, as the oracle
    assert (host(scale)[0], host(shift)[0]) == (rscale, rshift)


def test_quantize_asym_shapes_and_bert_activation(contrib):
    rng = np.random.default_rng(5)
    x = rng.standard_normal((32, 128, 768)).astype(np.float32)
    q, scale, shift = contrib.quantize_asym(dev(x))
    ref, rscale, rshift = oracle.quantize_asym(x)
    assert tuple(q.shape) == x.shape
    np.testing.assert_array_equal(host(q), ref)
    assert (host(scale)[0], host(shift)[0]) == (rscale, rshift)
    # the extremes land on the ends of the uint8 range
    assert int(host(q).min()) == 0 and int(host(q).max()) == 255


@pytest.mark.parametrize("in_type,dtype", [(5, np.int8), (3, np.uint8)])
@pytest.mark.parametrize("n,offset", [(1, 0), (4099, 0), (70000, 3)])
def test_quantize_asym_byte_inputs(lib, in_type, dtype, n, offset):
    """int8 / uint8 inputs (quantize_asym-inl.h:85-101) are only reachable through the C ABI:
    the operator's type function admits float32 alone (quantize_asym.cc:60)."""
    rng = np.random.default_rng(n)
    lo, hi = (0, 256) if dtype == np.uint8 else (-128, 128)
    x = rng.integers(lo, hi, n + 16).astype(dtype)
    dx = dev(x)
    out = torch.zeros(n + 16, dtype=torch.uint8, device="cuda")
    scale, shift = scalar(0.0), scalar(0.0)
    lib.check(lib.lib.mxq_quantize_asym(stream(), ctypes.c_void_p(dx.data_ptr() + offset), in_type,
                                        ctypes.c_void_p(out.data_ptr() + offset), P(scale),
                                        P(shift), n, 0, 0.0, 0.0, None, 0))
    ref, rscale, rshift = oracle.quantize_asym(x[offset:offset + n])
    np.testing.assert_array_equal(host(out)[offset:offset + n], ref)
    assert (host(scale)[0], host(shift)[0]) == (rscale, rshift)
    assert not host(out)[offset + n:].any() and not host(out)[:offset].any()


def test_quantize_asym_errors(lib):
    x = torch.zeros(8, dtype=torch.float32, device="cuda")
    out = torch.zeros(8, dtype=torch.uint8, device="cuda")
    s = scalar(0.0)
    rc = lib.lib.mxq_quantize_asym(stream(), P(x), 0, P(out), P(s), P(s), 8, 0, 0.0, 0.0, None, 0)
    assert rc != 0 and "workspace" in lib.last_error()
    rc = lib.lib.mxq_quantize_asym(stream(), P(x), 4, P(out), P(s), P(s), 8, 1, 0.0, 1.0, None, 0)
    assert rc != 0 and "only supports int8, uint8 and float" in lib.last_error()


# ---- batch norm -----------------------------------------------------------------------------

def bn_params(rng, C):
    return (rng.uniform(0.5, 2.0, C).astype(np.float32), rng.normal(0, 0.5, C).astype(np.float32),
            rng.normal(0, 0.3, C).astype(np.float32), rng.uniform(0.3, 2.0, C).astype(np.float32))


@pytest.mark.parametrize("shape,axis", [((32, 512, 4, 4), 1), ((4, 3, 224, 224), 1),
                                        ((8, 7, 5, 3), 1), ((6, 5, 4, 16), -1), ((10, 33), 1),
                                        ((2, 16, 1), 1), ((0, 4, 3), 1),
                                        ((3, 5, 4112), 1), ((2, 4, 1040), 1), ((2, 3, 1024), 1)])
@pytest.mark.parametrize("dtype", [np.int8, np.uint8])
@pytest.mark.parametrize("relu", [False, True])
def test_quantized_batch_norm_matches_oracle(contrib, shape, axis, dtype, relu):
    rng = np.random.default_rng(len(shape) + shape[-1])
    C = shape[axis]
    lo, hi = (0, 256) if dtype == np.uint8 else (-128, 128)
    d = rng.integers(lo, hi, shape).astype(dtype)
    gamma, beta, mean, var = bn_params(rng, C)
    rd = (0.0, 3.1) if dtype == np.uint8 else (-2.7, 3.1)
    out, mn, mx = contrib.quantized_batch_norm(
        dev(d), dev(gamma), dev(beta), dev(mean), dev(var), scalar(rd[0]), scalar(rd[1]),
        eps=2e-5, axis=axis, min_calib_range=-6.5, max_calib_range=7.25, relu=relu)
    ref, rmn, rmx = oracle.quantized_batch_norm(d, gamma, beta, mean, var, rd[0], rd[1], -6.5,
                                                7.25, eps=2e-5, axis=axis, relu=relu)
    assert out.dtype == torch.int8 and tuple(out.shape) == shape
    np.testing.assert_array_equal(host(out), ref)
    assert (host(mn)[0], host(mx)[0]) == (rmn, rmx)


def test_reference_quantized_bn(contrib):
    """check_quantized_bn (test_quantization.py:1005-1050): against the float batch norm with
    the statistics of the data itself, rtol 0.1 / atol 8 as there."""
    rng = np.random.default_rng(71)
    shape = (32, 512, 4, 4)
    data = rng.uniform(-127.0, 127.0, size=shape).astype(np.float32)
    gamma = rng.uniform(-127.0, 127.0, 512).astype(np.float32)
    beta = rng.uniform(-127.0, 127.0, 512).astype(np.float32)
    mean = data.mean(axis=(0, 2, 3))
    var = data.var(axis=(0, 2, 3))
    want = (data - mean.reshape(1, -1, 1, 1)) / np.sqrt(var.reshape(1, -1, 1, 1) + 1e-5) * \
        gamma.reshape(1, -1, 1, 1) + beta.reshape(1, -1, 1, 1)
    r_in = float(np.abs(data).max())
    q, _, _ = oracle.quantize_v2(data, "int8", -r_in, r_in)
    R = float(np.abs(want).max())
    out, mn, mx = contrib.quantized_batch_norm(
        dev(q), dev(gamma), dev(beta), dev(mean), dev(var), scalar(-r_in), scalar(r_in),
        eps=1e-5, min_calib_range=-R, max_calib_range=R)
    back = host(out).astype(np.float32) * np.float32(R / 127.0)
    np.testing.assert_allclose(back, want, rtol=1e-1, atol=8)


def test_quantized_batch_norm_errors(lib, contrib):
    import mxnet_amd
    x = torch.zeros((2, 4, 3), dtype=torch.int8, device="cuda")
    v = torch.ones(4, device="cuda")
    s = scalar(1.0)
    with pytest.raises(mxnet_amd.operator.MXNetError, match="calib"):
        contrib.quantized_batch_norm(x, v, v, v, v, s, s)
    out = torch.zeros_like(x)
    rc = lib.lib.mxq_quantized_batch_norm(stream(), P(x), 5, P(v), P(v), P(v), P(v), P(s), P(s),
                                          P(out), P(s), P(s), 2, 4, 3, 1e-3, -1.0, 1.0, 0, None, 0)
    assert rc != 0 and "workspace" in lib.last_error()
    rc = lib.lib.mxq_quantized_batch_norm(stream(), P(x), 0, P(v), P(v), P(v), P(v), P(s), P(s),
                                          P(out), P(s), P(s), 2, 4, 3, 1e-3, -1.0, 1.0, 0, P(v), 64)
    assert rc != 0 and "int8/uint8" in lib.last_error()


# ---- numpy-namespace reshape / transpose ----------------------------------------------------

@pytest.mark.parametrize("shape,axes", [((3, 5, 7), None), ((3, 5, 7), (-1, 0, 1)),
                                        ((2, 16, 8, 64), (0, -2, 1, 3)), ((4, 6), (1, 0)),
                                        ((5,), None), ((2, 3, 4, 5, 6), (-1, -3, 0, 1, 3))])
@pytest.mark.parametrize("dtype", [np.int8, np.uint8])
def test_npx_quantized_transpose(contrib, shape, axes, dtype):
    rng = np.random.default_rng(len(shape))
    d = rng.integers(0, 128, shape).astype(dtype)
    out, mn, mx = contrib.npx_quantized_transpose(dev(d), scalar(-1.5), scalar(2.0), axes=axes)
    np.testing.assert_array_equal(host(out), np.transpose(d, axes))
    assert (host(mn)[0], host(mx)[0]) == (np.float32(-1.5), np.float32(2.0))


@pytest.mark.parametrize("shape,newshape,reverse,want", [
    ((2, 3, 8), (-2, -2, 2, -1), False, (2, 3, 2, 4)),
    ((8, 3, 2, 4, 8), (-4, -1, 2, -6), True, (8, 3, 2, 4, 4, 2)),
    ((64, 1, 2, 3), (-6, 16, -1, -4), False, (16, 4, 1, 2, 3)),
    ((1, 1, 1, 1), (-3, -3, -3, -3), False, ()),
    ((2, 3, 5, 6), (-5, -1), False, (6, 30))])
def test_npx_quantized_reshape(contrib, shape, newshape, reverse, want):
    d = np.random.default_rng(3).integers(-128, 128, shape).astype(np.int8)
    out, mn, mx = contrib.npx_quantized_reshape(dev(d), scalar(-1.5), scalar(2.0), newshape,
                                                reverse=reverse)
    assert tuple(out.shape) == want
    np.testing.assert_array_equal(host(out), d.reshape(want))
    assert (host(mn)[0], host(mx)[0]) == (np.float32(-1.5), np.float32(2.0))
