"""_contrib_quantized_pooling and _contrib_quantized_flatten on the GPU: the reference's
operator test restated (tests/python/quantization/test_quantization.py:572-658: max equals
fp32 pooling of the integer-valued data, avg within 2 of it) plus bit-exact comparison with
the oracle over window geometries, both conventions, both integer types, and the three
launch shapes of the kernel (several small planes per work-group, row bands of a large
plane, the no-LDS fallback for very wide rows)."""
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


REFERENCE_CASES = [((3, 4, 56, 56), (3, 3), "max", (0, 0), (2, 2), False),
                   ((3, 4, 56, 56), (3, 3), "max", (0, 0), (2, 2), True),
                   ((3, 512, 7, 7), (7, 7), "avg", (0, 0), (1, 1), False),
                   ((3, 512, 7, 7), (7, 7), "avg", (0, 0), (1, 1), True)]


@pytest.mark.parametrize("convention", ["valid", "full"])
@pytest.mark.parametrize("qdtype", ["int8", "uint8"])
@pytest.mark.parametrize("shape,kernel,pool_type,pad,stride,global_pool", REFERENCE_CASES)
def test_reference_quantized_pooling(contrib, shape, kernel, pool_type, pad, stride, global_pool,
                                     qdtype, convention):
    rng = np.random.default_rng(17)
    lo = 0.0 if qdtype == "uint8" else -127.0
    data = rng.uniform(lo, 127.0, size=shape).astype(np.int32).astype(np.float32)
    q = data.astype(qdtype)
    out, mn, mx = contrib.quantized_pooling(dev(q), scalar(-127.0), scalar(127.0), kernel=kernel,
                                            pool_type=pool_type, global_pool=global_pool,
                                            pooling_convention=convention, stride=stride, pad=pad)
    ref, _, _ = oracle.quantized_pooling(q, -127.0, 127.0, kernel, pool_type, stride, pad,
                                         global_pool, convention)
    assert tuple(out.shape) == ref.shape and out.dtype == dev(q).dtype
    np.testing.assert_array_equal(out.cpu().numpy(), ref)
    assert mn.item() == -127.0 and mx.item() == 127.0
    # the reference's own check against fp32 pooling
    t = torch.from_numpy(data)
    if global_pool:
        fp = t.amax(dim=(2, 3), keepdim=True) if pool_type == "max" else \
            t.mean(dim=(2, 3), keepdim=True)
    elif pool_type == "max":
        fp = torch.nn.functional.max_pool2d(t, kernel, stride, pad, ceil_mode=convention == "full")
    else:
        fp = torch.nn.functional.avg_pool2d(t, kernel, stride, pad, ceil_mode=convention == "full")
    diff = np.abs(fp.numpy() - out.cpu().numpy().astype(np.float32))
    assert diff.max() == 0 if pool_type == "max" else diff.max() <= 2


GEOMETRIES = [((2, 3, 13, 10), (3, 3), (2, 2), (1, 1)),       # several planes per group
              ((2, 3, 13, 10), (2, 3), (1, 2), (1, 0)),
              ((5, 7, 9, 9), (5, 5), (3, 3), (2, 2)),
              ((1, 2, 300, 301), (3, 3), (2, 2), (1, 1)),     # row bands, odd row pitch
              ((2, 2, 200, 260), (7, 5), (3, 2), (3, 2)),
              ((1, 1, 3, 40000), (3, 3), (1, 2), (1, 1)),     # one band does not fit the LDS
              ((64, 8, 112, 112), (3, 3), (2, 2), (1, 1)),    # ResNet stem pool, fewer channels
              ((4, 2048, 7, 7), (7, 7), (1, 1), (0, 0))]      # ResNet global average pool


@pytest.mark.parametrize("qdtype", [np.int8, np.uint8])
@pytest.mark.parametrize("pool_type", ["max", "avg"])
@pytest.mark.parametrize("shape,kernel,stride,pad", GEOMETRIES)
def test_pooling_matches_oracle(contrib, shape, kernel, stride, pad, pool_type, qdtype):
    rng = np.random.default_rng(hash((shape, kernel, pool_type)) % (2 ** 32))
    lo, hi = (0, 256) if qdtype == np.uint8 else (-128, 128)
    q = rng.integers(lo, hi, shape).astype(qdtype)
    for convention in ("valid", "full"):
        for include_pad in ((True, False) if pool_type == "avg" else (None,)):
            out, mn, mx = contrib.quantized_pooling(
                dev(q), scalar(-3.5), scalar(2.25), kernel=kernel, pool_type=pool_type,
                pooling_convention=convention, stride=stride, pad=pad,
                count_include_pad=include_pad)
            ref, _, _ = oracle.quantized_pooling(
                q, -3.5, 2.25, kernel, pool_type, stride, pad, False, convention,
                True if include_pad is None else include_pad)
            assert tuple(out.shape) == ref.shape
            np.testing.assert_array_equal(out.cpu().numpy(), ref)
            assert mn.item() == -3.5 and mx.item() == 2.25


def test_pooling_unaligned_input_view(contrib):
    """A tensor that starts 1 byte into an allocation takes the byte-granular loader."""
    rng = np.random.default_rng(3)
    q = rng.integers(-128, 128, (2, 5, 17, 19)).astype(np.int8)
    buf = torch.empty(q.size + 1, dtype=torch.int8, device="cuda")
    view = buf[1:].view(q.shape)
    view.copy_(dev(q))
    assert view.data_ptr() % 16 != 0
    out, _, _ = contrib.quantized_pooling(view, scalar(-1.0), scalar(1.0), kernel=(3, 3),
                                          pool_type="max", stride=(2, 2), pad=(1, 1))
    ref, _, _ = oracle.quantized_pooling(q, -1.0, 1.0, (3, 3), "max", (2, 2), (1, 1))
    np.testing.assert_array_equal(out.cpu().numpy(), ref)


def test_flatten(contrib):
    rng = np.random.default_rng(4)
    for dtype in (np.int8, np.uint8):
        for shape in [(2, 3, 4, 5), (7, 33), (1, 100003), (64, 2048, 1, 1)]:
            q = rng.integers(0, 128, shape).astype(dtype)
            out, mn, mx = contrib.quantized_flatten(dev(q), scalar(-0.5), scalar(4.0))
            ref, _, _ = oracle.quantized_flatten(q, -0.5, 4.0)
            assert tuple(out.shape) == ref.shape and out.dtype == dev(q).dtype
            np.testing.assert_array_equal(out.cpu().numpy(), ref)
            assert mn.item() == -0.5 and mx.item() == 4.0


def test_pooling_errors():
    import mxnet_amd
    lib = mxnet_amd._lib.lib
    x = torch.zeros((1, 1, 8, 8), dtype=torch.int8, device="cuda")
    o = torch.zeros((1, 1, 3, 3), dtype=torch.int8, device="cuda")
    s = [torch.zeros(1, device="cuda") for _ in range(4)]
    P = lambda t: ctypes.c_void_p(t.data_ptr())
    args = lambda in_type, pool: (None, P(x), in_type, 1, 1, 8, 8, 3, 3, 2, 2, 0, 0, 3, 3, pool,
                                  1, P(s[0]), P(s[1]), P(o), P(s[2]), P(s[3]))
    assert lib.mxq_quantized_pooling_nchw(*args(4, 0)) == -1
    assert "int8 or uint8" in lib.mxq_last_error().decode()
    assert lib.mxq_quantized_pooling_nchw(*args(5, 2)) == -1
    assert "max/avg" in lib.mxq_last_error().decode()
    assert lib.mxq_quantized_pooling_nchw(*args(5, 0)) == 0
    torch.cuda.synchronize()
