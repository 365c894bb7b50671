"""Pins the integer half of the CPU oracle (qref_fc, qref_conv_nchw): exact integer
arithmetic compared with independent implementations (numpy int64 matmul, torch's
integer matmul and float64 convolution on integer-valued operands), textbook special
cases, and the reference test's own construction (integer-valued fp32 Dense / Conv,
tests/python/quantization/test_quantization.py:238-371, 661-808)."""
import numpy as np
import pytest
import torch

import oracle


@pytest.mark.parametrize("M,K,N", [(1, 1, 1), (3, 7, 5), (32, 444, 100), (64, 1024, 96),
                                   (17, 4099, 9)])
def test_fc_matches_numpy_int64(M, K, N):
    rng = np.random.default_rng(M * 131 + K)
    d = rng.integers(-128, 128, size=(M, K), dtype=np.int8)
    w = rng.integers(-128, 128, size=(N, K), dtype=np.int8)
    b = rng.integers(-2 ** 20, 2 ** 20, size=N).astype(np.int32)
    want = d.astype(np.int64) @ w.astype(np.int64).T
    np.testing.assert_array_equal(oracle.fc_int32(d, w), want)
    np.testing.assert_array_equal(oracle.fc_int32(d, w, b), want + b)


def test_fc_matches_torch_int_mm():
    rng = np.random.default_rng(0)
    d = rng.integers(-128, 128, size=(64, 256), dtype=np.int8)
    w = rng.integers(-128, 128, size=(128, 256), dtype=np.int8)
    want = torch._int_mm(torch.from_numpy(d), torch.from_numpy(w).t().contiguous()).numpy()
    np.testing.assert_array_equal(oracle.fc_int32(d, w), want)


def test_fc_special_cases():
    K = 48
    d = np.random.default_rng(1).integers(-128, 128, size=(5, K), dtype=np.int8)
    eye = np.eye(K, dtype=np.int8)
    np.testing.assert_array_equal(oracle.fc_int32(d, eye), d.astype(np.int32))     # identity
    ones = np.ones((3, K), np.int8)
    np.testing.assert_array_equal(oracle.fc_int32(d, ones),
                                  np.repeat(d.sum(1, dtype=np.int32)[:, None], 3, 1))
    single = np.zeros((1, K), np.int8)
    single[0, 7] = -3                                                               # one tap
    np.testing.assert_array_equal(oracle.fc_int32(d, single)[:, 0], -3 * d[:, 7].astype(np.int32))
    # extreme values: K * 128 * 128 fits int32 for K = 4096
    big = np.full((2, 4096), -128, np.int8)
    assert int(oracle.fc_int32(big, big)[0, 0]) == 4096 * 128 * 128
    # transposing the weight changes the answer (guards against a transposed operand)
    w = np.random.default_rng(2).integers(-128, 128, size=(K, K), dtype=np.int8)
    assert not np.array_equal(oracle.fc_int32(d, w), oracle.fc_int32(d, w.T.copy()))


def test_fc_wraps_like_int32():
    d = np.full((1, 1), 127, np.int8)
    w = np.full((1, 1), 127, np.int8)
    b = np.array([np.iinfo(np.int32).max], np.int32)
    got = oracle.fc_int32(d, w, b)
    assert int(got[0, 0]) == ((127 * 127 + int(b[0]) + 2 ** 31) % 2 ** 32) - 2 ** 31


def test_quantized_fc_reference_construction():
    # integer-valued fp32 Dense == int32 output when the ranges are the observed maxabs
    rng = np.random.default_rng(3)
    for shape, nh, use_bias in [((32, 111, 2, 2), 100, False), ((32, 512, 2, 2), 100, True)]:
        data = rng.uniform(-63.0, 63.0, size=shape).astype(np.int32).astype(np.float32)
        K = int(np.prod(shape[1:]))
        weight = rng.uniform(-63.0, 63.0, size=(nh, K)).astype(np.int32).astype(np.float32)
        dr, wr = float(np.abs(data).max()), float(np.abs(weight).max())
        want = data.reshape(shape[0], -1).astype(np.float64) @ weight.astype(np.float64).T
        bias = None
        if use_bias:
            bias = rng.uniform(-63.0, 63.0, size=nh).astype(np.int32).astype(np.float32)
            br = float(np.abs(bias).max())
            rescale = (127.0 / dr) * (127.0 / wr) / (127.0 / br)
            want = want + (bias * rescale).astype(np.int32)
        out, mn, mx = oracle.quantized_fully_connected(
            data.astype(np.int8), weight.astype(np.int8),
            None if bias is None else bias.astype(np.int8), -dr, dr, -wr, wr,
            None if bias is None else -br, None if bias is None else br)
        if use_bias:
            assert np.abs(out - want).max() <= 2   # the reference's own tolerance
        else:
            np.testing.assert_array_equal(out.astype(np.float64), want)


CONV_CASES = [  # N, C, H, W, O, KH, KW, stride, pad, dilate
    (3, 4, 28, 28, 16, 3, 3, 1, 1, 1), (2, 8, 9, 11, 6, 1, 1, 1, 0, 1),
    (2, 8, 9, 11, 6, 1, 1, 2, 0, 1), (1, 5, 13, 12, 7, 3, 3, 2, 1, 1),
    (1, 3, 12, 12, 4, 3, 3, 1, 2, 2), (2, 6, 8, 10, 5, 5, 3, 1, 2, 1),
]


@pytest.mark.parametrize("case", CONV_CASES)
def test_conv_matches_torch_float64(case):
    N, C, H, W, O, KH, KW, s, p, dl = case
    rng = np.random.default_rng(sum(case))
    d = rng.integers(-128, 128, size=(N, C, H, W), dtype=np.int8)
    w = rng.integers(-128, 128, size=(O, C, KH, KW), dtype=np.int8)
    b = rng.integers(-1000, 1000, size=O).astype(np.int32)
    want = torch.nn.functional.conv2d(torch.from_numpy(d).double(), torch.from_numpy(w).double(),
                                      torch.from_numpy(b).double(), stride=s, padding=p,
                                      dilation=dl).numpy()
    got = oracle.conv_int32_nchw(d, w, b, (s, s), (p, p), (dl, dl))
    assert got.shape == want.shape
    np.testing.assert_array_equal(got.astype(np.float64), want)


def test_conv_special_cases():
    rng = np.random.default_rng(9)
    d = rng.integers(-128, 128, size=(2, 3, 6, 7), dtype=np.int8)
    # 1x1 identity kernel copies the channel
    w = np.zeros((3, 3, 1, 1), np.int8)
    for c in range(3):
        w[c, c, 0, 0] = 1
    np.testing.assert_array_equal(oracle.conv_int32_nchw(d, w), d.astype(np.int32))
    # single off-centre tap = shifted image with zero padding (cross-correlation, not flipped)
    w = np.zeros((1, 3, 3, 3), np.int8)
    w[0, 1, 0, 2] = 2      # kh = 0, kw = 2 -> reads (h-1, w+1)
    got = oracle.conv_int32_nchw(d, w, pad=(1, 1))
    want = np.zeros((2, 1, 6, 7), np.int32)
    want[:, 0, 1:, :-1] = 2 * d[:, 1, :-1, 1:].astype(np.int32)
    np.testing.assert_array_equal(got, want)
    # a 1x1 convolution is the FC of the pixels
    w = rng.integers(-128, 128, size=(5, 3, 1, 1), dtype=np.int8)
    got = oracle.conv_int32_nchw(d, w)
    fc = oracle.fc_int32(d.transpose(0, 2, 3, 1).reshape(-1, 3), w.reshape(5, 3))
    np.testing.assert_array_equal(got.transpose(0, 2, 3, 1).reshape(-1, 5), fc)


def test_relu():
    q = np.arange(-128, 128).astype(np.int8)
    np.testing.assert_array_equal(oracle.relu_i8(q), np.maximum(q, 0))
