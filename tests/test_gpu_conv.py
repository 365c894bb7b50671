"""Parity of the HIP implicit-GEMM quantized convolution with the CPU oracle (exact
int32 cross-correlation), through the C ABI and the NCHW<->NHWC adapters."""
import numpy as np
import pytest
import torch

import oracle
from tests.data_gen import int8_uniform

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def capi():
    import mxnet_amd
    return mxnet_amd.capi


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def f32(v):
    return dev(np.array([v], np.float32))


def run_conv_nchw(capi, d, w, b, rd, rw, rb, stride, pad, dilate, calib=None, relu=False,
                  force=None, want_int32=True):
    """force = (cfg, splits) pins the kernel variant through the test-only entry point."""
    dn = capi.nchw_to_nhwc_i8(dev(d))
    wn = capi.nchw_to_nhwc_i8(dev(w))
    res = capi.quantized_conv_nhwc(dn, wn, None if b is None else dev(b), f32(-rd), f32(rd),
                                   f32(-rw), f32(rw), None if b is None else f32(-rb),
                                   None if b is None else f32(rb), stride=stride, pad=pad,
                                   dilate=dilate, calib=calib, relu=relu, force=force,
                                   want_int32=want_int32)
    if want_int32:
        res["out32_nchw"] = capi.nhwc_to_nchw(res["out32"])
    if res["out8"] is not None:
        res["out8_nchw"] = capi.nhwc_to_nchw(res["out8"])
    return res


# (N, C, H, W, O, KH, KW, stride, pad, dilate)
CASES = [
    (3, 4, 28, 28, 128, 3, 3, 1, 1, 1),    # the reference's test (test_quantization.py:365-367)
    (2, 64, 56, 56, 64, 1, 1, 1, 0, 1),    # ResNet stage-1 1x1
    (2, 64, 56, 56, 64, 3, 3, 1, 1, 1),    # ResNet stage-1 3x3
    (2, 64, 28, 28, 256, 1, 1, 1, 0, 1),
    (2, 256, 56, 56, 128, 1, 1, 2, 0, 1),  # stride-2 downsample
    (2, 128, 28, 28, 128, 3, 3, 1, 1, 1),
    (1, 512, 7, 7, 512, 3, 3, 1, 1, 1),
    (1, 1024, 14, 14, 2048, 1, 1, 2, 0, 1),
    (2, 32, 17, 13, 48, 3, 3, 2, 1, 1),    # odd sizes, stride 2 with pad
    (1, 16, 12, 12, 20, 3, 3, 1, 2, 2),    # dilation
    (2, 20, 9, 11, 36, 5, 3, 1, 2, 1),     # C % 16 != 0, rectangular kernel
    (1, 3, 16, 16, 8, 7, 7, 2, 3, 1),      # first-layer-like, C = 3
]


@pytest.mark.parametrize("case", CASES)
@pytest.mark.parametrize("use_bias", [False, True])
def test_conv_int32(capi, case, use_bias):
    N, C, H, W, O, KH, KW, s, p, dl = case
    d = int8_uniform((N, C, H, W), seed=C + H)
    w = int8_uniform((O, C, KH, KW), seed=O + KH)
    b = int8_uniform((O,), seed=O) if use_bias else None
    rd, rw, rb = 3.0, 0.2, 1.5
    res = run_conv_nchw(capi, d, w, b, rd, rw, rb, (s, s), (p, p), (dl, dl))
    ro, rmn, rmx = oracle.quantized_conv(d, w, b, -rd, rd, -rw, rw, None if b is None else -rb,
                                         None if b is None else rb, (s, s), (p, p), (dl, dl))
    np.testing.assert_array_equal(res["out32_nchw"].cpu().numpy(), ro)
    assert (res["omin"].item(), res["omax"].item()) == (rmn, rmx)


@pytest.mark.parametrize("cfg", [1, 2, 3, 4, 5, 11, 12, 13, 14, 15, 16, 22, 23, 24, 25, 31, 32, 33, 34,
                                 35, 36, 37, 38, 39])
def test_conv_every_tile_config(capi, cfg):
    N, C, H, W, O, KH, KW, s, p, dl = (2, 32, 19, 19, 72, 3, 3, 1, 1, 1)
    d = int8_uniform((N, C, H, W), seed=cfg)
    w = int8_uniform((O, C, KH, KW), seed=cfg + 1)
    b = int8_uniform((O,), seed=cfg + 2)
    res = run_conv_nchw(capi, d, w, b, 1.0, 1.0, 1.0, (s, s), (p, p), (dl, dl),
                        calib=(-0.02, 0.02), relu=True, force=(cfg, 1))
    ro, rmn, rmx = oracle.quantized_conv(d, w, b, -1.0, 1.0, -1.0, 1.0, -1.0, 1.0, (s, s),
                                         (p, p), (dl, dl))
    np.testing.assert_array_equal(res["out32_nchw"].cpu().numpy(), ro)
    rq, qmn, qmx = oracle.requantize(ro, rmn, rmx, -0.02, 0.02)
    np.testing.assert_array_equal(res["out8_nchw"].cpu().numpy(), oracle.relu_i8(rq))
    assert (res["rmin"].item(), res["rmax"].item()) == (qmn, qmx)


@pytest.mark.parametrize("cfg", [11, 12, 13, 14, 15, 16, 22, 23, 24, 25, 31, 32, 33, 34, 35, 36, 37,
                                 38, 39])
@pytest.mark.parametrize("case", [(2, 16, 9, 11, 40, 3, 3, 1, 1, 1), (1, 48, 8, 8, 24, 5, 3, 2, 2, 1),
                                  (2, 64, 14, 14, 96, 1, 1, 2, 0, 1), (1, 16, 12, 12, 20, 3, 3, 1, 2, 2),
                                  (3, 128, 7, 7, 130, 3, 3, 1, 1, 1)])
def test_conv_direct_to_lds_configs(capi, cfg, case):
    """The buffer-load kernels on shapes that stress the tap bookkeeping: C = 16 (four
    taps per 64-byte stage), C = 48 (taps straddle stages), stride 2, dilation, K tails."""
    N, C, H, W, O, KH, KW, s, p, dl = case
    d = int8_uniform((N, C, H, W), seed=cfg + C)
    w = int8_uniform((O, C, KH, KW), seed=cfg + O)
    b = int8_uniform((O,), seed=cfg)
    res = run_conv_nchw(capi, d, w, b, 1.0, 1.0, 1.0, (s, s), (p, p), (dl, dl),
                        calib=(-0.05, 0.04), relu=False, force=(cfg, 1))
    ro, rmn, rmx = oracle.quantized_conv(d, w, b, -1.0, 1.0, -1.0, 1.0, -1.0, 1.0, (s, s),
                                         (p, p), (dl, dl))
    np.testing.assert_array_equal(res["out32_nchw"].cpu().numpy(), ro)
    rq, qmn, qmx = oracle.requantize(ro, rmn, rmx, -0.05, 0.04)
    np.testing.assert_array_equal(res["out8_nchw"].cpu().numpy(), rq)


# split-K through the convolution kernels: the K slices start in the middle of the
# (kh, kw, c) walk (C = 16: four taps per 64-byte stage; C = 48: taps straddle stages),
# stride 2, dilation, K tails, more splits than stages
@pytest.mark.parametrize("cfg", [11, 12, 13, 14, 15, 16, 22, 23, 24, 25, 31, 32, 33, 34, 35, 36, 37,
                                 38, 39])
@pytest.mark.parametrize("case,splits", [((2, 16, 9, 11, 40, 3, 3, 1, 1, 1), 2),
                                         ((1, 48, 8, 8, 24, 5, 3, 2, 2, 1), 3),
                                         ((2, 64, 14, 14, 96, 1, 1, 2, 0, 1), 2),
                                         ((1, 16, 12, 12, 20, 3, 3, 1, 2, 2), 9),
                                         ((3, 128, 7, 7, 130, 3, 3, 1, 1, 1), 4),
                                         ((1, 512, 7, 7, 192, 3, 3, 1, 1, 1), 6)])
def test_conv_split_k(capi, cfg, case, splits):
    N, C, H, W, O, KH, KW, s, p, dl = case
    d = int8_uniform((N, C, H, W), seed=cfg + C + 1)
    w = int8_uniform((O, C, KH, KW), seed=cfg + O + 1)
    b = int8_uniform((O,), seed=cfg + 1)
    res = run_conv_nchw(capi, d, w, b, 1.0, 1.0, 1.0, (s, s), (p, p), (dl, dl),
                        calib=(-0.05, 0.04), relu=True, force=(cfg, splits))
    ro, rmn, rmx = oracle.quantized_conv(d, w, b, -1.0, 1.0, -1.0, 1.0, -1.0, 1.0, (s, s),
                                         (p, p), (dl, dl))
    np.testing.assert_array_equal(res["out32_nchw"].cpu().numpy(), ro)
    rq, qmn, qmx = oracle.requantize(ro, rmn, rmx, -0.05, 0.04)
    np.testing.assert_array_equal(res["out8_nchw"].cpu().numpy(), oracle.relu_i8(rq))


# the parked-weights 3 x 3 kernel (64 -> 64 channels, one output row per wave item): odd
# extents, a single column, the widest row it takes, rows shorter than one MFMA block, more
# rows than waves, with and without bias and relu
@pytest.mark.parametrize("N,H,W", [(2, 56, 56), (3, 7, 9), (1, 5, 58), (2, 13, 1), (5, 3, 33),
                                   (1, 1, 1), (70, 6, 31), (6, 56, 56), (24, 7, 40)])
@pytest.mark.parametrize("relu,use_bias", [(True, True), (False, True), (True, False)])
@pytest.mark.parametrize("forced", [True, False])
def test_conv3x3_parked_weights(capi, N, H, W, relu, use_bias, forced):
    d = int8_uniform((N, 64, H, W), seed=N + H + W)
    w = int8_uniform((64, 64, 3, 3), seed=H + 1, lo=-50, hi=50)
    b = int8_uniform((64,), seed=W + 2) if use_bias else None
    ro, rmn, rmx = oracle.quantized_conv(d, w, b, -1.0, 1.0, -1.0, 1.0,
                                         -1.0 if use_bias else None, 1.0 if use_bias else None,
                                         (1, 1), (1, 1), (1, 1))
    fl = ro.astype(np.float64) * (float(rmx) / 2147483648.0)
    R = float(np.percentile(np.abs(fl), 98.0)) or 1.0
    res = run_conv_nchw(capi, d, w, b, 1.0, 1.0, 1.0, (1, 1), (1, 1), (1, 1), calib=(-R, 0.9 * R),
                        relu=relu, force=(61, 1) if forced else None, want_int32=False)
    rq, qmn, qmx = oracle.requantize(ro, rmn, rmx, -R, 0.9 * R)
    if relu:
        rq = oracle.relu_i8(rq)
    np.testing.assert_array_equal(res["out8_nchw"].cpu().numpy(), rq)
    assert (res["omin"].item(), res["omax"].item()) == (rmn, rmx)
    assert (res["rmin"].item(), res["rmax"].item()) == (qmn, qmx)


# the resident-patch 3 x 3 kernel (C a multiple of 128): whole planes smaller than a tile
# (several images and their zero rows inside one patch), rows that straddle tiles, one
# column, the last tile short, output channels off the tile, int32 and fused int8 outputs
@pytest.mark.parametrize("N,C,H,W,O", [(2, 128, 28, 28, 128), (4, 128, 6, 14, 128),
                                       (3, 128, 9, 6, 64), (3, 128, 28, 28, 144),
                                       (40, 128, 6, 6, 32), (2, 128, 31, 29, 48),
                                       (1, 128, 8, 20, 16)])
@pytest.mark.parametrize("fused", [True, False])
def test_conv3x3_resident_patch(capi, N, C, H, W, O, fused, cfg=62):
    d = int8_uniform((N, C, H, W), seed=N + H + W)
    w = int8_uniform((O, C, 3, 3), seed=H + 1, lo=-50, hi=50)
    b = int8_uniform((O,), seed=W + 2)
    ro, rmn, rmx = oracle.quantized_conv(d, w, b, -1.0, 1.0, -1.0, 1.0, -1.0, 1.0, (1, 1), (1, 1),
                                         (1, 1))
    fl = ro.astype(np.float64) * (float(rmx) / 2147483648.0)
    R = float(np.percentile(np.abs(fl), 98.0)) or 1.0
    res = run_conv_nchw(capi, d, w, b, 1.0, 1.0, 1.0, (1, 1), (1, 1), (1, 1),
                        calib=(-R, 0.9 * R) if fused else None, relu=fused, force=(cfg, 1),
                        want_int32=not fused)
    assert (res["omin"].item(), res["omax"].item()) == (rmn, rmx)
    if fused:
        rq, qmn, qmx = oracle.requantize(ro, rmn, rmx, -R, 0.9 * R)
        np.testing.assert_array_equal(res["out8_nchw"].cpu().numpy(), oracle.relu_i8(rq))
    else:
        np.testing.assert_array_equal(res["out32_nchw"].cpu().numpy(), ro)


def test_conv3x3_resident_patch_refuses_other_shapes(capi):
    import mxnet_amd
    # C off 128; patches past their room (long rows; 1 x 1 planes: 128 images per tile)
    for shape in [(1, 64, 8, 8), (1, 128, 8, 600), (2, 256, 14, 14), (3, 128, 1, 1)]:
        d = int8_uniform(shape, seed=1)
        w = int8_uniform((64, shape[1], 3, 3), seed=2)
        with pytest.raises(mxnet_amd._lib.MXQError, match="resident-patch"):
            run_conv_nchw(capi, d, w, None, 1.0, 1.0, 1.0, (1, 1), (1, 1), (1, 1),
                          calib=(-1.0, 1.0), force=(62, 1), want_int32=False)


def test_conv3x3_parked_weights_refuses_other_shapes(capi):
    import mxnet_amd
    d = int8_uniform((1, 32, 8, 8), seed=1)
    w = int8_uniform((64, 32, 3, 3), seed=2)
    with pytest.raises(mxnet_amd._lib.MXQError, match="parked-weights"):
        run_conv_nchw(capi, d, w, None, 1.0, 1.0, 1.0, (1, 1), (1, 1), (1, 1), calib=(-1.0, 1.0),
                      force=(61, 1), want_int32=False)


def test_layout_adapters(capi):
    x = int8_uniform((3, 5, 7, 9), seed=1)
    y = capi.nchw_to_nhwc_i8(dev(x))
    np.testing.assert_array_equal(y.cpu().numpy(), x.transpose(0, 2, 3, 1))
    z = capi.nhwc_to_nchw(y)
    np.testing.assert_array_equal(z.cpu().numpy(), x)
    # int8 NHWC -> NCHW: the dword kernel, and from 128 pixels with 16 | C the 16-byte one
    # (ragged last tiles in both directions)
    for shape in ((2, 8, 8, 64), (3, 4, 12, 20), (1, 16, 16, 132), (2, 16, 8, 144),
                  (2, 13, 12, 272), (1, 56, 56, 256), (3, 14, 14, 256), (2, 10, 15, 144),
                  (2, 14, 14, 1040),    # the last three: planes of 4 | H*W bytes, dword stores
                  (3, 7, 7, 256), (2, 5, 5, 128), (2, 3, 3, 384), (2, 1, 1, 128),
                  (2, 7, 9, 128)):      # thin planes (at most 64 bytes) beside 128 | C
        v8 = int8_uniform(shape, seed=4)
        z8 = capi.nhwc_to_nchw(dev(v8))
        np.testing.assert_array_equal(z8.cpu().numpy(), v8.transpose(0, 3, 1, 2))
    v = np.random.default_rng(2).integers(-2**31, 2**31 - 1, size=(2, 70, 66, 130),
                                          dtype=np.int32)
    z = capi.nhwc_to_nchw(dev(v))
    np.testing.assert_array_equal(z.cpu().numpy(), v.transpose(0, 3, 1, 2))
    # channel padding: zeros behind the C real channels of every pixel
    import ctypes
    import mxnet_amd
    # (the last six take the dword kernel: H*W % 4 == 0; 1, 2, 3 and 4 sixteen-byte pieces
    # per output row, more than 64 channels, a ragged last 128-column tile)
    for shape, cp in (((3, 5, 7, 9), 16), ((2, 3, 70, 33), 16), ((1, 70, 5, 5), 80),
                      ((2, 16, 4, 4), 16), ((2, 3, 8, 8), 16), ((2, 64, 12, 12), 64),
                      ((3, 70, 4, 8), 80), ((2, 130, 16, 4), 144), ((1, 40, 4, 4), 48),
                      ((2, 20, 10, 30), 32), ((2, 256, 12, 12), 256), ((1, 200, 20, 12), 208),
                      ((2, 128, 56, 56), 128), ((3, 256, 7, 7), 256), ((2, 128, 5, 5), 128),
                      ((2, 384, 3, 3), 384), ((2, 128, 1, 1), 128), ((2, 128, 7, 9), 128)):
        x = int8_uniform(shape, seed=3)
        n, c, h, w = shape
        out = torch.full((n, h, w, cp), 77, dtype=torch.int8, device="cuda")
        st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
        rc = mxnet_amd._lib.lib.mxq_nchw_to_nhwc_pad_i8(st, ctypes.c_void_p(dev(x).data_ptr()),
                                                        ctypes.c_void_p(out.data_ptr()), n, c, h,
                                                        w, cp)
        assert rc == 0
        want = np.zeros((n, h, w, cp), np.int8)
        want[..., :c] = x.transpose(0, 2, 3, 1)
        np.testing.assert_array_equal(out.cpu().numpy(), want)
    rc = mxnet_amd._lib.lib.mxq_nchw_to_nhwc_pad_i8(st, None, None, 1, 8, 2, 2, 4)
    assert rc == -1 and b"C_padded" in mxnet_amd._lib.lib.mxq_last_error()
    # space-to-depth by 2 with an offset of 0 or 1 in each direction
    for shape, off_h, off_w, cp in (((2, 3, 8, 10), 1, 1, 16), ((1, 3, 7, 9), 0, 1, 16),
                                    ((2, 4, 5, 5), 1, 0, 16), ((3, 1, 6, 6), 0, 0, 4),
                                    ((1, 2, 224, 224), 1, 1, 32)):
        x = int8_uniform(shape, seed=5)
        n, c, h, w = shape
        h2, w2 = (h + off_h + 1) // 2, (w + off_w + 1) // 2
        out = torch.full((n, h2, w2, cp), 77, dtype=torch.int8, device="cuda")
        rc = mxnet_amd._lib.lib.mxq_nchw_to_s2d_nhwc_i8(st, ctypes.c_void_p(dev(x).data_ptr()),
                                                        ctypes.c_void_p(out.data_ptr()), n, c, h,
                                                        w, off_h, off_w, cp)
        assert rc == 0
        padded = np.zeros((n, c, 2 * h2 + 2, 2 * w2 + 2), np.int8)
        padded[:, :, off_h:off_h + h, off_w:off_w + w] = x
        want = np.zeros((n, h2, w2, cp), np.int8)
        for dh in range(2):
            for dw in range(2):
                blk = padded[:, :, dh:dh + 2 * h2:2, dw:dw + 2 * w2:2]     # [n, c, h2, w2]
                want[..., (dh * 2 + dw) * c:(dh * 2 + dw + 1) * c] = blk.transpose(0, 2, 3, 1)
        np.testing.assert_array_equal(out.cpu().numpy(), want)
    rc = mxnet_amd._lib.lib.mxq_nchw_to_s2d_nhwc_i8(st, None, None, 1, 8, 2, 2, 0, 0, 16)
    assert rc == -1 and b"4 * C" in mxnet_amd._lib.lib.mxq_last_error()


def test_conv_1x1_equals_fc(capi):
    """A 1x1 stride-1 convolution is the FC of the flattened pixels."""
    N, H, W, C, O = 2, 14, 14, 256, 320
    d = int8_uniform((N, H, W, C), seed=4)
    w = int8_uniform((O, 1, 1, C), seed=5)
    one = torch.ones(1, device="cuda")
    rc = capi.quantized_conv_nhwc(dev(d), dev(w), None, -one, one, -one, one)
    rf = capi.quantized_fc(dev(d.reshape(-1, C)), dev(w.reshape(O, C)), None, -one, one, -one,
                           one)
    assert torch.equal(rc["out32"].reshape(-1, O), rf["out32"])


@pytest.mark.parametrize("case", [
    (2, 64, 56, 56, 64, 3, 3, 1, 1, 1),     # planes of 3136 pixels: whole 128-byte runs
    (3, 32, 28, 28, 96, 1, 1, 1, 0, 1),     # 1x1: the fully-connected route; 784-pixel planes straddle tiles
    (5, 16, 7, 7, 40, 3, 3, 1, 1, 1),       # 49-pixel planes (not a multiple of 4), O % 16 != 0
    (2, 16, 13, 9, 33, 3, 3, 2, 1, 1),      # ragged everything, odd O
    (1, 48, 14, 14, 256, 1, 1, 2, 0, 1),    # strided 1x1
    (2, 20, 9, 11, 36, 5, 3, 1, 2, 1),      # C % 16 != 0: the register-staged kernel
])
@pytest.mark.parametrize("use_bias", [False, True])
def test_conv_int32_written_as_nchw(capi, case, use_bias):
    """mxq_quantized_conv_nhwc_out_nchw == the NHWC convolution followed by the layout
    adapter, and both equal the oracle."""
    import ctypes
    import mxnet_amd
    lib = mxnet_amd._lib.lib
    N, C, H, W, O, KH, KW, stride, pad, dilate = case
    d = int8_uniform((N, C, H, W), seed=sum(case))
    w = int8_uniform((O, C, KH, KW), seed=sum(case) + 1)
    b = int8_uniform((O,), seed=3) if use_bias else None
    dn, wn = capi.nchw_to_nhwc_i8(dev(d)), capi.nchw_to_nhwc_i8(dev(w))
    eh, ew = dilate * (KH - 1) + 1, dilate * (KW - 1) + 1
    OH, OW = (H + 2 * pad - eh) // stride + 1, (W + 2 * pad - ew) // stride + 1
    out = torch.full((N, O, OH, OW), 12345, dtype=torch.int32, device="cuda")
    sc = [f32(v) for v in (-1.0, 1.0, -0.5, 0.5, -2.0, 2.0)]
    omin, omax = f32(0.0), f32(0.0)
    P = lambda t: ctypes.c_void_p(t.data_ptr()) if t is not None else None
    bd = dev(b) if use_bias else None
    st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    rc = lib.mxq_quantized_conv_nhwc_out_nchw(
        st, P(dn), P(wn), P(bd), N, H, W, C, O, KH, KW, stride, stride, pad, pad, dilate, dilate,
        P(sc[0]), P(sc[1]), P(sc[2]), P(sc[3]), P(sc[4]) if use_bias else None,
        P(sc[5]) if use_bias else None, P(out), P(omin), P(omax), None, 0)
    assert rc == 0, lib.mxq_last_error()
    ro, rmn, rmx = oracle.quantized_conv(d, w, b, -1.0, 1.0, -0.5, 0.5, -2.0 if use_bias else None,
                                         2.0 if use_bias else None, (stride, stride), (pad, pad),
                                         (dilate, dilate))
    np.testing.assert_array_equal(out.cpu().numpy(), ro)
    assert (omin.item(), omax.item()) == (rmn, rmx)


def test_conv_without_images_still_writes_its_range(capi):
    x = torch.zeros((0, 8, 8, 16), dtype=torch.int8, device="cuda")
    w = torch.ones((32, 3, 3, 16), dtype=torch.int8, device="cuda")
    f = lambda v: torch.tensor([v], dtype=torch.float32, device="cuda")
    res = capi.quantized_conv_nhwc(x, w, None, f(-1.0), f(1.0), f(-0.5), f(0.5), None, None,
                                   stride=(1, 1), pad=(1, 1))
    _, rmn, rmx = oracle.quantized_conv(np.zeros((0, 16, 8, 8), np.int8),
                                        np.ones((32, 16, 3, 3), np.int8), None, -1.0, 1.0, -0.5,
                                        0.5, pad=(1, 1))
    assert tuple(res["out32"].shape) == (0, 8, 8, 32)
    assert (res["omin"].item(), res["omax"].item()) == (rmn, rmx)


# Exact ties and saturation in the fused requantize of the convolution kernels (see the FC
# test of the same name): power-of-two scales, a centre-tap-only 3 x 3 window so that the
# accumulators sweep the small integers of both signs; the tiled kernel, the parked-weights
# kernel and the resident-patch kernel, each with and without the relu.
@pytest.mark.parametrize("C,O,force", [(64, 64, None), (64, 64, (61, 1)), (128, 128, (62, 1)),
                                       (32, 48, None)])
@pytest.mark.parametrize("relu", [False, True])
def test_conv_fused_requantize_on_exact_ties(capi, C, O, force, relu):
    N, H, W = 3, 12, 28
    d = np.zeros((N, C, H, W), np.int8)
    w = np.zeros((O, C, 3, 3), np.int8)
    px = np.arange(N * H * W).reshape(N, H, W)
    o = np.arange(O)
    d[:, 0] = (px * 37) % 256 - 128
    d[:, 1] = (px * 7) % 5 - 2
    d[:, 2] = 2
    w[:, 0, 1, 1] = 1
    w[:, 1, 1, 1] = (o % 64) - 32
    w[:, 2, 1, 1] = 127 * (o % 3 - 1)
    ro, rmn, rmx = oracle.quantized_conv(d, w, None, -127.0, 127.0, -127.0, 127.0, None, None,
                                         (1, 1), (1, 1), (1, 1))
    assert ro.min() < -255 and ro.max() > 255 and (ro % 2 != 0).sum() > ro.size // 4
    rq, qmn, qmx = oracle.requantize(ro, rmn, rmx, -254.0, 254.0)
    want = np.clip(np.sign(ro) * np.floor(np.abs(ro) / 2.0 + 0.5), -127, 127).astype(np.int8)
    np.testing.assert_array_equal(rq, want)
    if relu:
        rq = oracle.relu_i8(rq)
    res = run_conv_nchw(capi, d, w, None, 127.0, 127.0, 1.0, (1, 1), (1, 1), (1, 1),
                        calib=(-254.0, 254.0), relu=relu, force=force, want_int32=False)
    np.testing.assert_array_equal(res["out8_nchw"].cpu().numpy(), rq)
    assert (res["rmin"].item(), res["rmax"].item()) == (qmn, qmx)
