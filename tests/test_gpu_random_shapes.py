"""Seeded random shapes through the operators' own entry points (the launcher chooses the
kernel): every route the tile chooser can take for small and mid-size problems, with ragged
extents, K tails, stride / pad / dilation mixes, against the CPU oracle bit for bit."""
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


def fc_shapes():
    rng = np.random.default_rng(20240611)
    shapes = []
    for _ in range(60):
        M = int(rng.integers(1, 700))
        N = int(rng.integers(1, 700))
        K = int(rng.choice([rng.integers(1, 300), 16 * rng.integers(1, 40), 64 * rng.integers(1, 24)]))
        shapes.append((M, N, K))
    # chooser corner cases: widths that are multiples of 192, tall and narrow, few tiles
    # under a long K (split-K with the workspace the entry point asks for), one row
    shapes += [(512, 384, 512), (300, 192, 1024), (2048, 64, 64), (4100, 128, 128),
               (64, 320, 8192), (40, 130, 9000), (1, 1000, 4096), (700, 1, 48)]
    # either side of the row count from which the int8 tiles are written with streaming
    # stores (8192), ragged there, through the tiled, the short-K and the fallback kernels
    shapes += [(8191, 64, 48), (8192, 128, 64), (8200, 80, 256), (9000, 256, 64),
               (33000, 64, 128), (8193, 100, 37)]
    return shapes


@pytest.mark.parametrize("M,N,K", fc_shapes())
def test_fc_random_shape(capi, M, N, K):
    d = int8_uniform((M, K), seed=M * 7 + K)
    w = int8_uniform((N, K), seed=N * 5 + K + 1)
    b = int8_uniform((N,), seed=N + 3) if (M + N + K) % 3 else None
    rd, rw, rb = 1.5, 0.2, 0.7
    relu = bool((M + K) % 2)
    ro, rmn, rmx = oracle.quantized_fully_connected(d, w, b, -rd, rd, -rw, rw,
                                                    None if b is None else -rb,
                                                    None if b is None else rb)
    fl = ro.astype(np.float64) * (float(rmx) / 2147483648.0)
    R = float(np.percentile(np.abs(fl), 97.0)) or 1.0   # 3 % of the outputs saturate
    res = capi.quantized_fc(dev(d), dev(w), None if b is None else dev(b), f32(-rd), f32(rd),
                            f32(-rw), f32(rw), None if b is None else f32(-rb),
                            None if b is None else f32(rb), want_int32=True,
                            calib=(-R, 0.8 * R), relu=relu)
    np.testing.assert_array_equal(res["out32"].cpu().numpy(), ro)
    assert (res["omin"].item(), res["omax"].item()) == (rmn, rmx)
    rq, qmn, qmx = oracle.requantize(ro, rmn, rmx, -R, 0.8 * R)
    if relu:
        rq = oracle.relu_i8(rq)
    np.testing.assert_array_equal(res["out8"].cpu().numpy(), rq)
    assert (res["rmin"].item(), res["rmax"].item()) == (qmn, qmx)
    # the fused form alone (no int32 output) takes other kernels for some shapes
    res8 = capi.quantized_fc(dev(d), dev(w), None if b is None else dev(b), f32(-rd), f32(rd),
                             f32(-rw), f32(rw), None if b is None else f32(-rb),
                             None if b is None else f32(rb), want_int32=False,
                             calib=(-R, 0.8 * R), relu=relu)
    np.testing.assert_array_equal(res8["out8"].cpu().numpy(), rq)
    # requantize and dequantize both in the launch: the float the three operators give
    resf = capi.quantized_fc_f32(dev(d), dev(w), None if b is None else dev(b), f32(-rd), f32(rd),
                                 f32(-rw), f32(rw), None if b is None else f32(-rb),
                                 None if b is None else f32(rb), calib=(-R, 0.8 * R), relu=relu)
    ref = oracle.dequantize(rq, qmn, qmx)
    np.testing.assert_array_equal(resf["outf"].cpu().numpy().view(np.uint32), ref.view(np.uint32))
    assert (resf["rmin"].item(), resf["rmax"].item()) == (qmn, qmx)
    # the residual sum (and its relu) behind the requantization
    res8 = int8_uniform((M, N), seed=M + N + 9)
    ro2, _, _ = oracle.requantize(ro, rmn, rmx, -R, 0.8 * R)       # no relu before the sum
    sref, smn, smx = oracle.quantized_elemwise_add(ro2, res8, qmn, qmx, -0.6 * R, 0.6 * R,
                                                   min_calib_range=-R, max_calib_range=1.1 * R)
    if relu:
        sref = oracle.relu_i8(sref)
    ress = capi.quantized_fc_sum(dev(d), dev(w), None if b is None else dev(b), dev(res8),
                                 f32(-rd), f32(rd), f32(-rw), f32(rw),
                                 None if b is None else f32(-rb), None if b is None else f32(rb),
                                 f32(-0.6 * R), f32(0.6 * R), (-R, 0.8 * R), (-R, 1.1 * R),
                                 sum_relu=relu)
    np.testing.assert_array_equal(ress["out8"].cpu().numpy(), sref)
    assert (ress["rmin"].item(), ress["rmax"].item()) == (smn, smx)


def conv_cases():
    rng = np.random.default_rng(77)
    cases = []
    while len(cases) < 40:
        N = int(rng.integers(1, 4))
        C = int(rng.choice([3, 4, 16, 20, 32, 48, 64, 128]))
        H = int(rng.integers(3, 20))
        W = int(rng.integers(3, 20))
        O = int(rng.choice([8, 24, 64, 70, 128, 200]))
        KH = int(rng.choice([1, 3, 5]))
        KW = int(rng.choice([1, 3]))
        s = int(rng.choice([1, 2]))
        p = int(rng.integers(0, 3))
        dl = int(rng.choice([1, 1, 2]))
        if (H + 2 * p - dl * (KH - 1) - 1) < 0 or (W + 2 * p - dl * (KW - 1) - 1) < 0:
            continue
        cases.append((N, C, H, W, O, KH, KW, s, p, dl))
    # more than 8192 output pixels: the streaming-store flavour of the tiled kernels, ragged
    # last tiles
    cases += [(3, 16, 64, 64, 32, 3, 3, 1, 1, 1), (2, 64, 70, 58, 64, 3, 3, 1, 1, 1),
              (5, 32, 45, 41, 48, 1, 1, 1, 0, 1), (9, 64, 62, 60, 24, 3, 3, 2, 1, 1)]
    return cases


@pytest.mark.parametrize("case", conv_cases())
def test_conv_random_geometry(capi, case):
    N, C, H, W, O, KH, KW, s, p, dl = case
    d = int8_uniform((N, C, H, W), seed=C + H * 3 + W)
    w = int8_uniform((O, C, KH, KW), seed=O + KH + 11)
    b = int8_uniform((O,), seed=O + 1) if (N + C + O) % 2 else None
    relu = bool((H + W) % 2)
    ro, rmn, rmx = oracle.quantized_conv(d, w, b, -1.0, 1.0, -1.0, 1.0,
                                         None if b is None else -1.0,
                                         None if b is None else 1.0, (s, s), (p, p), (dl, dl))
    fl = ro.astype(np.float64) * (float(rmx) / 2147483648.0)
    R = float(np.percentile(np.abs(fl), 97.0)) or 1.0
    dn, wn = capi.nchw_to_nhwc_i8(dev(d)), capi.nchw_to_nhwc_i8(dev(w))
    one = [f32(-1.0), f32(1.0)]
    res = capi.quantized_conv_nhwc(dn, wn, None if b is None else dev(b), one[0], one[1], one[0],
                                   one[1], None if b is None else one[0],
                                   None if b is None else one[1], stride=(s, s), pad=(p, p),
                                   dilate=(dl, dl), calib=(-R, 0.8 * R), relu=relu,
                                   want_int32=True)
    np.testing.assert_array_equal(capi.nhwc_to_nchw(res["out32"]).cpu().numpy(), ro)
    rq, qmn, qmx = oracle.requantize(ro, rmn, rmx, -R, 0.8 * R)
    if relu:
        rq = oracle.relu_i8(rq)
    np.testing.assert_array_equal(capi.nhwc_to_nchw(res["out8"]).cpu().numpy(), rq)
    assert (res["omin"].item(), res["omax"].item()) == (rmn, rmx)
    assert (res["rmin"].item(), res["rmax"].item()) == (qmn, qmx)


def conv_nchw_cases():
    """Mostly unpadded 1 x 1 layers (the routes of the NCHW kernel: whole planes, the
    gathering loaders, the pre-pass), planes of every residue mod 16, strides 1-3 alone and
    mixed, batches large enough for pixel tiles to run across several images; a few padded
    and 3 x 3 geometries for the adapters behind the same call."""
    rng = np.random.default_rng(2024)
    cases = []
    while len(cases) < 56:
        one = rng.random() < 0.8
        N = int(rng.choice([1, 2, 3, 5, 17, 40]))
        C = int(rng.choice([16, 32, 48, 64, 80, 128, 272, 512, 20]))
        H = int(rng.integers(1, 30))
        W = int(rng.integers(1, 30))
        O = int(rng.choice([8, 24, 64, 72, 128, 136, 264]))
        KH, KW = (1, 1) if one else (int(rng.choice([1, 3])), int(rng.choice([1, 3])))
        sh, sw = int(rng.choice([1, 1, 2, 2, 3])), int(rng.choice([1, 1, 2, 2, 3]))
        p = 0 if one else int(rng.integers(0, 2))
        if H + 2 * p < KH or W + 2 * p < KW or N * C * H * W > (3 << 20):
            continue
        cases.append((N, C, H, W, O, KH, KW, sh, sw, p))
    return cases


@pytest.mark.parametrize("case", conv_nchw_cases())
def test_conv_nchw_random_geometry(capi, case):
    N, C, H, W, O, KH, KW, sh, sw, p = case
    d = int8_uniform((N, C, H, W), seed=C + H * 3 + W)
    w = int8_uniform((O, C, KH, KW), seed=O + KH + 11)
    b = int8_uniform((O,), seed=O + 1) if (N + C + O + H) % 2 else None
    ro, rmn, rmx = oracle.quantized_conv(d, w, b, -2.0, 2.0, -0.5, 0.5,
                                         None if b is None else -1.0,
                                         None if b is None else 1.0, (sh, sw), (p, p), (1, 1))
    res = capi.quantized_conv_nchw(dev(d), dev(w), None if b is None else dev(b), f32(-2.0),
                                   f32(2.0), f32(-0.5), f32(0.5),
                                   None if b is None else f32(-1.0),
                                   None if b is None else f32(1.0), stride=(sh, sw), pad=(p, p))
    np.testing.assert_array_equal(res["out32"].cpu().numpy(), ro)
    assert (res["omin"].item(), res["omax"].item()) == (rmn, rmx)
    # the route through the layout adapters writes the same tensor
    alt = capi.quantized_conv_nchw(dev(d), dev(w), None if b is None else dev(b), f32(-2.0),
                                   f32(2.0), f32(-0.5), f32(0.5),
                                   None if b is None else f32(-1.0),
                                   None if b is None else f32(1.0), stride=(sh, sw), pad=(p, p),
                                   cfg=1)
    assert torch.equal(res["out32"], alt["out32"])
