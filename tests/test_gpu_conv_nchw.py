"""Parity of mxq_quantized_conv_nchw (the convolution on the operator's own NCHW / OIHW
tensors, int32 NCHW out) with the CPU oracle: the 1x1 kernel that reads channel planes with
the transposing LDS load, its strided form, and the adapter route behind the same call."""
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


def run(capi, case, use_bias, cfg=None, guard=True):
    N, C, H, W, O, KH, KW, s, p, dl = case
    d = int8_uniform((N, C, H, W), seed=sum(case))
    w = int8_uniform((O, C, KH, KW), seed=sum(case) + 1)
    b = int8_uniform((O,), seed=O) if use_bias else None
    rd, rw, rb = 3.0, 0.2, 1.5
    eh, ew = dl * (KH - 1) + 1, dl * (KW - 1) + 1
    OH, OW = (H + 2 * p - eh) // s + 1, (W + 2 * p - ew) // s + 1
    # the output sits between two guard bands that must come back untouched
    n_out = N * O * OH * OW
    flat = torch.full((n_out + 512,), 0x5A5A5A5A, dtype=torch.int32, device="cuda")
    out = flat[256:256 + n_out].view(N, O, OH, OW)
    res = capi.quantized_conv_nchw(dev(d), dev(w), None if b is None else dev(b), f32(-rd),
                                   f32(rd), f32(-rw), f32(rw), None if b is None else f32(-rb),
                                   None if b is None else f32(rb), stride=(s, s), pad=(p, p),
                                   dilate=(dl, dl), cfg=cfg, out=out)
    ro, rmn, rmx = oracle.quantized_conv(d, w, b, -rd, rd, -rw, rw, None if b is None else -rb,
                                         None if b is None else rb, (s, s), (p, p), (dl, dl))
    np.testing.assert_array_equal(res["out32"].cpu().numpy(), ro)
    assert (res["omin"].item(), res["omax"].item()) == (rmn, rmx)
    g = flat.cpu().numpy()
    assert (g[:256] == 0x5A5A5A5A).all() and (g[256 + n_out:] == 0x5A5A5A5A).all()
    return res


# (N, C, H, W, O, KH, KW, stride, pad, dilate): 1x1 layers whose planes are whole 16-byte runs
PLANE_CASES = [
    (2, 64, 56, 56, 64, 1, 1, 1, 0, 1),     # ResNet stage 1: 3136-pixel planes, one K stage
    (2, 64, 56, 56, 256, 1, 1, 1, 0, 1),
    (2, 256, 56, 56, 64, 1, 1, 1, 0, 1),    # four K stages
    (3, 128, 28, 28, 512, 1, 1, 1, 0, 1),   # 784-pixel planes: the last tile is 16 pixels
    (2, 512, 28, 28, 128, 1, 1, 1, 0, 1),
    (3, 48, 8, 12, 40, 1, 1, 1, 0, 1),      # K tail (48 of 64 channels), O % 32 != 0, 96 pixels
    (1, 16, 4, 4, 8, 1, 1, 1, 0, 1),        # one 16-pixel chunk, everything smaller than a tile
    (5, 80, 16, 16, 136, 1, 1, 1, 0, 1),    # two K stages with a tail, O one past a tile
]


@pytest.mark.parametrize("case", PLANE_CASES)
@pytest.mark.parametrize("use_bias", [False, True])
def test_conv_nchw_planes(capi, case, use_bias):
    res = run(capi, case, use_bias)
    assert res["workspace_bytes"] == 0  # nothing is copied for a unit-stride 1x1 layer


@pytest.mark.parametrize("cfg", [71, 72, 73, 74, 75, 77, 78, 84])
@pytest.mark.parametrize("case", [PLANE_CASES[2], PLANE_CASES[3], PLANE_CASES[5], PLANE_CASES[7],
                                  (3, 320, 7, 7, 200, 1, 1, 1, 0, 1),
                                  (2, 1024, 14, 14, 136, 1, 1, 1, 0, 1)])
def test_conv_nchw_every_plane_tile(capi, cfg, case):
    run(capi, case, True, cfg=cfg)


STRIDED_CASES = [
    (2, 256, 56, 56, 128, 1, 1, 2, 0, 1),   # ResNet downsampling: 28 x 28 = 784 output pixels
    (2, 256, 56, 56, 512, 1, 1, 2, 0, 1),
    (2, 32, 16, 24, 48, 1, 1, 2, 0, 1),     # 8 x 12 output
    (2, 32, 15, 31, 48, 1, 1, 2, 0, 1),     # odd extents: 8 x 16 output, rows off the dword marks
    (1, 16, 24, 24, 16, 1, 1, 3, 0, 1),     # stride 3: the byte-wise gather
    (2, 256, 14, 14, 1024, 1, 1, 1, 0, 1),  # 196-pixel planes moved to a pitch of 208 bytes
    (2, 512, 28, 28, 256, 1, 1, 2, 0, 1),   # 28 -> 14: dword gather, 196 of 208
    (2, 1024, 14, 14, 512, 1, 1, 2, 0, 1),  # 14 -> 7: 49-pixel planes, pitch 64
    (3, 512, 7, 7, 2048, 1, 1, 1, 0, 1),    # 7 x 7 planes repacked, O in 256-wide tiles
    (2, 48, 5, 3, 40, 1, 1, 1, 0, 1),       # 15 pixels
    (2, 16, 9, 7, 24, 1, 1, (2), 0, 1),     # 5 x 4 = 20 pixels
    (3, 32, 12, 12, 72, 1, 1, 2, 0, 1),     # 6 x 6: pairs of pixels, 36 per plane
    (2, 64, 20, 12, 32, 1, 1, 2, 0, 1),     # 10 x 6
]


@pytest.mark.parametrize("case", STRIDED_CASES)
def test_conv_nchw_strided_planes(capi, case):
    res = run(capi, case, True)
    N, C, H, W, O, _, _, s = case[:8]
    OH, OW = (H - 1) // s + 1, (W - 1) // s + 1
    dwords = s == 1 and (H * W) % 4 == 0
    pairs = s == 2 and OW % 4 == 0 and (s * W) % 8 == 0 and (H * W) % 8 == 0 and 2 * OW <= W
    pairs2 = s == 2 and OW % 2 == 0 and (s * W) % 4 == 0 and (H * W) % 4 == 0 and 2 * OW <= W
    if (dwords or pairs or pairs2) and O * C <= 256 * 1024:
        assert res["workspace_bytes"] == 0  # the kernel's loader gathers: no pre-pass, no copy
    else:
        row = (N * ((OH * OW + 3) // 4 * 4) + 15) // 16 * 16  # one row per channel over the batch
        assert res["workspace_bytes"] == (C * row + 255) // 256 * 256  # the pixels it reads, once


# everything else goes through the adapters inside the same call
ADAPTER_CASES = [
    (3, 4, 28, 28, 128, 3, 3, 1, 1, 1),     # the reference's test shape
    (2, 64, 56, 56, 64, 3, 3, 1, 1, 1),
    (2, 128, 28, 28, 128, 3, 3, 1, 1, 1),
    (1, 3, 32, 32, 16, 7, 7, 2, 3, 1),      # stem: space-to-depth route
    (2, 20, 9, 11, 36, 5, 3, 1, 2, 1),      # C % 16 != 0
    (2, 24, 8, 8, 32, 1, 1, 1, 0, 1),       # 1x1 with C % 16 != 0
    (2, 16, 8, 8, 32, 1, 1, 1, 1, 1),       # padded 1x1
    (1, 16, 12, 12, 20, 3, 3, 1, 2, 2),     # dilation
]


@pytest.mark.parametrize("case", ADAPTER_CASES)
@pytest.mark.parametrize("use_bias", [False, True])
def test_conv_nchw_other_geometries(capi, case, use_bias):
    run(capi, case, use_bias)


# 3 x 3 over 64 -> 64 channels with many rows behind the adapters (more than 8192 output
# pixels: int32 planes from the tiled kernel's many tiles), rows longer than one MFMA tile,
# an odd last row
@pytest.mark.parametrize("case", [(74, 64, 28, 8, 64, 3, 3, 1, 1, 1), (90, 64, 28, 8, 64, 3, 3, 1, 1, 1),
                                  (100, 64, 21, 33, 64, 3, 3, 1, 1, 1),
                                  (120, 64, 21, 33, 64, 3, 3, 1, 1, 1)])
@pytest.mark.parametrize("use_bias", [False, True])
def test_conv_nchw_3x3_64_channels_many_rows(capi, case, use_bias):
    run(capi, case, use_bias)


@pytest.mark.parametrize("case", [PLANE_CASES[0], PLANE_CASES[3], STRIDED_CASES[0]])
def test_conv_nchw_routes_agree(capi, case):
    """The NCHW kernel and the adapter route (pinned through the test-only entry point)
    write the same tensor."""
    a = run(capi, case, True)
    b = run(capi, case, True, cfg=1)
    assert torch.equal(a["out32"], b["out32"])


def test_conv_nchw_unaligned_operands_take_the_adapters(capi):
    """A data pointer off the 16-byte marks cannot feed the direct-to-LDS loads."""
    case = (2, 64, 8, 8, 64, 1, 1, 1, 0, 1)
    N, C, H, W, O = case[:5]
    d = int8_uniform((N, C, H, W), seed=1)
    w = int8_uniform((O, C, 1, 1), seed=2)
    buf = torch.zeros(d.size + 16, dtype=torch.int8, device="cuda")
    view = buf[4:4 + d.size].view(N, C, H, W)
    view.copy_(dev(d))
    res = capi.quantized_conv_nchw(view, dev(w), None, f32(-1.0), f32(1.0), f32(-1.0), f32(1.0))
    ro, _, _ = oracle.quantized_conv(d, w, None, -1.0, 1.0, -1.0, 1.0)
    np.testing.assert_array_equal(res["out32"].cpu().numpy(), ro)


def test_conv_nchw_output_off_the_16_byte_marks(capi):
    """An int32 output that starts 4 bytes past a 16-byte mark takes the dword stores."""
    case = (2, 64, 8, 8, 96, 1, 1, 1, 0, 1)
    N, C, H, W, O = case[:5]
    d = int8_uniform((N, C, H, W), seed=5)
    w = int8_uniform((O, C, 1, 1), seed=6)
    flat = torch.zeros(N * O * H * W + 8, dtype=torch.int32, device="cuda")
    out = flat[1:1 + N * O * H * W].view(N, O, H, W)
    res = capi.quantized_conv_nchw(dev(d), dev(w), None, f32(-1.0), f32(1.0), f32(-1.0), f32(1.0),
                                   out=out)
    ro, _, _ = oracle.quantized_conv(d, w, None, -1.0, 1.0, -1.0, 1.0)
    np.testing.assert_array_equal(res["out32"].cpu().numpy(), ro)
    assert flat[0].item() == 0 and flat[-1].item() == 0


def test_conv_nchw_without_images(capi):
    x = torch.zeros((0, 16, 8, 8), dtype=torch.int8, device="cuda")
    w = torch.ones((32, 16, 1, 1), dtype=torch.int8, device="cuda")
    res = capi.quantized_conv_nchw(x, w, None, f32(-1.0), f32(1.0), f32(-0.5), f32(0.5))
    _, rmn, rmx = oracle.quantized_conv(np.zeros((0, 16, 8, 8), np.int8),
                                        np.ones((32, 16, 1, 1), np.int8), None, -1.0, 1.0, -0.5,
                                        0.5)
    assert tuple(res["out32"].shape) == (0, 32, 8, 8)
    assert (res["omin"].item(), res["omax"].item()) == (rmn, rmx)


def test_conv_nchw_refuses_what_it_cannot_run(capi):
    """Error behaviour of the entry point: a workspace smaller than the query's answer, a
    missing range pointer, a window larger than the padded input; the output stays
    untouched."""
    import ctypes
    import mxnet_amd
    lib = mxnet_amd._lib.lib
    P = lambda t: ctypes.c_void_p(t.data_ptr()) if t is not None else None
    N, C, H, W, O = 2, 32, 9, 11, 40
    d = dev(int8_uniform((N, C, H, W), seed=1))
    w = dev(int8_uniform((O, C, 3, 3), seed=2))
    out = torch.full((N, O, H, W), 7, dtype=torch.int32, device="cuda")
    r = [f32(0.0), f32(0.0)]
    one = [f32(-1.0), f32(1.0)]
    geo = (N, C, H, W, O, 3, 3, 1, 1, 1, 1, 1, 1)
    need = lib.mxq_quantized_conv_nchw_workspace(*geo, 1)
    assert need > 0
    ws = torch.empty(need, dtype=torch.uint8, device="cuda")
    st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)

    def call(geo, ranges, ws_ptr, ws_bytes):
        return lib.mxq_quantized_conv_nchw(st, P(d), P(w), None, *geo, *ranges, None, None, P(out),
                                           P(r[0]), P(r[1]), ws_ptr, ws_bytes)

    ok_ranges = (P(one[0]), P(one[1]), P(one[0]), P(one[1]))
    assert call(geo, ok_ranges, P(ws), need - 16) != 0
    assert b"workspace too small" in lib.mxq_last_error()
    assert call(geo, ok_ranges, None, 0) != 0
    assert call(geo, (None, P(one[1]), P(one[0]), P(one[1])), P(ws), need) != 0
    assert b"range pointer" in lib.mxq_last_error()
    big = (N, C, H, W, O, 13, 3, 1, 1, 1, 1, 1, 1)       # 13 rows over 9 + 2
    assert call(big, ok_ranges, P(ws), need) != 0
    assert b"kernel larger than padded input" in lib.mxq_last_error()
    torch.cuda.synchronize()
    assert bool((out == 7).all())
    assert call(geo, ok_ranges, P(ws), need) == 0        # and the same call with its workspace runs
    torch.cuda.synchronize()
    assert not bool((out == 7).all())
