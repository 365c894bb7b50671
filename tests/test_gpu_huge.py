"""Tensors past the 32-bit marks: more than 2^32 elements through the casts, the relu, the
element-wise sum, concat and transpose, operands and outputs of 2 GiB and more through the fully-connected and
convolution launchers (the direct-to-LDS kernels address operands with 32-bit offsets, so
the launchers must route these elsewhere).  The oracle recomputes windows that sit on the
marks (start, 2^31, 2^32, end); every other element is covered by a size-independent
property: a cast of element i does not depend on i, so the big call must equal the same
entry point called on each 2^26-element (or row-block) piece."""
import numpy as np
import pytest
import torch

import oracle

pytestmark = pytest.mark.gpu

N_BIG = (1 << 32) + 4099          # ragged: not a multiple of 4
WIN = 1 << 18
PIECE = 1 << 26


@pytest.fixture(scope="module")
def capi():
    import mxnet_amd
    return mxnet_amd.capi


@pytest.fixture(scope="module")
def contrib():
    import mxnet_amd
    return mxnet_amd.contrib


@pytest.fixture(autouse=True)
def release_memory():
    yield
    torch.cuda.empty_cache()


def f32(v):
    return torch.tensor([v], dtype=torch.float32, device="cuda")


def windows(n):
    marks = [0, (1 << 31) - WIN // 2, (1 << 32) - WIN // 2, n - WIN]
    return [(s, s + WIN) for s in marks if 0 <= s and s + WIN <= n]


def pieces(n):
    return [(s, min(s + PIECE, n)) for s in range(0, n, PIECE)]


def big_floats():
    g = torch.Generator(device="cuda").manual_seed(5)
    x = torch.empty(N_BIG, dtype=torch.float32, device="cuda")
    x.normal_(generator=g)
    x.clamp_(-4.0, 4.0)
    return x


def test_quantize_v2_past_4g_elements(capi):
    x = big_floats()
    # the extremes sit behind the 2^32 mark and in the ragged tail
    x[(1 << 32) + 1] = 7.25
    x[N_BIG - 2] = -9.5
    q, mn, mx = capi.quantize_v2(x, "int8", min_calib_range=-9.5, max_calib_range=7.25)
    torch.cuda.synchronize()
    assert (mn.item(), mx.item()) == (-9.5, 9.5)
    for a, b in windows(N_BIG):
        ref, rmn, rmx = oracle.quantize_v2(x[a:b].cpu().numpy(), "int8", -9.5, 7.25)
        np.testing.assert_array_equal(q[a:b].cpu().numpy(), ref, err_msg=f"window {a}")
        assert (rmn, rmx) == (-9.5, 9.5)
    for a, b in pieces(N_BIG):
        part, _, _ = capi.quantize_v2(x[a:b], "int8", min_calib_range=-9.5, max_calib_range=7.25)
        assert torch.equal(q[a:b], part), f"piece at {a}"
    # uncalibrated: the reduction must see both planted extremes
    qu, umn, umx = capi.quantize_v2(x, "int8")
    torch.cuda.synchronize()
    assert (umn.item(), umx.item()) == (-9.5, 9.5)
    assert torch.equal(qu, q)
    del qu
    # uint8 over the observed range
    q8, mn8, mx8 = capi.quantize_v2(x, "uint8")
    torch.cuda.synchronize()
    assert (mn8.item(), mx8.item()) == (-9.5, 7.25)
    for a, b in windows(N_BIG):
        ref, _, _ = oracle.quantize_v2(x[a:b].cpu().numpy(), "uint8", -9.5, 7.25)
        np.testing.assert_array_equal(q8[a:b].cpu().numpy(), ref, err_msg=f"uint8 window {a}")


def test_dequantize_past_4g_elements(capi):
    g = torch.Generator(device="cuda").manual_seed(6)
    q = torch.randint(-127, 128, (N_BIG,), dtype=torch.int8, device="cuda", generator=g)
    out = capi.dequantize(q, f32(-3.0), f32(2.5))
    torch.cuda.synchronize()
    for a, b in windows(N_BIG):
        ref = oracle.dequantize(q[a:b].cpu().numpy(), -3.0, 2.5)
        got = out[a:b].cpu().numpy()
        assert got.tobytes() == ref.tobytes(), f"window {a}"
    for a, b in pieces(N_BIG):
        assert torch.equal(out[a:b], capi.dequantize(q[a:b], f32(-3.0), f32(2.5))), f"piece {a}"


def test_requantize_past_4g_elements(capi):
    g = torch.Generator(device="cuda").manual_seed(7)
    v = torch.randint(-(1 << 24), 1 << 24, (N_BIG,), dtype=torch.int32, device="cuda",
                      generator=g)
    v[(1 << 32) + 5] = (1 << 28) + 12345       # the largest magnitude, behind the mark
    v[N_BIG - 1] = -(1 << 27)
    lo, hi = -5000.0, 5000.0
    # calibrated
    real = 5000.0 * ((1 << 26) / 2147483648.0)
    q, mn, mx = capi.requantize(v, f32(lo), f32(hi), min_calib_range=-real,
                                max_calib_range=0.5 * real)
    torch.cuda.synchronize()
    for a, b in windows(N_BIG):
        ref, rmn, rmx = oracle.requantize(v[a:b].cpu().numpy(), lo, hi, -real, 0.5 * real)
        np.testing.assert_array_equal(q[a:b].cpu().numpy(), ref, err_msg=f"window {a}")
        assert (mn.item(), mx.item()) == (rmn, rmx)
    for a, b in pieces(N_BIG):
        part, _, _ = capi.requantize(v[a:b], f32(lo), f32(hi), min_calib_range=-real,
                                     max_calib_range=0.5 * real)
        assert torch.equal(q[a:b], part), f"piece at {a}"
    del q
    # uncalibrated: the range comes from the planted element; a window that holds it gives
    # the oracle the same extremes
    qu, umn, umx = capi.requantize(v, f32(lo), f32(hi))
    torch.cuda.synchronize()
    a = (1 << 32) - WIN // 2
    ref, rmn, rmx = oracle.requantize(v[a:a + WIN].cpu().numpy(), lo, hi)
    assert (umn.item(), umx.item()) == (rmn, rmx)
    np.testing.assert_array_equal(qu[a:a + WIN].cpu().numpy(), ref)
    tail, _, _ = oracle.requantize(
        np.concatenate([v[N_BIG - 4096:].cpu().numpy(), v[(1 << 32) + 5:(1 << 32) + 6].cpu().numpy()]),
        lo, hi)
    np.testing.assert_array_equal(qu[N_BIG - 4096:].cpu().numpy(), tail[:4096])


def test_elemwise_add_past_4g_elements(contrib):
    g = torch.Generator(device="cuda").manual_seed(8)
    a8 = torch.randint(-127, 128, (N_BIG,), dtype=torch.int8, device="cuda", generator=g)
    b8 = torch.randint(-127, 128, (N_BIG,), dtype=torch.int8, device="cuda", generator=g)
    rng = (-1.5, 1.5, -0.75, 0.5)
    scal = [f32(r) for r in rng]
    for kw in ({}, {"min_calib_range": -2.0, "max_calib_range": 2.0}):
        out, mn, mx = contrib.quantized_elemwise_add(a8, b8, *scal, **kw)
        torch.cuda.synchronize()
        for s, e in windows(N_BIG):
            ref, rmn, rmx = oracle.quantized_elemwise_add(a8[s:e].cpu().numpy(),
                                                          b8[s:e].cpu().numpy(), *rng, **kw)
            np.testing.assert_array_equal(out[s:e].cpu().numpy(), ref, err_msg=f"window {s}")
            assert (mn.item(), mx.item()) == (rmn, rmx)
        for s, e in pieces(N_BIG):
            part, _, _ = contrib.quantized_elemwise_add(a8[s:e], b8[s:e], *scal, **kw)
            assert torch.equal(out[s:e], part), f"piece at {s}"
        del out


def test_quantized_act_past_4g_elements(contrib):
    g = torch.Generator(device="cuda").manual_seed(12)
    x = torch.randint(-128, 128, (N_BIG,), dtype=torch.int8, device="cuda", generator=g)
    out, mn, mx = contrib.quantized_act(x, f32(-2.0), f32(3.0), act_type="relu")
    torch.cuda.synchronize()
    assert (mn.item(), mx.item()) == (-2.0, 3.0)
    for s, e in windows(N_BIG):
        np.testing.assert_array_equal(out[s:e].cpu().numpy(), oracle.relu_i8(x[s:e].cpu().numpy()),
                                      err_msg=f"window {s}")
    for s, e in pieces(N_BIG):
        assert torch.equal(out[s:e], torch.clamp(x[s:e], min=0)), f"piece at {s}"


def test_concat_past_4g_bytes(contrib):
    """Two rows of two inputs, 2^30 + 4096 + 16 bytes per row and input: the output passes
    2^32 bytes, one input is rescaled to the hull of the ranges and one is copied."""
    L = (1 << 30) + 4096 + 16
    g = torch.Generator(device="cuda").manual_seed(13)
    a = torch.randint(-128, 128, (2, L), dtype=torch.int8, device="cuda", generator=g)
    b = torch.randint(-128, 128, (2, L), dtype=torch.int8, device="cuda", generator=g)
    rng = [(-1.0, 0.5), (-2.0, 2.0)]
    scal = [f32(v) for r in rng for v in r]
    out, mn, mx = contrib.quantized_concat(a, b, *scal, num_args=2, dim=1)
    torch.cuda.synchronize()
    assert tuple(out.shape) == (2, 2 * L)
    for s in (0, (1 << 29), L - WIN):
        cols = slice(s, s + WIN)
        ref, rmn, rmx = oracle.quantized_concat([a[:, cols].cpu().numpy(), b[:, cols].cpu().numpy()],
                                                [r[0] for r in rng], [r[1] for r in rng], dim=1)
        assert (mn.item(), mx.item()) == (rmn, rmx)
        got = torch.cat([out[:, cols], out[:, L + s:L + s + WIN]], dim=1)
        np.testing.assert_array_equal(got.cpu().numpy(), ref, err_msg=f"columns from {s}")
    step = 1 << 26
    for s in range(0, L, step):
        cols = slice(s, min(s + step, L))
        part, _, _ = contrib.quantized_concat(a[:, cols].contiguous(), b[:, cols].contiguous(),
                                              *scal, num_args=2, dim=1)
        w = part.shape[1] // 2
        assert torch.equal(out[:, cols], part[:, :w]), f"first input, columns from {s}"
        assert torch.equal(out[:, L + cols.start:L + cols.stop], part[:, w:]), \
            f"second input, columns from {s}"


def test_transpose_past_4g_bytes(contrib):
    """(batch, seq, heads, 64) -> (batch, heads, seq, 64) over more than 2^32 bytes: pure byte
    movement, so torch's own permute is an independent check of every byte; the oracle
    recomputes the first and the last batch entry."""
    shape = (33, 4096, 512, 64)
    g = torch.Generator(device="cuda").manual_seed(14)
    x = torch.randint(-128, 128, shape, dtype=torch.int8, device="cuda", generator=g)
    out, mn, mx = contrib.quantized_transpose(x, f32(-1.5), f32(2.5), axes=(0, 2, 1, 3))
    torch.cuda.synchronize()
    assert tuple(out.shape) == (33, 512, 4096, 64)
    for n in (0, 32):
        ref, rmn, rmx = oracle.quantized_transpose(x[n:n + 1].cpu().numpy(), -1.5, 2.5, (0, 2, 1, 3))
        np.testing.assert_array_equal(out[n:n + 1].cpu().numpy(), ref, err_msg=f"batch entry {n}")
        assert (mn.item(), mx.item()) == (rmn, rmx)
    for n in range(shape[0]):
        assert torch.equal(out[n], x[n].permute(1, 0, 2)), f"batch entry {n}"


def fc_reference(d, w, b, rows, calib, relu):
    ro, rmn, rmx = oracle.quantized_fully_connected(d[rows].cpu().numpy(), w.cpu().numpy(),
                                                    b.cpu().numpy(), -1.0, 1.0, -0.5, 0.5,
                                                    -0.25, 0.25)
    rq, qmn, qmx = oracle.requantize(ro, rmn, rmx, *calib)
    if relu:
        rq = oracle.relu_i8(rq)
    return ro, rq, (rmn, rmx), (qmn, qmx)


def test_fc_data_operand_over_2gib(capi):
    """[2^21 + 5, 1024] int8 data (2 GiB + 5 KiB): too large for 32-bit operand offsets."""
    M, K, N = (1 << 21) + 5, 1024, 96
    g = torch.Generator(device="cuda").manual_seed(9)
    d = torch.randint(-127, 128, (M, K), dtype=torch.int8, device="cuda", generator=g)
    w = torch.randint(-127, 128, (N, K), dtype=torch.int8, device="cuda", generator=g)
    b = torch.randint(-127, 128, (N,), dtype=torch.int8, device="cuda", generator=g)
    ranges = [f32(-1.0), f32(1.0), f32(-0.5), f32(0.5), f32(-0.25), f32(0.25)]
    calib = (-12.0, 10.0)      # a few percent of the outputs saturate
    res = capi.quantized_fc(d, w, b, *ranges, want_int32=True, calib=calib, relu=False)
    torch.cuda.synchronize()
    for rows in (slice(0, 300), slice((1 << 21) - 300, M)):
        ro, rq, r32, r8 = fc_reference(d, w, b, rows, calib, False)
        np.testing.assert_array_equal(res["out32"][rows].cpu().numpy(), ro)
        np.testing.assert_array_equal(res["out8"][rows].cpu().numpy(), rq)
        assert (res["omin"].item(), res["omax"].item()) == r32
        assert (res["rmin"].item(), res["rmax"].item()) == r8
    # every row against the same launcher on row blocks that fit the direct-to-LDS kernels
    step = 1 << 19
    for r0 in range(0, M, step):
        blk = slice(r0, min(r0 + step, M))
        part = capi.quantized_fc(d[blk], w, b, *ranges, want_int32=True, calib=calib, relu=False)
        assert torch.equal(res["out32"][blk], part["out32"]), f"rows from {r0}"
        assert torch.equal(res["out8"][blk], part["out8"]), f"rows from {r0}"


def test_fc_short_k_output_over_2gib(capi):
    """[2^25 + 7, 64] x [64, 64]: 2 GiB of data and of int8 output through the streaming
    kernel (fused int8 output only)."""
    M, K, N = (1 << 25) + 7, 64, 64
    g = torch.Generator(device="cuda").manual_seed(10)
    d = torch.randint(-127, 128, (M, K), dtype=torch.int8, device="cuda", generator=g)
    w = torch.randint(-127, 128, (N, K), dtype=torch.int8, device="cuda", generator=g)
    b = torch.randint(-127, 128, (N,), dtype=torch.int8, device="cuda", generator=g)
    ranges = [f32(-1.0), f32(1.0), f32(-0.5), f32(0.5), f32(-0.25), f32(0.25)]
    calib = (-3.0, 2.5)
    res = capi.quantized_fc(d, w, b, *ranges, want_int32=False, calib=calib, relu=True)
    torch.cuda.synchronize()
    for rows in (slice(0, 2000), slice((1 << 25) - 2000, M)):
        _, rq, r32, r8 = fc_reference(d, w, b, rows, calib, True)
        np.testing.assert_array_equal(res["out8"][rows].cpu().numpy(), rq)
        assert (res["omin"].item(), res["omax"].item()) == r32
        assert (res["rmin"].item(), res["rmax"].item()) == r8
    step = 1 << 22
    for r0 in range(0, M, step):
        blk = slice(r0, min(r0 + step, M))
        part = capi.quantized_fc(d[blk], w, b, *ranges, want_int32=False, calib=calib, relu=True)
        assert torch.equal(res["out8"][blk], part["out8"]), f"rows from {r0}"


@pytest.mark.parametrize("O,ksize", [(64, 3), (128, 1)])
def test_conv_input_over_2gib(capi, O, ksize):
    """10702 images of 56 x 56 x 64 (2 GiB + 340 KiB) through a 3 x 3 convolution (the
    parked-weights kernel's shape) and a strided 1 x 1."""
    NB, H, W, C = 10702, 56, 56, 64
    stride = 1 if ksize == 3 else 2
    pad = 1 if ksize == 3 else 0
    g = torch.Generator(device="cuda").manual_seed(11 + O)
    d = torch.randint(-127, 128, (NB, H, W, C), dtype=torch.int8, device="cuda", generator=g)
    w = torch.randint(-127, 128, (O, ksize, ksize, C), dtype=torch.int8, device="cuda",
                      generator=g)
    b = torch.randint(-127, 128, (O,), dtype=torch.int8, device="cuda", generator=g)
    one = [f32(-1.0), f32(1.0)]
    calib = (-18.0, 15.0) if ksize == 3 else (-6.0, 5.0)
    kw = dict(stride=(stride, stride), pad=(pad, pad), dilate=(1, 1), calib=calib, relu=True,
              want_int32=False)
    res = capi.quantized_conv_nhwc(d, w, b, *one, *one, *one, **kw)
    torch.cuda.synchronize()
    w_nchw = w.permute(0, 3, 1, 2).contiguous().cpu().numpy()
    for imgs in (slice(0, 2), slice(10698, NB)):
        d_nchw = d[imgs].permute(0, 3, 1, 2).contiguous().cpu().numpy()
        ro, rmn, rmx = oracle.quantized_conv(d_nchw, w_nchw, b.cpu().numpy(), -1.0, 1.0, -1.0,
                                             1.0, -1.0, 1.0, (stride, stride), (pad, pad), (1, 1))
        rq, qmn, qmx = oracle.requantize(ro, rmn, rmx, *calib)
        rq = oracle.relu_i8(rq)
        got = res["out8"][imgs].permute(0, 3, 1, 2).contiguous().cpu().numpy()
        np.testing.assert_array_equal(got, rq)
        assert (res["omin"].item(), res["omax"].item()) == (rmn, rmx)
        assert (res["rmin"].item(), res["rmax"].item()) == (qmn, qmx)
    step = 2048
    for n0 in range(0, NB, step):
        blk = slice(n0, min(n0 + step, NB))
        part = capi.quantized_conv_nhwc(d[blk], w, b, *one, *one, *one, **kw)
        assert torch.equal(res["out8"][blk], part["out8"]), f"images from {n0}"
