"""The benchmark configurations at their full sizes: 2^26-element cast tensors compared with
the oracle element for element; the 8192^3 fully-connected layer and the BERT-base layers
through sampled rows and columns the oracle recomputes, linearity, and the identity
fused-int8 == requantize(int32); every distinct ResNet-50 bottleneck convolution at batch 64
against the oracle on the first and last image of the batch."""
import numpy as np
import pytest
import torch

import oracle

pytestmark = pytest.mark.gpu

N_CAST = 1 << 26


@pytest.fixture(scope="module")
def capi():
    import mxnet_amd
    return mxnet_amd.capi


@pytest.fixture(scope="module")
def contrib():
    import mxnet_amd
    return mxnet_amd.contrib


def f32(v):
    return torch.tensor([v], dtype=torch.float32, device="cuda")


def cast_input(seed):
    """N(0,1) with 0.01 % of the positions at +-50, as the benchmark draws it."""
    g = torch.Generator(device="cuda").manual_seed(seed)
    x = torch.randn(N_CAST, device="cuda", generator=g)
    idx = torch.randint(0, N_CAST, (N_CAST // 10000,), device="cuda", generator=g)
    sign = torch.randint(0, 2, (N_CAST // 10000,), device="cuda", generator=g) * 2 - 1
    x[idx] = 50.0 * sign.to(torch.float32)
    return x


def laplace_input(seed):
    """Laplace(0,1) (by inversion) with 0.01 % of the positions at +-50."""
    g = torch.Generator(device="cuda").manual_seed(seed)
    u = torch.rand(N_CAST, device="cuda", generator=g) - 0.5
    x = -torch.sign(u) * torch.log1p(-2.0 * u.abs())
    del u
    idx = torch.randint(0, N_CAST, (N_CAST // 10000,), device="cuda", generator=g)
    sign = torch.randint(0, 2, (N_CAST // 10000,), device="cuda", generator=g) * 2 - 1
    x[idx] = 50.0 * sign.to(torch.float32)
    return x


@pytest.mark.parametrize("dist", ["normal", "laplace"])
@pytest.mark.parametrize("calib", [None, (-50.0, 50.0), (-4.0, 4.0)])
def test_quantize_v2_64m(capi, calib, dist):
    x = cast_input(1) if dist == "normal" else laplace_input(11)
    kw = {} if calib is None else {"min_calib_range": calib[0], "max_calib_range": calib[1]}
    q, mn, mx = capi.quantize_v2(x, "int8", **kw)
    ref, rmn, rmx = oracle.quantize_v2(x.cpu().numpy(), "int8", *(calib or ()))
    assert (mn.item(), mx.item()) == (rmn, rmx)
    assert np.array_equal(q.cpu().numpy(), ref)


@pytest.mark.parametrize("dist", ["normal", "laplace"])
@pytest.mark.parametrize("calibrated", [True, False])
def test_quantize_v2_uint8_64m(capi, calibrated, dist):
    """fp32 -> uint8 over the data's own range: given as the calibrated range, or found by
    the on-device min/max reduction (uncalibrated)."""
    x = cast_input(2) if dist == "normal" else laplace_input(12)
    xn = x.cpu().numpy()
    if calibrated:
        lo, hi = float(x.min()), float(x.max())
        q, mn, mx = capi.quantize_v2(x, "uint8", min_calib_range=lo, max_calib_range=hi)
        ref, rmn, rmx = oracle.quantize_v2(xn, "uint8", lo, hi)
    else:
        q, mn, mx = capi.quantize_v2(x, "uint8")
        ref, rmn, rmx = oracle.quantize_v2(xn, "uint8")
        assert (rmn, rmx) == (float(xn.min()), float(xn.max()))
    assert (mn.item(), mx.item()) == (rmn, rmx)
    assert np.array_equal(q.cpu().numpy(), ref)


@pytest.mark.parametrize("calibrated", [False, True])
def test_requantize_64m(capi, calibrated):
    g = torch.Generator(device="cuda").manual_seed(3)
    x = torch.randint(-2 ** 28, 2 ** 28, (N_CAST,), device="cuda", generator=g, dtype=torch.int32)
    kw = {"min_calib_range": -0.1, "max_calib_range": 0.1} if calibrated else {}
    q, mn, mx = capi.requantize(x, f32(-1.0), f32(1.0), **kw)
    ref, rmn, rmx = oracle.requantize(x.cpu().numpy(), -1.0, 1.0, *kw.values())
    assert (mn.item(), mx.item()) == (rmn, rmx)
    assert np.array_equal(q.cpu().numpy(), ref)


def test_dequantize_64m(capi):
    g = torch.Generator(device="cuda").manual_seed(4)
    q = torch.randint(-127, 128, (N_CAST,), device="cuda", generator=g, dtype=torch.int8)
    y = capi.dequantize(q, f32(-3.0), f32(3.0))
    ref = oracle.dequantize(q.cpu().numpy(), -3.0, 3.0)
    got = y.cpu().numpy()
    assert np.array_equal(got.view(np.uint32), ref.view(np.uint32))


@pytest.mark.parametrize("dtype", ["int8", "uint8"])
@pytest.mark.parametrize("n", [(1 << 24), (1 << 24) + 1, (1 << 24) + 1023 * 4 + 3,
                               (1 << 25) - 4097, 3 * (1 << 23) + 2048 * 4])
def test_dequantize_chunk_kernel_edges(capi, dtype, n):
    """From 16 M elements on the widening cast runs one chunk of 2048 quads per work-group:
    last chunks that are full, hold one quad, end one quad short, and ragged tails of 1-3
    elements, for both input types."""
    g = torch.Generator(device="cuda").manual_seed(n % 1000)
    if dtype == "int8":
        q = torch.randint(-128, 128, (n,), device="cuda", generator=g, dtype=torch.int8)
        lo, hi = -3.0, 2.5
    else:
        q = torch.randint(0, 256, (n,), device="cuda", generator=g, dtype=torch.uint8)
        lo, hi = -1.0, 7.0
    guard = torch.full((n + 64,), 7.5, dtype=torch.float32, device="cuda")
    y = guard[:n]
    from mxnet_amd._lib import check, lib
    import ctypes
    code = 5 if dtype == "int8" else 3
    rlo, rhi = f32(lo), f32(hi)   # kept alive across the call
    check(lib.mxq_dequantize(ctypes.c_void_p(torch.cuda.current_stream().cuda_stream),
                             ctypes.c_void_p(q.data_ptr()), code,
                             ctypes.c_void_p(rlo.data_ptr()), ctypes.c_void_p(rhi.data_ptr()),
                             ctypes.c_void_p(y.data_ptr()), n))
    torch.cuda.synchronize()
    ref = oracle.dequantize(q.cpu().numpy(), lo, hi)
    assert np.array_equal(y.cpu().numpy().view(np.uint32), ref.view(np.uint32))
    assert bool((guard[n:] == 7.5).all()), "wrote past the end"


@pytest.mark.parametrize("lu,ru", [(False, False), (True, False), (False, True), (True, True)])
@pytest.mark.parametrize("n", [(1 << 24), (1 << 24) + 3, (1 << 24) + 1023 * 4 + 1,
                               (1 << 25) - 4097])
def test_elemwise_add_int32_chunk_kernel_edges(contrib, lu, ru, n):
    """From 16 M elements on the int32 sum runs one chunk of 2048 quads per work-group: full
    and partial last chunks, ragged tails, every operand type pair."""
    g = torch.Generator(device="cuda").manual_seed(n % 997 + 2 * lu + ru)
    def operand(unsigned):
        if unsigned:
            return torch.randint(0, 256, (n,), device="cuda", generator=g, dtype=torch.uint8)
        return torch.randint(-128, 128, (n,), device="cuda", generator=g, dtype=torch.int8)
    a, b = operand(lu), operand(ru)
    rng = (-1.5, 2.0, -0.75, 0.5)
    out, mn, mx = contrib.quantized_elemwise_add(a, b, *[f32(v) for v in rng])
    ref, rmn, rmx = oracle.quantized_elemwise_add(a.cpu().numpy(), b.cpu().numpy(), *rng)
    assert out.dtype == torch.int32
    assert (mn.item(), mx.item()) == (rmn, rmx)
    assert np.array_equal(out.cpu().numpy(), ref)


@pytest.mark.parametrize("n", [(1 << 26), (1 << 26) + 5, (1 << 26) + 2047 * 16 + 15,
                               (1 << 26) + 2048 * 16 + 1])
def test_quantized_act_chunk_kernel_edges(contrib, n):
    """From 64 M elements on the relu runs one chunk of 2048 16-byte pieces per work-group:
    full and partial last chunks, ragged tails."""
    g = torch.Generator(device="cuda").manual_seed(n % 991)
    guard = torch.randint(-128, 128, (n + 64,), device="cuda", generator=g, dtype=torch.int8)
    x = guard[:n]
    out_buf = torch.full((n + 64,), 77, dtype=torch.int8, device="cuda")
    import ctypes
    from mxnet_amd._lib import check, lib
    lo, hi, omn, omx = f32(-2.0), f32(3.0), f32(0.0), f32(0.0)
    P = lambda t: ctypes.c_void_p(t.data_ptr())
    check(lib.mxq_quantized_relu(ctypes.c_void_p(torch.cuda.current_stream().cuda_stream), P(x),
                                 P(lo), P(hi), P(out_buf), P(omn), P(omx), n))
    torch.cuda.synchronize()
    assert torch.equal(out_buf[:n], torch.clamp(x, min=0))
    assert bool((out_buf[n:] == 77).all()), "wrote past the end"
    assert (omn.item(), omx.item()) == (-2.0, 3.0)
    ref = oracle.relu_i8(x[:1 << 20].cpu().numpy())
    assert np.array_equal(out_buf[:1 << 20].cpu().numpy(), ref)


CONCAT_EDGE_CASES = [
    # (shapes, axis, dtype, (min, max) per input)
    ([((1 << 25) + 16,), ((1 << 25) + 4096 * 16 - 16,)], 0, np.int8, [(-1.0, 1.0), (-2.0, 2.0)]),
    ([(8, 3, 1 << 20), (8, 0, 1 << 20), (8, 5, (1 << 20))], 1, np.int8,
     [(-1.0, 0.5), (-1.0, 1.0), (-3.0, 4.0)]),
    ([(4, (1 << 23) + 48), (4, (1 << 23) + 16 * 1023)], 1, np.uint8, [(0.0, 1.0), (0.0, 2.5)]),
    ([(2, 1 << 24, 2), (2, (1 << 24) + 8, 2)], 1, np.int8, [(-2.0, 2.0), (-2.0, 2.0)]),
]


@pytest.mark.parametrize("case", range(len(CONCAT_EDGE_CASES)))
def test_concat_chunk_kernel_edges(contrib, case):
    """From 16 MiB per launch, with every input 16-byte aligned, concat runs one chunk of 1024
    16-byte pieces per work-group: partial last chunks, several rows with a pitch, an empty
    input between two others, uint8, and equal ranges (the byte copy)."""
    shapes, axis, dtype, ranges = CONCAT_EDGE_CASES[case]
    rng = np.random.default_rng(100 + case)
    lo, hi = (0, 256) if dtype == np.uint8 else (-128, 128)
    xs = [rng.integers(lo, hi, size=s, dtype=np.int64).astype(dtype) for s in shapes]
    args = [torch.from_numpy(x).cuda() for x in xs]
    for mn, mx in ranges:
        args += [f32(mn), f32(mx)]
    out, omn, omx = contrib.quantized_concat(*args, num_args=len(xs), dim=axis)
    ref, rmn, rmx = oracle.quantized_concat(xs, [r[0] for r in ranges], [r[1] for r in ranges],
                                            dim=axis)
    assert tuple(out.shape) == ref.shape
    assert (omn.item(), omx.item()) == (rmn, rmx)
    assert np.array_equal(out.cpu().numpy(), ref)


@pytest.mark.parametrize("dtype,relu", [(np.int8, True), (np.uint8, False)])
def test_batch_norm_64m_one_launch(contrib, dtype, relu):
    """With rows of 2 KiB and more the batch norm is one launch whose waves fold their channel's
    parameters themselves, from 64 M elements on a grid of one piece per wave: the oracle on
    the first and last image, and every block of 16 images against a call of its own (the
    capped grid whose waves stride over the pieces)."""
    N, C, H, W = 64, 256, 64, 64
    g = torch.Generator(device="cuda").manual_seed(31)
    lo, hi = (0, 256) if dtype == np.uint8 else (-128, 128)
    x = torch.randint(lo, hi, (N, C, H, W), device="cuda", generator=g,
                      dtype=torch.uint8 if dtype == np.uint8 else torch.int8)
    rng = np.random.default_rng(32)
    gamma = rng.uniform(0.5, 2.0, C).astype(np.float32)
    beta = rng.normal(0, 0.5, C).astype(np.float32)
    mean = rng.normal(0, 0.3, C).astype(np.float32)
    var = rng.uniform(0.3, 2.0, C).astype(np.float32)
    rd = (0.0, 3.1) if dtype == np.uint8 else (-2.7, 3.1)
    par = [torch.from_numpy(v).cuda() for v in (gamma, beta, mean, var)]
    kw = dict(eps=2e-5, axis=1, min_calib_range=-6.5, max_calib_range=7.25, relu=relu)
    out, mn, mx = contrib.quantized_batch_norm(x, *par, f32(rd[0]), f32(rd[1]), **kw)
    for n in (0, N - 1):
        ref, rmn, rmx = oracle.quantized_batch_norm(x[n:n + 1].cpu().numpy(), gamma, beta, mean,
                                                    var, rd[0], rd[1], -6.5, 7.25, eps=2e-5,
                                                    axis=1, relu=relu)
        assert np.array_equal(out[n:n + 1].cpu().numpy(), ref), f"image {n}"
        assert (mn.item(), mx.item()) == (rmn, rmx)
    for n0 in range(0, N, 16):
        part, _, _ = contrib.quantized_batch_norm(x[n0:n0 + 16], *par, f32(rd[0]), f32(rd[1]), **kw)
        assert torch.equal(out[n0:n0 + 16], part), f"images from {n0}"


def test_elemwise_add_64m(contrib):
    g = torch.Generator(device="cuda").manual_seed(5)
    a = torch.randint(-127, 128, (N_CAST,), device="cuda", generator=g, dtype=torch.int8)
    b = torch.randint(-127, 128, (N_CAST,), device="cuda", generator=g, dtype=torch.int8)
    for kw in ({}, {"min_calib_range": -5.0, "max_calib_range": 5.0}):
        out, mn, mx = contrib.quantized_elemwise_add(a, b, f32(-3.0), f32(3.0), f32(-3.0),
                                                     f32(3.0), **kw)
        ref, rmn, rmx = oracle.quantized_elemwise_add(a.cpu().numpy(), b.cpu().numpy(), -3.0, 3.0,
                                                      -3.0, 3.0, **kw)
        assert (mn.item(), mx.item()) == (rmn, rmx)
        assert np.array_equal(out.cpu().numpy(), ref)


def check_fc(capi, M, K, N, seed):
    g = torch.Generator(device="cuda").manual_seed(seed)
    d1 = torch.randint(-60, 61, (M, K), device="cuda", generator=g, dtype=torch.int8)
    d2 = torch.randint(-60, 61, (M, K), device="cuda", generator=g, dtype=torch.int8)
    w = torch.randint(-127, 128, (N, K), device="cuda", generator=g, dtype=torch.int8)
    b = torch.randint(-127, 128, (N,), device="cuda", generator=g, dtype=torch.int8)
    one = f32(1.0)
    args = (-one, one, -one, one)
    r1 = capi.quantized_fc(d1, w, None, *args)["out32"]
    r2 = capi.quantized_fc(d2, w, None, *args)["out32"]
    r12 = capi.quantized_fc(d1 + d2, w, None, *args)["out32"]
    assert torch.equal(r1 + r2, r12)                      # linear in the data operand
    rows = sorted({0, 1, 255, 256, M // 2 - 1, M // 2, M - 257, M - 1})
    want = oracle.fc_int32(d1[rows].cpu().numpy(), w.cpu().numpy())
    assert np.array_equal(r1[rows].cpu().numpy(), want)
    cols = sorted({0, 31, 32, 255, 256, N // 2, N - 1})
    want_c = oracle.fc_int32(d1.cpu().numpy(), w[cols].cpu().numpy())
    assert np.array_equal(r1[:, cols].cpu().numpy(), want_c)
    del r2, r12
    # the fused epilogue (bias + relu + requantize) is the int32 result requantized
    # calibrated to two standard deviations of the accumulator (in its float units)
    c = 2.0 * 35.0 * 73.0 * K ** 0.5 / 127.0 ** 2
    res = capi.quantized_fc(d1, w, b, *args, -one, one, calib=(-c, c), relu=True)
    q, mn, mx = capi.requantize(res["out32"], res["omin"], res["omax"], min_calib_range=-c,
                                max_calib_range=c)
    assert torch.equal(res["out8"], torch.clamp(q, min=0))
    assert (res["rmin"].item(), res["rmax"].item()) == (mn.item(), mx.item())
    assert int(res["out8"].max()) == 127 and 0.2 < float((res["out8"] > 0).float().mean()) < 0.8
    # ... and the oracle's own chain on the sampled rows: int8 bias rescaled to int32,
    # exact accumulation, requantize, relu
    acc_o, omin_o, omax_o = oracle.quantized_fully_connected(
        d1[rows].cpu().numpy(), w.cpu().numpy(), b.cpu().numpy(), -1.0, 1.0, -1.0, 1.0, -1.0, 1.0)
    assert np.array_equal(res["out32"][rows].cpu().numpy(), acc_o)
    assert (res["omin"].item(), res["omax"].item()) == (omin_o, omax_o)
    q_o, qmn_o, qmx_o = oracle.requantize(acc_o, omin_o, omax_o, -c, c)
    assert np.array_equal(res["out8"][rows].cpu().numpy(), oracle.relu_i8(q_o))
    assert (res["rmin"].item(), res["rmax"].item()) == (qmn_o, qmx_o)
    # the form the benchmark times: int8 output only (no int32 store)
    fused = capi.quantized_fc(d1, w, b, *args, -one, one, calib=(-c, c), relu=True,
                              want_int32=False)
    assert torch.equal(fused["out8"], res["out8"])
    assert (fused["omin"].item(), fused["omax"].item()) == (omin_o, omax_o)


def test_fc_4096(capi):
    check_fc(capi, 4096, 4096, 4096, seed=4)


def test_fc_8192(capi):
    check_fc(capi, 8192, 8192, 8192, seed=8)


@pytest.mark.parametrize("K,N", [(768, 2304), (768, 768), (768, 3072), (3072, 768)])
def test_fc_bert_base_layers(capi, K, N):
    check_fc(capi, 4096, K, N, seed=K + N)


RESNET50_CONVS = [(56, 64, 64, 1, 1), (56, 64, 64, 3, 1), (56, 64, 256, 1, 1), (56, 256, 64, 1, 1),
                  (56, 256, 128, 1, 2), (28, 128, 128, 3, 1), (28, 128, 512, 1, 1),
                  (28, 512, 128, 1, 1), (56, 256, 512, 1, 2), (28, 512, 256, 1, 2),
                  (14, 256, 256, 3, 1), (14, 256, 1024, 1, 1), (14, 1024, 256, 1, 1),
                  (28, 512, 1024, 1, 2), (14, 1024, 512, 1, 2), (7, 512, 512, 3, 1),
                  (7, 512, 2048, 1, 1), (7, 2048, 512, 1, 1), (14, 1024, 2048, 1, 2)]


@pytest.mark.parametrize("H,C,O,k,s", RESNET50_CONVS)
def test_resnet50_conv_batch64(capi, H, C, O, k, s):
    batch, pad = 64, (1 if k == 3 else 0)
    g = torch.Generator(device="cuda").manual_seed(H + C + O + k)
    d = torch.randint(-127, 128, (batch, H, H, C), device="cuda", generator=g, dtype=torch.int8)
    w = torch.randint(-127, 128, (O, k, k, C), device="cuda", generator=g, dtype=torch.int8)
    b = torch.randint(-127, 128, (O,), device="cuda", generator=g, dtype=torch.int8)
    one = f32(1.0)
    r = 2.0 * 73.0 * 73.0 * (k * k * C) ** 0.5 / 127.0 ** 2   # two standard deviations
    res = capi.quantized_conv_nhwc(d, w, b, -one, one, -one, one, -one, one, stride=(s, s),
                                   pad=(pad, pad), calib=(-r, r), relu=True)
    images = [0, batch - 1]
    dn = d[images].permute(0, 3, 1, 2).contiguous().cpu().numpy()
    wn = w.permute(0, 3, 1, 2).contiguous().cpu().numpy()
    acc, omin, omax = oracle.quantized_conv(dn, wn, b.cpu().numpy(), -1.0, 1.0, -1.0, 1.0, -1.0,
                                            1.0, stride=(s, s), pad=(pad, pad))
    got32 = res["out32"][images].permute(0, 3, 1, 2).contiguous().cpu().numpy()
    assert np.array_equal(got32, acc)
    assert (res["omin"].item(), res["omax"].item()) == (omin, omax)
    q, rmin, rmax = oracle.requantize(acc, omin, omax, -r, r)
    got8 = res["out8"][images].permute(0, 3, 1, 2).contiguous().cpu().numpy()
    assert np.array_equal(got8, np.maximum(q, 0))
    # the images between them through the identity fused == requantize(int32)
    q_all, _, _ = capi.requantize(res["out32"], res["omin"], res["omax"], min_calib_range=-r,
                                  max_calib_range=r)
    assert torch.equal(res["out8"], torch.clamp(q_all, min=0))
    frac = float((res["out8"] > 0).float().mean())
    assert 0.2 < frac < 0.8 and int(res["out8"].max()) == 127


@pytest.mark.parametrize("H,C,O,k,s", RESNET50_CONVS)
def test_resnet50_conv_batch64_through_the_operator(capi, contrib, H, C, O, k, s):
    """The same 19 layers at batch 64 through the registered _contrib_quantized_conv: NCHW int8
    data and OIHW int8 weights in, int32 NCHW out, temp space sized by the operator host.  The
    first and last image against the oracle, every image against the NHWC entry point's
    result brought to NCHW by torch (another kernel, another layout, another epilogue)."""
    batch, pad = 64, (1 if k == 3 else 0)
    g = torch.Generator(device="cuda").manual_seed(3 * H + C + O + k)
    d = torch.randint(-127, 128, (batch, C, H, H), device="cuda", generator=g, dtype=torch.int8)
    w = torch.randint(-127, 128, (O, C, k, k), device="cuda", generator=g, dtype=torch.int8)
    b = torch.randint(-127, 128, (O,), device="cuda", generator=g, dtype=torch.int8)
    one = f32(1.0)
    out, mn, mx = contrib.quantized_conv(d, w, b, -one, one, -one, one, -one, one,
                                         kernel=(k, k), stride=(s, s), dilate=(1, 1),
                                         pad=(pad, pad), num_filter=O, no_bias=False,
                                         layout="NCHW")
    OH = (H + 2 * pad - k) // s + 1
    assert out.dtype == torch.int32 and tuple(out.shape) == (batch, O, OH, OH)
    images = [0, batch - 1]
    acc, omin, omax = oracle.quantized_conv(d[images].cpu().numpy(), w.cpu().numpy(),
                                            b.cpu().numpy(), -1.0, 1.0, -1.0, 1.0, -1.0, 1.0,
                                            stride=(s, s), pad=(pad, pad))
    assert np.array_equal(out[images].cpu().numpy(), acc)
    assert (mn.item(), mx.item()) == (omin, omax)
    ref = capi.quantized_conv_nhwc(d.permute(0, 2, 3, 1).contiguous(),
                                   w.permute(0, 2, 3, 1).contiguous(), b, -one, one, -one, one,
                                   -one, one, stride=(s, s), pad=(pad, pad))
    assert torch.equal(out, ref["out32"].permute(0, 3, 1, 2))
