"""Parity of the HIP quantized fully-connected kernel with the CPU oracle through the
C ABI: int32 accumulators and fused int8 outputs bit-exact."""
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


def run_fc(capi, d, w, b, rd, rw, rb, calib=None, relu=False, want_int32=True, force=None):
    """force = (cfg, splits, stream_groups) pins the kernel variant through the test-only
    entry point; None is the operator's own entry point."""
    return capi.quantized_fc(dev(d), dev(w), None if b is None else dev(b), f32(-rd), f32(rd),
                             f32(-rw), f32(rw), None if b is None else f32(-rb),
                             None if b is None else f32(rb), want_int32=want_int32, calib=calib,
                             relu=relu, force=force)


def oracle_fc(d, w, b, rd, rw, rb):
    return oracle.quantized_fully_connected(d, w, b, -rd, rd, -rw, rw,
                                            None if b is None else -rb,
                                            None if b is None else rb)


# (M, K, N): tile-aligned, ragged in each dimension, K not a multiple of 16 (scalar
# loader), the reference's own test shapes (test_quantization.py:795-808)
SHAPES = [(128, 1024, 1024), (256, 256, 256), (1, 16, 1), (33, 80, 100), (257, 144, 259),
          (32, 2048, 100), (32, 444, 100), (256, 8192, 800), (256, 444, 800), (64, 64, 4096),
          (300, 1000, 37), (512, 768, 768)]


@pytest.mark.parametrize("M,K,N", SHAPES)
@pytest.mark.parametrize("use_bias", [False, True])
def test_fc_int32(capi, M, K, N, use_bias):
    d = int8_uniform((M, K), seed=M + K)
    w = int8_uniform((N, K), seed=N + K + 1)
    b = int8_uniform((N,), seed=N) if use_bias else None
    rd, rw, rb = 1.0, 0.08, 0.5
    res = run_fc(capi, d, w, b, rd, rw, rb)
    ro, rmn, rmx = oracle_fc(d, w, b, rd, rw, rb)
    np.testing.assert_array_equal(res["out32"].cpu().numpy(), ro)
    assert (res["omin"].item(), res["omax"].item()) == (rmn, rmx)


@pytest.mark.parametrize("cfg", [1, 2, 3, 4, 11, 12, 14, 16, 21, 22, 23, 24, 31, 32, 41, 42, 43, 44,
                                 51, 52, 53, 54, 55, 56, 57, 58, 59, 60])
@pytest.mark.parametrize("M,K,N", [(512, 512, 512), (300, 208, 270), (70, 444, 33),
                                   (300, 192, 270), (1, 64, 1), (1024, 1024, 520),
                                   (130, 16, 70), (257, 80, 64)])
def test_fc_every_tile_config(capi, cfg, M, K, N):
    if 10 < cfg < 20 and K % 64 != 0:
        pytest.skip("the global-load direct-to-LDS kernels need K % 64 == 0")
    if cfg > 20 and K % 16 != 0:
        pytest.skip("the buffer-load direct-to-LDS kernels need K % 16 == 0")
    d = int8_uniform((M, K), seed=cfg + M)
    w = int8_uniform((N, K), seed=cfg + N + 7)
    b = int8_uniform((N,), seed=cfg)
    res = run_fc(capi, d, w, b, 2.0, 0.1, 1.0, calib=(-30.0, 28.0), force=(cfg, 1, 0))
    ro, rmn, rmx = oracle_fc(d, w, b, 2.0, 0.1, 1.0)
    np.testing.assert_array_equal(res["out32"].cpu().numpy(), ro)
    rq, qmn, qmx = oracle.requantize(ro, rmn, rmx, -30.0, 28.0)
    np.testing.assert_array_equal(res["out8"].cpu().numpy(), rq)


@pytest.mark.parametrize("M,K,N", [(128, 1024, 1024), (257, 144, 259), (32, 444, 100)])
@pytest.mark.parametrize("relu", [False, True])
def test_fc_fused_requantize_equals_unfused(capi, M, K, N, relu):
    d = int8_uniform((M, K), seed=1)
    w = int8_uniform((N, K), seed=2, lo=-20, hi=20)
    b = int8_uniform((N,), seed=3)
    rd, rw, rb = 1.0, 0.08, 0.5
    ro, rmn, rmx = oracle_fc(d, w, b, rd, rw, rb)
    # calibration range that clips part of the distribution
    fl = ro.astype(np.float64) * (float(rmx) / 2147483648.0)
    R = float(np.percentile(np.abs(fl), 99.0))
    res = run_fc(capi, d, w, b, rd, rw, rb, calib=(-R, 0.9 * R), relu=relu, want_int32=False)
    rq, qmn, qmx = oracle.requantize(ro, rmn, rmx, -R, 0.9 * R)
    if relu:
        rq = oracle.relu_i8(rq)
    np.testing.assert_array_equal(res["out8"].cpu().numpy(), rq)
    assert (res["rmin"].item(), res["rmax"].item()) == (qmn, qmx)
    # and the stand-alone requantize kernel on the int32 output agrees too
    res2 = run_fc(capi, d, w, b, rd, rw, rb)
    q2, mn2, mx2 = capi.requantize(res2["out32"], res2["omin"], res2["omax"],
                                   min_calib_range=-R, max_calib_range=0.9 * R)
    if relu:
        q2 = torch.clamp(q2, min=0)
    assert torch.equal(q2, res["out8"])


def test_fc_reference_test_construction(capi):
    """The reference's own check (test_quantization.py:661-793): integer-valued data in
    [-63,63], ranges = observed maxabs, no bias -> the int32 output equals the fp32
    Dense output exactly."""
    rng = np.random.default_rng(0)
    for shape, nh in [((32, 512, 2, 2), 100), ((32, 111, 2, 2), 100), ((256, 111, 2, 2), 800)]:
        data = rng.uniform(-63.0, 63.0, size=shape).astype(np.int32).astype(np.float32)
        K = int(np.prod(shape[1:]))
        weight = rng.uniform(-63.0, 63.0, size=(nh, K)).astype(np.int32).astype(np.float32)
        want = data.reshape(shape[0], -1).astype(np.float64) @ weight.astype(np.float64).T
        dr, wr = float(np.abs(data).max()), float(np.abs(weight).max())
        res = run_fc(capi, data.reshape(shape[0], -1).astype(np.int8), weight.astype(np.int8),
                     None, dr, wr, 0.0)
        np.testing.assert_array_equal(res["out32"].cpu().numpy().astype(np.float64), want)


def test_fc_large_linearity(capi):
    """At the benchmark size (4096^3) check properties that need no CPU GEMM:
    (a) rows of the output that the oracle recomputes (sampled), (b) linearity in the
    data operand: fc(d1) + fc(d2) == fc(d1 + d2) for small-valued operands."""
    M = K = N = 4096
    g = torch.Generator(device="cuda").manual_seed(0)
    d1 = torch.randint(-60, 61, (M, K), device="cuda", generator=g, dtype=torch.int8)
    d2 = torch.randint(-60, 61, (M, K), device="cuda", generator=g, dtype=torch.int8)
    w = torch.randint(-127, 128, (N, K), device="cuda", generator=g, dtype=torch.int8)
    one = torch.ones(1, device="cuda")
    r1 = capi.quantized_fc(d1, w, None, -one, one, -one, one)["out32"]
    r2 = capi.quantized_fc(d2, w, None, -one, one, -one, one)["out32"]
    r12 = capi.quantized_fc(d1 + d2, w, None, -one, one, -one, one)["out32"]
    assert torch.equal(r1 + r2, r12)
    rows = [0, 1, 255, 256, 1023, 2048, 4095]
    want = oracle.fc_int32(d1[rows].cpu().numpy(), w.cpu().numpy())
    np.testing.assert_array_equal(r1[rows].cpu().numpy(), want)
    cols = [0, 31, 32, 255, 256, 4095]
    want_c = oracle.fc_int32(d1.cpu().numpy(), w[cols].cpu().numpy())
    np.testing.assert_array_equal(r1[:, cols].cpu().numpy(), want_c)


def test_fc_errors(capi):
    import mxnet_amd
    d = torch.zeros((4, 16), dtype=torch.int8, device="cuda")
    one = torch.ones(1, device="cuda")
    with pytest.raises(mxnet_amd._lib.MXQError, match="no output buffer"):
        capi.quantized_fc(d, d, None, -one, one, -one, one, want_int32=False)
    b = torch.zeros(4, dtype=torch.int8, device="cuda")
    with pytest.raises(mxnet_amd._lib.MXQError, match="bias given without its range"):
        capi.quantized_fc(d, d, b, -one, one, -one, one)


@pytest.mark.parametrize("cfg", [61, 62])
@pytest.mark.parametrize("M,K,N", [(32, 64, 64), (1, 32, 128), (33, 64, 256), (1000, 128, 128),
                                   (4099, 64, 512), (257, 128, 768), (70, 32, 1024),
                                   (6272, 64, 256), (300, 256, 64), (1111, 256, 384)])
@pytest.mark.parametrize("relu,use_bias", [(False, True), (True, True), (True, False)])
def test_fc_short_k_streaming_kernel(capi, cfg, M, K, N, relu, use_bias):
    """The short-K kernel (weights parked in LDS, data streamed by independent waves): fused
    int8 output against requantize(oracle int32), ragged M, one to several column groups."""
    if cfg == 62 and N % 128 != 0:
        pytest.skip("128-column strips need N % 128 == 0")
    d = int8_uniform((M, K), seed=cfg + M)
    w = int8_uniform((N, K), seed=K + N, lo=-40, hi=40)
    b = int8_uniform((N,), seed=N) if use_bias else None
    rd, rw, rb = 1.0, 0.08, 0.5
    ro, rmn, rmx = oracle_fc(d, w, b, rd, rw, rb)
    fl = ro.astype(np.float64) * (float(rmx) / 2147483648.0)
    R = float(np.percentile(np.abs(fl), 98.0))
    res = run_fc(capi, d, w, b, rd, rw, rb, calib=(-R, 0.9 * R), relu=relu, want_int32=False,
                 force=(cfg, 1, 2))
    rq, qmn, qmx = oracle.requantize(ro, rmn, rmx, -R, 0.9 * R)
    if relu:
        rq = oracle.relu_i8(rq)
    np.testing.assert_array_equal(res["out8"].cpu().numpy(), rq)
    assert (res["omin"].item(), res["omax"].item()) == (rmn, rmx)
    assert (res["rmin"].item(), res["rmax"].item()) == (qmn, qmx)


def test_fc_short_k_streaming_kernel_refuses_other_shapes(capi):
    import mxnet_amd
    d, w = int8_uniform((64, 96), seed=1), int8_uniform((64, 96), seed=2)
    with pytest.raises(mxnet_amd._lib.MXQError, match="short-K"):
        run_fc(capi, d, w, None, 1.0, 1.0, 1.0, calib=(-1.0, 1.0), want_int32=False,
               force=(61, 1, 2))
    with pytest.raises(mxnet_amd._lib.MXQError, match="short-K"):   # int32 output wanted
        run_fc(capi, d[:, :64].copy(), w[:, :64].copy(), None, 1.0, 1.0, 1.0, force=(61, 1, 2))


# every direct-to-LDS configuration, split along K over 2 .. 5 work-groups per tile: the
# int32 sum and the fused int8 output must not depend on the split (integer addition is
# associative).  Shapes: tile-aligned, ragged M / N, K not a multiple of the stage depth,
# more splits than K stages (clamped), one stage per split.
@pytest.mark.parametrize("cfg", [11, 12, 14, 16, 21, 22, 23, 24, 31, 32, 41, 42, 43, 44, 51, 52, 53,
                                 54, 55, 56, 57, 58, 59, 60])
@pytest.mark.parametrize("M,K,N,splits", [(512, 1024, 512, 2), (300, 2064, 270, 3),
                                          (70, 4096, 33, 5), (257, 208, 64, 4),
                                          (1024, 1536, 520, 4), (64, 128, 64, 2)])
def test_fc_split_k(capi, cfg, M, K, N, splits):
    if 10 < cfg < 20 and K % 64 != 0:
        pytest.skip("the global-load direct-to-LDS kernels need K % 64 == 0")
    d = int8_uniform((M, K), seed=cfg + M + 1)
    w = int8_uniform((N, K), seed=cfg + N + 3)
    b = int8_uniform((N,), seed=cfg + 5)
    res = run_fc(capi, d, w, b, 2.0, 0.1, 1.0, calib=(-30.0, 28.0), force=(cfg, splits, 0))
    ro, rmn, rmx = oracle_fc(d, w, b, 2.0, 0.1, 1.0)
    np.testing.assert_array_equal(res["out32"].cpu().numpy(), ro)
    rq, qmn, qmx = oracle.requantize(ro, rmn, rmx, -30.0, 28.0)
    np.testing.assert_array_equal(res["out8"].cpu().numpy(), rq)
    assert (res["omin"].item(), res["omax"].item()) == (rmn, rmx)


def test_fc_split_k_workspace_reuse(capi):
    """The same workspace handed to split launches of different data back to back: every
    launch must read the partial sums of its own work-groups, not an earlier launch's
    (stale lines in another XCD's L2), and clear its own counters."""
    import ctypes
    from mxnet_amd._lib import lib, check
    M, K, N = 640, 3072, 384
    ws = torch.empty(64 << 20, dtype=torch.uint8, device="cuda")
    one = [f32(v) for v in (-1.0, 1.0, -0.1, 0.1)]
    out = torch.empty((M, N), dtype=torch.int32, device="cuda")
    om = [torch.empty(1, device="cuda") for _ in range(2)]
    P = lambda t: ctypes.c_void_p(t.data_ptr())
    st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    for it in range(12):
        d = int8_uniform((M, K), seed=100 + it)
        w = int8_uniform((N, K), seed=200 + it)
        cfg, splits = [(53, 4), (43, 6), (12, 3), (58, 8)][it % 4]
        dd, wd = dev(d), dev(w)   # kept alive until the result has been read back
        check(lib.mxq_test_quantized_fc(st, P(dd), P(wd), None, M, N, K, P(one[0]),
                                        P(one[1]), P(one[2]), P(one[3]), None, None, P(out),
                                        P(om[0]), P(om[1]), None, None, None, 0, 0.0, 0.0,
                                        P(ws), ws.numel(), cfg, splits, 0))
        ro, _, _ = oracle_fc(d, w, None, 1.0, 0.1, 1.0)
        np.testing.assert_array_equal(out.cpu().numpy(), ro)


def test_fc_split_is_chosen_for_few_tiles_and_long_k(capi):
    """The launcher's own choice: the reference's small-batch test shape (256 x 8192 -> 800)
    asks for a split-K workspace and gives the oracle's result with it and without it; the
    square and BERT shapes ask for none."""
    from mxnet_amd._lib import lib
    assert lib.mxq_quantized_fc_workspace(256, 800, 8192, 0) > 0
    assert lib.mxq_quantized_fc_workspace(4096, 4096, 4096, 1) == 0
    assert lib.mxq_quantized_fc_workspace(4096, 2304, 768, 1) == 0
    d = int8_uniform((256, 8192), seed=5)
    w = int8_uniform((800, 8192), seed=6)
    b = int8_uniform((800,), seed=7)
    ro, rmn, rmx = oracle_fc(d, w, b, 1.0, 0.08, 0.5)
    res = run_fc(capi, d, w, b, 1.0, 0.08, 0.5)                 # with the workspace
    np.testing.assert_array_equal(res["out32"].cpu().numpy(), ro)
    res = run_fc(capi, d, w, b, 1.0, 0.08, 0.5, force=(0, 0, 0))  # chooser, no workspace
    np.testing.assert_array_equal(res["out32"].cpu().numpy(), ro)


def test_fc_split_k_needs_workspace(capi):
    import mxnet_amd
    d, w = int8_uniform((256, 1024), seed=1), int8_uniform((256, 1024), seed=2)
    args = [dev(d), dev(w), None, f32(-1.0), f32(1.0), f32(-1.0), f32(1.0)]
    import ctypes
    from mxnet_amd._lib import lib
    out = torch.empty((256, 256), dtype=torch.int32, device="cuda")
    om = [torch.empty(1, device="cuda") for _ in range(2)]
    P = lambda t: ctypes.c_void_p(t.data_ptr())
    rc = lib.mxq_test_quantized_fc(None, P(args[0]), P(args[1]), None, 256, 256, 1024, P(args[3]),
                                   P(args[4]), P(args[5]), P(args[6]), None, None, P(out),
                                   P(om[0]), P(om[1]), None, None, None, 0, 0.0, 0.0, None, 0,
                                   53, 4, 0)
    assert rc != 0 and "workspace" in mxnet_amd._lib.last_error()


def test_fc_degenerate_extents(capi):
    """No rows: nothing to compute, but the output range is still written.  K = 0: the
    output is the rescaled bias alone."""
    w = int8_uniform((24, 48), seed=1)
    b = int8_uniform((24,), seed=2)
    res = run_fc(capi, np.zeros((0, 48), np.int8), w, b, 1.0, 0.08, 0.5)
    ro, rmn, rmx = oracle_fc(np.zeros((0, 48), np.int8), w, b, 1.0, 0.08, 0.5)
    assert tuple(res["out32"].shape) == (0, 24)
    assert (res["omin"].item(), res["omax"].item()) == (rmn, rmx)
    d0, w0 = np.zeros((5, 0), np.int8), np.zeros((24, 0), np.int8)
    res = run_fc(capi, d0, w0, b, 1.0, 0.08, 0.5)
    ro, rmn, rmx = oracle_fc(d0, w0, b, 1.0, 0.08, 0.5)
    np.testing.assert_array_equal(res["out32"].cpu().numpy(), ro)
    assert (res["omin"].item(), res["omax"].item()) == (rmn, rmx)


# ---- quantized_fc -> requantize -> dequantize in one launch ---------------------------------
def oracle_fc_f32(d, w, b, rd, rw, rb, calib, relu):
    """The three reference operators one after the other."""
    ro, rmn, rmx = oracle_fc(d, w, b, rd, rw, rb)
    rq, qmn, qmx = oracle.requantize(ro, rmn, rmx, *calib)
    if relu:
        rq = oracle.relu_i8(rq)
    return oracle.dequantize(rq, qmn, qmx), (rmn, rmx), (qmn, qmx)


def check_fc_f32(capi, d, w, b, calib, relu, force=None):
    rd, rw, rb = 2.0, 0.1, 1.0
    res = capi.quantized_fc_f32(dev(d), dev(w), None if b is None else dev(b), f32(-rd), f32(rd),
                                f32(-rw), f32(rw), None if b is None else f32(-rb),
                                None if b is None else f32(rb), calib=calib, relu=relu,
                                force=force)
    ref, r32, r8 = oracle_fc_f32(d, w, b, rd, rw, rb, calib, relu)
    got = res["outf"].cpu().numpy()
    # bit for bit, the sign of a zero included
    np.testing.assert_array_equal(got.view(np.uint32), ref.view(np.uint32))
    assert (res["omin"].item(), res["omax"].item()) == r32
    assert (res["rmin"].item(), res["rmax"].item()) == r8


@pytest.mark.parametrize("M,K,N", SHAPES + [(4096, 768, 768), (512, 3072, 772), (100, 64, 6)])
@pytest.mark.parametrize("relu", [False, True])
def test_fc_dequantized_output(capi, M, K, N, relu):
    d = int8_uniform((M, K), seed=M + K + 2)
    w = int8_uniform((N, K), seed=N + K + 3)
    b = int8_uniform((N,), seed=N + 4) if (M + N) % 2 else None
    ro, rmn, rmx = oracle_fc(d, w, b, 2.0, 0.1, 1.0)
    fl = ro.astype(np.float64) * (float(rmx) / 2147483648.0)
    R = float(np.percentile(np.abs(fl), 98.0)) or 1.0
    check_fc_f32(capi, d, w, b, (-R, 0.85 * R), relu)


@pytest.mark.parametrize("cfg", [1, 2, 3, 4, 11, 12, 14, 16, 21, 22, 23, 24, 31, 32, 41, 42, 43, 44,
                                 51, 52, 53, 54, 55, 56, 57, 58, 59, 60])
@pytest.mark.parametrize("M,K,N,splits", [(512, 512, 512, 1), (300, 192, 270, 1), (70, 448, 36, 1),
                                          (257, 208, 64, 1), (300, 2064, 272, 3)])
def test_fc_dequantized_output_every_tile_config(capi, cfg, M, K, N, splits):
    if 10 < cfg < 20 and K % 64 != 0:
        pytest.skip("the global-load direct-to-LDS kernels need K % 64 == 0")
    if cfg < 10 and splits > 1:
        pytest.skip("the register-staged kernels have no split-K form")
    d = int8_uniform((M, K), seed=cfg + M + 11)
    w = int8_uniform((N, K), seed=cfg + N + 13)
    b = int8_uniform((N,), seed=cfg + 17)
    check_fc_f32(capi, d, w, b, (-30.0, 28.0), bool(cfg % 2), force=(cfg, splits))


def test_fc_dequantized_output_matches_the_three_kernels(capi):
    """The fused launch against this library's own quantized_fc -> requantize -> dequantize."""
    M, K, N = 4096, 768, 2304
    d = int8_uniform((M, K), seed=31)
    w = int8_uniform((N, K), seed=32, lo=-30, hi=30)
    b = int8_uniform((N,), seed=33)
    ranges = [f32(-1.0), f32(1.0), f32(-0.08), f32(0.08), f32(-0.5), f32(0.5)]
    dd, wd, bd = dev(d), dev(w), dev(b)
    res = capi.quantized_fc(dd, wd, bd, *ranges, want_int32=True)
    fl = res["out32"].float() * (res["omax"].item() / 2147483648.0)
    R = float(fl.abs().quantile(0.99).item())
    q, qmn, qmx = capi.requantize(res["out32"], res["omin"], res["omax"], min_calib_range=-R,
                                  max_calib_range=R)
    y = capi.dequantize(q, qmn, qmx)
    fused = capi.quantized_fc_f32(dd, wd, bd, *ranges, calib=(-R, R))
    assert torch.equal(fused["outf"].view(torch.int32), y.view(torch.int32))
    assert (fused["rmin"].item(), fused["rmax"].item()) == (qmn.item(), qmx.item())


def test_fc_dequantized_output_degenerate(capi):
    # no rows: only the range scalars are written
    res = capi.quantized_fc_f32(torch.empty((0, 64), dtype=torch.int8, device="cuda"),
                                dev(int8_uniform((32, 64), seed=1)), None, f32(-1.0), f32(1.0),
                                f32(-1.0), f32(1.0), calib=(-2.0, 3.0))
    assert res["outf"].shape == (0, 32)
    assert (res["rmin"].item(), res["rmax"].item()) == (-3.0, 3.0)
    # K = 0: every output is the requantized, dequantized bias
    b = int8_uniform((40,), seed=2)
    check_fc_f32(capi, np.zeros((5, 0), np.int8), np.zeros((40, 0), np.int8), b, (-0.5, 0.5),
                 False)
    from mxnet_amd._lib import last_error, lib
    rc = lib.mxq_quantized_fc_f32(None, None, None, None, 4, 4, 16, None, None, None, None, None,
                                  None, None, None, None, None, None, 0, 0.0, 1.0, None, 0)
    assert rc != 0 and "no output buffer" in last_error()


# ---- quantized_fc -> requantize -> elemwise_add (-> relu) in one launch -----------------------
def oracle_fc_sum(d, w, b, res, calib, res_range, sum_calib, sum_relu):
    """The reference's operators one after the other."""
    rd, rw, rb = 2.0, 0.1, 1.0
    ro, rmn, rmx = oracle_fc(d, w, b, rd, rw, rb)
    rq, qmn, qmx = oracle.requantize(ro, rmn, rmx, *calib)
    out, omn, omx = oracle.quantized_elemwise_add(rq, res, qmn, qmx, -res_range, res_range,
                                                  min_calib_range=sum_calib[0],
                                                  max_calib_range=sum_calib[1])
    if sum_relu:
        out = oracle.relu_i8(out)
    return out, (rmn, rmx), (omn, omx)


def check_fc_sum(capi, d, w, b, res, calib, res_range, sum_calib, sum_relu, force=None):
    rd, rw, rb = 2.0, 0.1, 1.0
    got = capi.quantized_fc_sum(dev(d), dev(w), None if b is None else dev(b), dev(res), f32(-rd),
                                f32(rd), f32(-rw), f32(rw), None if b is None else f32(-rb),
                                None if b is None else f32(rb), f32(-res_range), f32(res_range),
                                calib, sum_calib, sum_relu=sum_relu, force=force)
    ref, r32, rsum = oracle_fc_sum(d, w, b, res, calib, res_range, sum_calib, sum_relu)
    np.testing.assert_array_equal(got["out8"].cpu().numpy(), ref)
    assert (got["omin"].item(), got["omax"].item()) == r32
    assert (got["rmin"].item(), got["rmax"].item()) == rsum


def sum_case(M, K, N, seed):
    d = int8_uniform((M, K), seed=seed)
    w = int8_uniform((N, K), seed=seed + 1)
    b = int8_uniform((N,), seed=seed + 2) if (M + N) % 2 else None
    res = int8_uniform((M, N), seed=seed + 3)
    ro, rmn, rmx = oracle_fc(d, w, b, 2.0, 0.1, 1.0)
    fl = ro.astype(np.float64) * (float(rmx) / 2147483648.0)
    R = float(np.percentile(np.abs(fl), 98.0)) or 1.0
    return d, w, b, res, R


@pytest.mark.parametrize("M,K,N", SHAPES + [(4096, 64, 256), (40000, 64, 64), (33000, 128, 128),
                                            (3136, 512, 2048), (100, 64, 6)])
@pytest.mark.parametrize("sum_relu", [False, True])
def test_fc_residual_sum(capi, M, K, N, sum_relu):
    d, w, b, res, R = sum_case(M, K, N, seed=M + K + N)
    # the residual's range and the sum's range chosen so that part of the sums saturate
    check_fc_sum(capi, d, w, b, res, (-R, 0.85 * R), 0.7 * R, (-0.9 * R, 1.1 * R), sum_relu)


@pytest.mark.parametrize("cfg", [1, 2, 3, 4, 11, 12, 14, 16, 21, 22, 23, 24, 31, 32, 41, 42, 43, 44,
                                 51, 52, 53, 54, 55, 56, 57, 58, 59, 60])
@pytest.mark.parametrize("M,K,N,splits", [(512, 512, 512, 1), (300, 192, 272, 1), (70, 448, 36, 1),
                                          (257, 208, 64, 1), (300, 2064, 272, 3)])
def test_fc_residual_sum_every_tile_config(capi, cfg, M, K, N, splits):
    if 10 < cfg < 20 and K % 64 != 0:
        pytest.skip("the global-load direct-to-LDS kernels need K % 64 == 0")
    if cfg < 10 and splits > 1:
        pytest.skip("the register-staged kernels have no split-K form")
    d, w, b, res, R = sum_case(M, K, N, seed=cfg + M)
    check_fc_sum(capi, d, w, b, res, (-R, 0.85 * R), 0.7 * R, (-0.9 * R, 1.1 * R), bool(cfg % 2),
                 force=(cfg, splits, 0))


@pytest.mark.parametrize("cfg,M,K,N", [(61, 4096, 64, 64), (62, 5000, 64, 256), (61, 777, 32, 192),
                                       (62, 2100, 128, 128), (62, 300, 256, 256)])
@pytest.mark.parametrize("sum_relu", [False, True])
def test_fc_residual_sum_streaming_kernel(capi, cfg, M, K, N, sum_relu):
    d, w, b, res, R = sum_case(M, K, N, seed=cfg + N)
    check_fc_sum(capi, d, w, b, res, (-R, 0.85 * R), 0.7 * R, (-0.9 * R, 1.1 * R), sum_relu,
                 force=(cfg, 1, 0))


def test_fc_residual_sum_huge_scales_and_misalignment(capi):
    """A residual range so large that the products could overflow takes the overflow-safe
    rule; a residual or output that is not 16-byte aligned takes the general epilogue."""
    d, w, b, res, R = sum_case(300, 192, 272, seed=5)
    check_fc_sum(capi, d, w, b, res, (-R, R), 3e38, (-1e-8, 1e-8), True)
    check_fc_sum(capi, d, w, b, res, (-R, R), 1e-30, (-3e38, 3e38), False)
    # misaligned residual: a view that starts 1 byte into a larger buffer
    rd, rw = 2.0, 0.1
    buf = torch.empty(res.size + 16, dtype=torch.int8, device="cuda")
    view = buf[1:1 + res.size].view(res.shape)
    view.copy_(dev(res))
    got = capi.quantized_fc_sum(dev(d), dev(w), None if b is None else dev(b), view, f32(-rd),
                                f32(rd), f32(-rw), f32(rw), None if b is None else f32(-1.0),
                                None if b is None else f32(1.0), f32(-0.7 * R), f32(0.7 * R),
                                (-R, R), (-R, R), sum_relu=True)
    ref, _, _ = oracle_fc_sum(d, w, b, res, (-R, R), 0.7 * R, (-R, R), True)
    np.testing.assert_array_equal(got["out8"].cpu().numpy(), ref)


def test_fc_residual_sum_matches_the_three_kernels(capi, ):
    """Against this library's own quantized_fc -> elemwise_add -> relu on a ResNet shape."""
    import mxnet_amd
    M, K, N = 50176, 128, 512
    d, w, b, res, R = sum_case(M, K, N, seed=9)
    ranges = [f32(-2.0), f32(2.0), f32(-0.1), f32(0.1)]
    bias_r = [None, None] if b is None else [f32(-1.0), f32(1.0)]
    dd, wd, bd, rs = dev(d), dev(w), None if b is None else dev(b), dev(res)
    one = capi.quantized_fc(dd, wd, bd, *ranges, *bias_r, want_int32=False, calib=(-R, R))
    s8, smn, smx = mxnet_amd.contrib.quantized_elemwise_add(
        one["out8"], rs, one["rmin"], one["rmax"], f32(-0.7 * R), f32(0.7 * R),
        min_calib_range=-R, max_calib_range=R)
    s8 = torch.clamp(s8, min=0)
    fused = capi.quantized_fc_sum(dd, wd, bd, rs, *ranges, *bias_r, f32(-0.7 * R), f32(0.7 * R),
                                  (-R, R), (-R, R), sum_relu=True)
    assert torch.equal(fused["out8"], s8)
    assert (fused["rmin"].item(), fused["rmax"].item()) == (smn.item(), smx.item())


def test_fc_residual_sum_degenerate(capi):
    res = capi.quantized_fc_sum(torch.empty((0, 64), dtype=torch.int8, device="cuda"),
                                dev(int8_uniform((32, 64), seed=1)), None,
                                torch.empty((0, 32), dtype=torch.int8, device="cuda"), f32(-1.0),
                                f32(1.0), f32(-1.0), f32(1.0), None, None, f32(-1.0), f32(1.0),
                                (-2.0, 3.0), (-4.0, 5.0))
    assert res["out8"].shape == (0, 32)
    assert (res["rmin"].item(), res["rmax"].item()) == (-4.0, 5.0)


@pytest.mark.parametrize("M,K,N", [(50176, 128, 512), (40000, 64, 256), (300, 208, 100)])
def test_fc_residual_sum_in_place(capi, M, K, N):
    """The output may be the residual operand's own buffer (the sum updates the shortcut in
    place): every piece is read before the tile that owns it is stored."""
    import ctypes
    from mxnet_amd._lib import check, lib
    d, w, b, res, R = sum_case(M, K, N, seed=M + 1)
    ref, _, _ = oracle_fc_sum(d, w, b, res, (-R, R), 0.7 * R, (-R, 1.2 * R), True)
    dd, wd, rs = dev(d), dev(w), dev(res)
    bd = None if b is None else dev(b)
    sc = [f32(v) for v in (-2.0, 2.0, -0.1, 0.1, -1.0, 1.0, -0.7 * R, 0.7 * R)]
    out = [torch.empty(1, device="cuda") for _ in range(4)]
    P = lambda t: None if t is None else ctypes.c_void_p(t.data_ptr())
    st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    check(lib.mxq_quantized_fc_sum(st, P(dd), P(wd), P(bd), M, N, K, P(sc[0]), P(sc[1]), P(sc[2]),
                                   P(sc[3]), P(sc[4]) if b is not None else None,
                                   P(sc[5]) if b is not None else None, P(rs), P(sc[6]), P(sc[7]),
                                   P(rs), P(out[0]), P(out[1]), P(out[2]), P(out[3]), -R, R, -R,
                                   1.2 * R, 1, None, 0))
    np.testing.assert_array_equal(rs.cpu().numpy(), ref)


# Exact ties and saturation in the fused requantize: ranges chosen so that every scale is a
# power of two (data and weight range 127 -> one product level = 1.0; calibrated range 254 ->
# requantize scale 0.5), accumulators that sweep the small integers of both signs.  Odd
# accumulators land exactly on k + 0.5 (rounded away from zero by the reference,
# quantization_utils.h:80-96), |acc| >= 255 saturates at 127, and with the relu every negative
# value has to come out as 0 -- through the tiled kernels, the short-K streaming kernel and
# the register-staged fallback.
@pytest.mark.parametrize("M,K,N", [(256, 16, 64), (300, 64, 128), (512, 256, 256), (64, 20, 24)])
@pytest.mark.parametrize("relu", [False, True])
def test_fc_fused_requantize_on_exact_ties(capi, M, K, N, relu):
    d = np.zeros((M, K), np.int8)
    w = np.zeros((N, K), np.int8)
    m, n = np.arange(M), np.arange(N)
    d[:, 0] = (m * 37) % 256 - 128       # every residue within 256 rows, both signs within 8
    d[:, 1] = (m * 7) % 5 - 2
    d[:, 2] = 2
    w[:, 0] = 1
    w[:, 1] = (n % 64) - 32
    w[:, 2] = 127 * (n % 3 - 1)
    ro, rmn, rmx = oracle.quantized_fully_connected(d, w, None, -127.0, 127.0, -127.0, 127.0)
    assert ro.min() < -300 and ro.max() > 300 and (ro % 2 != 0).sum() > ro.size // 4
    rq, qmn, qmx = oracle.requantize(ro, rmn, rmx, -254.0, 254.0)
    # the scale really is 0.5: the oracle's answer is round-half-away-from-zero of acc / 2
    want = np.clip(np.sign(ro) * np.floor(np.abs(ro) / 2.0 + 0.5), -127, 127).astype(np.int8)
    np.testing.assert_array_equal(rq, want)
    if relu:
        rq = oracle.relu_i8(rq)
    for want_int32 in (True, False):
        res = capi.quantized_fc(dev(d), dev(w), None, f32(-127.0), f32(127.0), f32(-127.0),
                                f32(127.0), want_int32=want_int32, calib=(-254.0, 254.0),
                                relu=relu)
        np.testing.assert_array_equal(res["out8"].cpu().numpy(), rq)
        assert (res["rmin"].item(), res["rmax"].item()) == (qmn, qmx)
