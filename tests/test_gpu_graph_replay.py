"""The entry points under HIP graph capture: a chain of them is recorded once and replayed
several times on new input contents (written into the captured buffers between replays, with
the program's own eager work and synchronisations in between); every replay must give what
the oracle gives for that input.  Covers the launches that carry state between kernels of
one call: the uncalibrated casts (reduction partials in a workspace, or in the library's own
array for the no-allocation entry point) and a split-K fully-connected layer (tile counters
cleared by a kernel of the same call, partial sums in the workspace), also in its
float-output and residual-sum forms."""
import ctypes

import numpy as np
import pytest
import torch

import oracle
from tests.data_gen import int8_uniform

pytestmark = pytest.mark.gpu


def P(t):
    return ctypes.c_void_p(t.data_ptr()) if t is not None else None


def scalar():
    return torch.empty(1, dtype=torch.float32, device="cuda")


def test_replays_follow_their_inputs():
    import mxnet_amd
    lib = mxnet_amd._lib.lib
    M, K, N = 256, 8192, 800          # the launcher splits this one along K
    n = M * K
    x = torch.empty(n, dtype=torch.float32, device="cuda")
    q = torch.empty((M, K), dtype=torch.int8, device="cuda")
    q2 = torch.empty((M, K), dtype=torch.int8, device="cuda")
    qr = [scalar() for _ in range(4)]
    w_np = int8_uniform((N, K), seed=5)
    b_np = int8_uniform((N,), seed=6)
    w, b = torch.from_numpy(w_np).cuda(), torch.from_numpy(b_np).cuda()
    wr = [torch.tensor([v], device="cuda") for v in (-0.3, 0.3, -0.9, 0.9)]
    acc = torch.empty((M, N), dtype=torch.int32, device="cuda")
    out8 = torch.empty((M, N), dtype=torch.int8, device="cuda")
    fr = [scalar() for _ in range(4)]
    r8 = torch.empty((M, N), dtype=torch.int8, device="cuda")
    rr = [scalar() for _ in range(2)]
    y = torch.empty((M, N), dtype=torch.float32, device="cuda")
    ws_q = torch.empty(lib.mxq_quantize_v2_workspace(n), dtype=torch.uint8, device="cuda")
    ws_r = torch.empty(lib.mxq_requantize_workspace(M * N), dtype=torch.uint8, device="cuda")
    nfc = lib.mxq_quantized_fc_workspace(M, N, K, 0)
    assert nfc > 0, "this shape is expected to ask for a split-K workspace"
    ws_fc = torch.empty(nfc, dtype=torch.uint8, device="cuda")
    # the float-output and residual-sum forms of the same split layer, each with a workspace
    # of its own (launches of one graph may not share one)
    ws_f32 = torch.empty(nfc, dtype=torch.uint8, device="cuda")
    ws_sum = torch.empty(lib.mxq_quantized_fc_workspace(M, N, K, 1), dtype=torch.uint8,
                         device="cuda")
    yf = torch.empty((M, N), dtype=torch.float32, device="cuda")
    ff = [scalar() for _ in range(4)]
    res_np = int8_uniform((M, N), seed=8)
    res = torch.from_numpy(res_np).cuda()
    res_r = [torch.tensor([v], device="cuda") for v in (-30.0, 30.0)]
    s8 = torch.empty((M, N), dtype=torch.int8, device="cuda")
    fs = [scalar() for _ in range(4)]
    calib = 40.0

    def body():
        st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
        rcs = [
            # uncalibrated quantize: partials in the caller's workspace ...
            lib.mxq_quantize_v2(st, P(x), P(q), P(qr[0]), P(qr[1]), n, 5, 0, 0.0, 0.0, P(ws_q),
                                ws_q.numel()),
            # ... and in the library's own array
            lib.mxq_quantize_v2_noalloc(st, P(x), P(q2), P(qr[2]), P(qr[3]), n, 5, 0, 0.0, 0.0),
            lib.mxq_quantized_fc(st, P(q), P(w), P(b), M, N, K, P(qr[0]), P(qr[1]), P(wr[0]),
                                 P(wr[1]), P(wr[2]), P(wr[3]), P(acc), P(fr[0]), P(fr[1]),
                                 P(out8), P(fr[2]), P(fr[3]), 0, -calib, calib, P(ws_fc),
                                 ws_fc.numel()),
            # uncalibrated requantize of the int32 output
            lib.mxq_requantize(st, P(acc), P(fr[0]), P(fr[1]), P(r8), P(rr[0]), P(rr[1]), M * N,
                               0, 0.0, 0.0, P(ws_r), ws_r.numel()),
            lib.mxq_dequantize(st, P(r8), 5, P(rr[0]), P(rr[1]), P(y), M * N),
            lib.mxq_quantized_fc_f32(st, P(q), P(w), P(b), M, N, K, P(qr[0]), P(qr[1]), P(wr[0]),
                                     P(wr[1]), P(wr[2]), P(wr[3]), P(yf), P(ff[0]), P(ff[1]),
                                     P(ff[2]), P(ff[3]), 0, -calib, calib, P(ws_f32),
                                     ws_f32.numel()),
            lib.mxq_quantized_fc_sum(st, P(q), P(w), P(b), M, N, K, P(qr[0]), P(qr[1]), P(wr[0]),
                                     P(wr[1]), P(wr[2]), P(wr[3]), P(res), P(res_r[0]),
                                     P(res_r[1]), P(s8), P(fs[0]), P(fs[1]), P(fs[2]), P(fs[3]),
                                     -calib, calib, -50.0, 45.0, 1, P(ws_sum), ws_sum.numel()),
        ]
        assert not any(rcs), mxnet_amd._lib.last_error()

    rng = np.random.default_rng(3)
    first = rng.standard_normal(n).astype(np.float32)
    x.copy_(torch.from_numpy(first))
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        body()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        body()

    for it in range(4):
        data = (rng.standard_normal(n) * (1.0 + it)).astype(np.float32)
        data[it] = 7.0 * (it + 1)                     # the range changes with every replay
        x.copy_(torch.from_numpy(data))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        oq, omn, omx = oracle.quantize_v2(data, "int8")
        np.testing.assert_array_equal(q.cpu().numpy().ravel(), oq)
        np.testing.assert_array_equal(q2.cpu().numpy().ravel(), oq)
        assert (qr[0].item(), qr[1].item()) == (omn, omx)
        assert (qr[2].item(), qr[3].item()) == (omn, omx)
        ro, rmn, rmx = oracle.quantized_fully_connected(oq.reshape(M, K), w_np, b_np, omn, omx,
                                                        -0.3, 0.3, -0.9, 0.9)
        np.testing.assert_array_equal(acc.cpu().numpy(), ro)
        assert (fr[0].item(), fr[1].item()) == (rmn, rmx)
        fq, fmn, fmx = oracle.requantize(ro, rmn, rmx, -calib, calib)
        np.testing.assert_array_equal(out8.cpu().numpy(), fq)
        uq, umn, umx = oracle.requantize(ro, rmn, rmx)
        np.testing.assert_array_equal(r8.cpu().numpy(), uq)
        assert (rr[0].item(), rr[1].item()) == (umn, umx)
        np.testing.assert_array_equal(y.cpu().numpy(), oracle.dequantize(uq, umn, umx))
        np.testing.assert_array_equal(yf.cpu().numpy().view(np.uint32),
                                      oracle.dequantize(fq, fmn, fmx).view(np.uint32))
        sq, smn, smx = oracle.quantized_elemwise_add(fq, res_np, fmn, fmx, -30.0, 30.0,
                                                     min_calib_range=-50.0, max_calib_range=45.0)
        np.testing.assert_array_equal(s8.cpu().numpy(), oracle.relu_i8(sq))
        assert (fs[2].item(), fs[3].item()) == (smn, smx)
        # the program's own eager work between replays
        (x * 2.0).sum().item()


def test_conv_nchw_replays_follow_their_inputs():
    """mxq_quantized_conv_nchw under capture, one call per route that passes data between the
    launches of a call: the NCHW kernel alone (whole planes), its gathering loader, the
    pre-pass into the workspace, and the layout adapters (two operand copies in the
    workspace).  Replayed on new data and new weights."""
    import mxnet_amd
    lib = mxnet_amd._lib.lib
    # (N, C, H, W, O, K, stride, pad)
    cases = [(3, 64, 8, 12, 72, 1, 1, 0),       # whole planes of 96 pixels
             (3, 64, 16, 24, 72, 1, 2, 0),      # stride 2 over rows of 12: the loader gathers
             (4, 1024, 14, 14, 512, 1, 2, 0),   # 14 -> 7: the pre-pass
             (2, 32, 9, 11, 40, 3, 1, 1)]       # 3 x 3: the adapters
    one = [torch.tensor([v], device="cuda") for v in (-1.0, 1.0)]
    slots = []
    for (N, C, H, W, O, K, s, p) in cases:
        OH, OW = (H + 2 * p - K) // s + 1, (W + 2 * p - K) // s + 1
        geo = (N, C, H, W, O, K, K, s, s, p, p, 1, 1)
        nws = lib.mxq_quantized_conv_nchw_workspace(*geo, 1)
        slots.append(dict(
            geo=geo, d=torch.empty((N, C, H, W), dtype=torch.int8, device="cuda"),
            w=torch.empty((O, C, K, K), dtype=torch.int8, device="cuda"),
            b=torch.from_numpy(int8_uniform((O,), seed=O)).cuda(),
            out=torch.empty((N, O, OH, OW), dtype=torch.int32, device="cuda"),
            r=[scalar(), scalar()], nws=nws,
            ws=torch.empty(max(nws, 16), dtype=torch.uint8, device="cuda")))
    assert slots[0]["nws"] == 0 and slots[1]["nws"] == 0 and slots[2]["nws"] > 0 and slots[3]["nws"] > 0

    def body():
        st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
        for k in slots:
            rc = lib.mxq_quantized_conv_nchw(st, P(k["d"]), P(k["w"]), P(k["b"]), *k["geo"],
                                             P(one[0]), P(one[1]), P(one[0]), P(one[1]),
                                             P(one[0]), P(one[1]), P(k["out"]), P(k["r"][0]),
                                             P(k["r"][1]), P(k["ws"]) if k["nws"] else None,
                                             k["nws"])
            assert rc == 0, lib.mxq_last_error().decode()

    def load(seed):
        for i, k in enumerate(slots):
            k["d_np"] = int8_uniform(tuple(k["d"].shape), seed=seed + 10 * i)
            k["w_np"] = int8_uniform(tuple(k["w"].shape), seed=seed + 10 * i + 1)
            k["d"].copy_(torch.from_numpy(k["d_np"]))
            k["w"].copy_(torch.from_numpy(k["w_np"]))

    def check():
        torch.cuda.synchronize()
        for k in slots:
            g = k["geo"]
            ro, rmn, rmx = oracle.quantized_conv(k["d_np"], k["w_np"], k["b"].cpu().numpy(), -1.0,
                                                 1.0, -1.0, 1.0, -1.0, 1.0, (g[7], g[8]),
                                                 (g[9], g[10]), (1, 1))
            np.testing.assert_array_equal(k["out"].cpu().numpy(), ro)
            assert (k["r"][0].item(), k["r"][1].item()) == (rmn, rmx)

    load(1)
    body()                       # eager: also the warm-up a capture needs
    check()
    graph = torch.cuda.CUDAGraph()
    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        body()
        torch.cuda.synchronize()
        with torch.cuda.graph(graph, stream=stream):
            body()
    for seed in (100, 200, 300):
        load(seed)
        for k in slots:          # nothing left over from the last replay may pass as a result
            k["out"].fill_(-1)
        torch.cuda.synchronize()
        graph.replay()
        check()
