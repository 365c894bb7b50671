"""The C ABI keeps no state between calls: host threads that drive different streams at the
same time (engine worker threads) get the results each would get alone.  Four threads, each
on its own stream, interleave FC, conv, quantize (uncalibrated: private workspace) and
requantize calls of different shapes; every result is compared with the CPU oracle."""
import threading

import numpy as np
import pytest
import torch

import oracle
from tests.data_gen import int8_uniform

pytestmark = pytest.mark.gpu


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def f32(v):
    return dev(np.array([v], np.float32))


def worker(idx, capi, failures, rounds):
    try:
        stream = torch.cuda.Stream()
        rng = np.random.default_rng(idx)
        with torch.cuda.stream(stream):
            for it in range(rounds):
                M, N, K = [(70, 33, 444), (256, 192, 1024), (129, 64, 64), (40, 320, 8192)][(idx + it) % 4]
                d, w = int8_uniform((M, K), seed=idx * 100 + it), int8_uniform((N, K), seed=idx * 100 + it + 50)
                b = int8_uniform((N,), seed=idx + it)
                res = capi.quantized_fc(dev(d), dev(w), dev(b), f32(-1.0), f32(1.0), f32(-0.1), f32(0.1),
                                        f32(-0.5), f32(0.5), want_int32=True, calib=(-3.0, 2.5))
                x = rng.standard_normal(50000 + 1000 * idx + it).astype(np.float32)
                q, qmn, qmx = capi.quantize_v2(dev(x), "int8")
                c = int8_uniform((2, 32, 9, 7 + idx), seed=idx + it + 7)
                cw = int8_uniform((24, 32, 3, 3), seed=idx + it + 9)
                cres = capi.quantized_conv_nhwc(capi.nchw_to_nhwc_i8(dev(c)), capi.nchw_to_nhwc_i8(dev(cw)),
                                                None, f32(-1.0), f32(1.0), f32(-1.0), f32(1.0), stride=(1, 1),
                                                pad=(1, 1), want_int32=True)
                conv_out = capi.nhwc_to_nchw(cres["out32"])
                stream.synchronize()
                ro, rmn, rmx = oracle.quantized_fully_connected(d, w, b, -1.0, 1.0, -0.1, 0.1, -0.5, 0.5)
                np.testing.assert_array_equal(res["out32"].cpu().numpy(), ro)
                rq, _, _ = oracle.requantize(ro, rmn, rmx, -3.0, 2.5)
                np.testing.assert_array_equal(res["out8"].cpu().numpy(), rq)
                oq, omn, omx = oracle.quantize_v2(x, "int8")
                np.testing.assert_array_equal(q.cpu().numpy(), oq)
                assert (qmn.item(), qmx.item()) == (omn, omx)
                co, _, _ = oracle.quantized_conv(c, cw, None, -1.0, 1.0, -1.0, 1.0, None, None, (1, 1), (1, 1), (1, 1))
                np.testing.assert_array_equal(conv_out.cpu().numpy(), co)
    except BaseException as e:  # noqa: BLE001 - reported to the main thread
        failures.append((idx, repr(e)))


def test_concurrent_callers_on_their_own_streams():
    import mxnet_amd
    capi = mxnet_amd.capi
    failures = []
    threads = [threading.Thread(target=worker, args=(i, capi, failures, 6)) for i in range(4)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    torch.cuda.synchronize()
    assert not failures, failures
