"""Thin torch-tensor wrappers over the C ABI (one function per entry point).
Tensors must be contiguous CUDA(HIP) tensors; outputs are allocated with torch
and the calls are enqueued on torch's current stream."""
import ctypes

import torch

from . import _lib
from ._lib import INT8, UINT8, check, lib

_TYPE_CODE = {torch.int8: INT8, torch.uint8: UINT8}


def _stream():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _ptr(t):
    if t is None:
        return None
    assert t.is_cuda and t.is_contiguous(), "need a contiguous device tensor"
    return ctypes.c_void_p(t.data_ptr())


def _scalar(dev):
    return torch.empty(1, dtype=torch.float32, device=dev)


def _workspace(nbytes, dev):
    return torch.empty(nbytes, dtype=torch.uint8, device=dev)


# scratch handed to the test-only entry points when a test pins a split-K factor: room for
# the partial sums of every case the tests run (the launcher checks the size it needs)
_SPLIT_WS_BYTES = 96 << 20


def quantize_v2(data, out_type="int8", min_calib_range=None, max_calib_range=None):
    assert data.dtype == torch.float32
    calibrated = min_calib_range is not None and max_calib_range is not None
    if out_type == "auto":
        out_type = "uint8" if (calibrated and min_calib_range >= 0.0) else "int8"
    dt = {"int8": torch.int8, "uint8": torch.uint8}[out_type]
    out = torch.empty(data.shape, dtype=dt, device=data.device)
    omin, omax = _scalar(data.device), _scalar(data.device)
    n = data.numel()
    ws = None
    wsb = 0
    if not calibrated:
        wsb = lib.mxq_quantize_v2_workspace(n)
        ws = _workspace(wsb, data.device)
    check(lib.mxq_quantize_v2(_stream(), _ptr(data), _ptr(out), _ptr(omin), _ptr(omax), n,
                              _TYPE_CODE[dt], int(calibrated),
                              float(min_calib_range or 0.0), float(max_calib_range or 0.0),
                              _ptr(ws), wsb))
    return out, omin, omax


def quantize(data, min_range, max_range, out_type="int8"):
    assert data.dtype == torch.float32
    dt = {"int8": torch.int8, "uint8": torch.uint8}[out_type]
    out = torch.empty(data.shape, dtype=dt, device=data.device)
    omin, omax = _scalar(data.device), _scalar(data.device)
    check(lib.mxq_quantize(_stream(), _ptr(data), _ptr(min_range), _ptr(max_range), _ptr(out),
                           _ptr(omin), _ptr(omax), data.numel(), _TYPE_CODE[dt]))
    return out, omin, omax


def requantize(data, min_range, max_range, min_calib_range=None, max_calib_range=None):
    assert data.dtype == torch.int32
    calibrated = min_calib_range is not None and max_calib_range is not None
    out = torch.empty(data.shape, dtype=torch.int8, device=data.device)
    omin, omax = _scalar(data.device), _scalar(data.device)
    n = data.numel()
    ws = None
    wsb = 0
    if not calibrated:
        wsb = lib.mxq_requantize_workspace(n)
        ws = _workspace(wsb, data.device)
    check(lib.mxq_requantize(_stream(), _ptr(data), _ptr(min_range), _ptr(max_range), _ptr(out),
                             _ptr(omin), _ptr(omax), n, int(calibrated),
                             float(min_calib_range or 0.0), float(max_calib_range or 0.0),
                             _ptr(ws), wsb))
    return out, omin, omax


def dequantize(data, min_range, max_range):
    out = torch.empty(data.shape, dtype=torch.float32, device=data.device)
    check(lib.mxq_dequantize(_stream(), _ptr(data), _TYPE_CODE[data.dtype], _ptr(min_range),
                             _ptr(max_range), _ptr(out), data.numel()))
    return out


def quantized_fc(data, weight, bias, min_data, max_data, min_weight, max_weight, min_bias=None,
                 max_bias=None, want_int32=True, calib=None, relu=False, force=None):
    """data int8 [M,K], weight int8 [N,K], bias int8 [N] or None.
    Returns dict(out32, omin, omax[, out8, rmin, rmax]).  `force` = (cfg, splits,
    stream_groups) goes through the test-only entry point that pins the kernel variant."""
    M, K = data.shape
    N, K2 = weight.shape
    assert K == K2
    dev = data.device
    res = {"omin": _scalar(dev), "omax": _scalar(dev)}
    out32 = torch.empty((M, N), dtype=torch.int32, device=dev) if want_int32 else None
    out8 = rmin = rmax = None
    lo = hi = 0.0
    if calib is not None:
        out8 = torch.empty((M, N), dtype=torch.int8, device=dev)
        rmin, rmax = _scalar(dev), _scalar(dev)
        lo, hi = float(calib[0]), float(calib[1])
    args = [_stream(), _ptr(data), _ptr(weight), _ptr(bias), M, N, K, _ptr(min_data),
            _ptr(max_data), _ptr(min_weight), _ptr(max_weight), _ptr(min_bias), _ptr(max_bias),
            _ptr(out32), _ptr(res["omin"]), _ptr(res["omax"]), _ptr(out8), _ptr(rmin),
            _ptr(rmax), int(relu), lo, hi]
    if force is None:
        wsb = lib.mxq_quantized_fc_workspace(M, N, K, int(not want_int32))
        ws = _workspace(wsb, dev) if wsb else None
        check(lib.mxq_quantized_fc(*args, _ptr(ws), wsb))
    else:
        cfg, splits, groups = force
        wsb = _SPLIT_WS_BYTES if splits > 1 else 0
        ws = _workspace(wsb, dev) if wsb else None
        check(lib.mxq_test_quantized_fc(*args, _ptr(ws), wsb, cfg, splits, groups))
    res.update(out32=out32, out8=out8, rmin=rmin, rmax=rmax)
    return res


def quantized_fc_f32(data, weight, bias, min_data, max_data, min_weight, max_weight,
                     min_bias=None, max_bias=None, calib=(-1.0, 1.0), relu=False, force=None):
    """quantized_fc -> requantize over `calib` -> dequantize in one launch.  Returns
    dict(outf, omin, omax, rmin, rmax).  `force` = (cfg, splits) pins the kernel variant
    through the test-only entry point."""
    M, K = data.shape
    N, K2 = weight.shape
    assert K == K2
    dev = data.device
    res = {k: _scalar(dev) for k in ("omin", "omax", "rmin", "rmax")}
    res["outf"] = torch.empty((M, N), dtype=torch.float32, device=dev)
    args = [_stream(), _ptr(data), _ptr(weight), _ptr(bias), M, N, K, _ptr(min_data),
            _ptr(max_data), _ptr(min_weight), _ptr(max_weight), _ptr(min_bias), _ptr(max_bias),
            _ptr(res["outf"]), _ptr(res["omin"]), _ptr(res["omax"]), _ptr(res["rmin"]),
            _ptr(res["rmax"]), int(relu), float(calib[0]), float(calib[1])]
    if force is None:
        wsb = lib.mxq_quantized_fc_workspace(M, N, K, 0)
        ws = _workspace(wsb, dev) if wsb else None
        check(lib.mxq_quantized_fc_f32(*args, _ptr(ws), wsb))
    else:
        cfg, splits = force
        wsb = _SPLIT_WS_BYTES if splits > 1 else 0
        ws = _workspace(wsb, dev) if wsb else None
        check(lib.mxq_test_quantized_fc_f32(*args, _ptr(ws), wsb, cfg, splits))
    return res


def quantized_fc_sum(data, weight, bias, residual, min_data, max_data, min_weight, max_weight,
                     min_bias, max_bias, min_residual, max_residual, calib, sum_calib,
                     sum_relu=False, force=None):
    """quantized_fc -> requantize over `calib` -> elemwise_add with `residual` over `sum_calib`
    (-> relu) in one launch.  Returns dict(out8, omin, omax, rmin, rmax).  `force` = (cfg,
    splits, stream_groups) pins the kernel variant through the test-only entry point."""
    M, K = data.shape
    N, K2 = weight.shape
    assert K == K2 and tuple(residual.shape) == (M, N) and residual.dtype == torch.int8
    dev = data.device
    res = {k: _scalar(dev) for k in ("omin", "omax", "rmin", "rmax")}
    res["out8"] = torch.empty((M, N), dtype=torch.int8, device=dev)
    args = [_stream(), _ptr(data), _ptr(weight), _ptr(bias), M, N, K, _ptr(min_data),
            _ptr(max_data), _ptr(min_weight), _ptr(max_weight), _ptr(min_bias), _ptr(max_bias),
            _ptr(residual), _ptr(min_residual), _ptr(max_residual), _ptr(res["out8"]),
            _ptr(res["omin"]), _ptr(res["omax"]), _ptr(res["rmin"]), _ptr(res["rmax"]),
            float(calib[0]), float(calib[1]), float(sum_calib[0]), float(sum_calib[1]),
            int(sum_relu)]
    if force is None:
        wsb = lib.mxq_quantized_fc_workspace(M, N, K, 1)
        ws = _workspace(wsb, dev) if wsb else None
        check(lib.mxq_quantized_fc_sum(*args, _ptr(ws), wsb))
    else:
        cfg, splits, groups = force
        wsb = _SPLIT_WS_BYTES if splits > 1 else 0
        ws = _workspace(wsb, dev) if wsb else None
        check(lib.mxq_test_quantized_fc_sum(*args, _ptr(ws), wsb, cfg, splits, groups))
    return res


def quantized_conv_nhwc(data, weight, bias, min_data, max_data, min_weight, max_weight,
                        min_bias=None, max_bias=None, stride=(1, 1), pad=(0, 0), dilate=(1, 1),
                        want_int32=True, calib=None, relu=False, force=None):
    """data int8 [N,H,W,C], weight int8 [O,KH,KW,C] -> out [N,OH,OW,O].  `force` = (cfg,
    splits) goes through the test-only entry point that pins the kernel variant."""
    N, H, W, C = data.shape
    O, KH, KW, C2 = weight.shape
    assert C == C2
    OH = (H + 2 * pad[0] - (dilate[0] * (KH - 1) + 1)) // stride[0] + 1
    OW = (W + 2 * pad[1] - (dilate[1] * (KW - 1) + 1)) // stride[1] + 1
    dev = data.device
    res = {"omin": _scalar(dev), "omax": _scalar(dev)}
    out32 = torch.empty((N, OH, OW, O), dtype=torch.int32, device=dev) if want_int32 else None
    out8 = rmin = rmax = None
    lo = hi = 0.0
    if calib is not None:
        out8 = torch.empty((N, OH, OW, O), dtype=torch.int8, device=dev)
        rmin, rmax = _scalar(dev), _scalar(dev)
        lo, hi = float(calib[0]), float(calib[1])
    geo = [N, H, W, C, O, KH, KW, stride[0], stride[1], pad[0], pad[1], dilate[0], dilate[1]]
    args = [_stream(), _ptr(data), _ptr(weight), _ptr(bias)] + geo + [
        _ptr(min_data), _ptr(max_data), _ptr(min_weight), _ptr(max_weight), _ptr(min_bias),
        _ptr(max_bias), _ptr(out32), _ptr(res["omin"]), _ptr(res["omax"]), _ptr(out8),
        _ptr(rmin), _ptr(rmax), int(relu), lo, hi]
    if force is None:
        wsb = lib.mxq_quantized_conv_workspace(*geo, int(not want_int32))
        ws = _workspace(wsb, dev) if wsb else None
        check(lib.mxq_quantized_conv_nhwc(*args, _ptr(ws), wsb))
    else:
        cfg, splits = force
        wsb = _SPLIT_WS_BYTES if splits > 1 else 0
        ws = _workspace(wsb, dev) if wsb else None
        check(lib.mxq_test_quantized_conv_nhwc(*args, _ptr(ws), wsb, cfg, splits))
    res.update(out32=out32, out8=out8, rmin=rmin, rmax=rmax)
    return res


def quantized_conv_nchw(data, weight, bias, min_data, max_data, min_weight, max_weight,
                        min_bias=None, max_bias=None, stride=(1, 1), pad=(0, 0), dilate=(1, 1),
                        cfg=None, out=None):
    """The operator's contract: data int8 [N,C,H,W], weight int8 [O,C,KH,KW] -> int32
    [N,O,OH,OW].  `cfg` pins the route through the test-only entry point (1 = layout
    adapters, 71... = a tile of the NCHW 1x1 kernel)."""
    N, C, H, W = data.shape
    O, C2, KH, KW = weight.shape
    assert C == C2
    OH = (H + 2 * pad[0] - (dilate[0] * (KH - 1) + 1)) // stride[0] + 1
    OW = (W + 2 * pad[1] - (dilate[1] * (KW - 1) + 1)) // stride[1] + 1
    dev = data.device
    res = {"omin": _scalar(dev), "omax": _scalar(dev)}
    out32 = out if out is not None else torch.empty((N, O, OH, OW), dtype=torch.int32, device=dev)
    geo = [N, C, H, W, O, KH, KW, stride[0], stride[1], pad[0], pad[1], dilate[0], dilate[1]]
    both_aligned = data.data_ptr() % 16 == 0 and weight.data_ptr() % 16 == 0 and cfg != 1
    wsb = lib.mxq_quantized_conv_nchw_workspace(*geo, int(both_aligned))
    ws = _workspace(wsb, dev) if wsb else None
    args = [_stream(), _ptr(data), _ptr(weight), _ptr(bias)] + geo + [
        _ptr(min_data), _ptr(max_data), _ptr(min_weight), _ptr(max_weight), _ptr(min_bias),
        _ptr(max_bias), _ptr(out32), _ptr(res["omin"]), _ptr(res["omax"]), _ptr(ws), wsb]
    if cfg is None:
        check(lib.mxq_quantized_conv_nchw(*args))
    else:
        check(lib.mxq_test_quantized_conv_nchw(*args, int(cfg)))
    res["out32"] = out32
    res["workspace_bytes"] = wsb
    return res


def nchw_to_nhwc_i8(x):
    N, C, H, W = x.shape
    out = torch.empty((N, H, W, C), dtype=torch.int8, device=x.device)
    check(lib.mxq_nchw_to_nhwc_i8(_stream(), _ptr(x), _ptr(out), N, C, H, W))
    return out


def nhwc_to_nchw(x):
    N, H, W, C = x.shape
    out = torch.empty((N, C, H, W), dtype=x.dtype, device=x.device)
    check(lib.mxq_nhwc_to_nchw(_stream(), _ptr(x), _ptr(out), N, C, H, W, x.element_size()))
    return out
