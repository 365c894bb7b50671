"""ctypes binding of oracle/mxq_oracle.c (the CPU restatement of the
reference's native int8 arithmetic).  TEST INFRASTRUCTURE ONLY: the product
never imports this module."""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libmxq_oracle.so")


def build(force=False):
    """Compile the oracle with gcc (see Makefile for the flags)."""
    if force and os.path.exists(_SO):
        os.remove(_SO)
    subprocess.check_call(["make", "-s", "-C", _HERE, "libmxq_oracle.so"])
    return _SO


def _load():
    if not os.path.exists(_SO):
        build()
    return ctypes.CDLL(_SO)


_lib = _load()
_f = ctypes.c_float
_sz = ctypes.c_size_t
_i = ctypes.c_int
_p = ctypes.c_void_p
_pf = ctypes.POINTER(ctypes.c_float)

_lib.qref_num_threads.restype = _i
_lib.qref_quantize_int8.argtypes = [_p, _sz, _f, _f, _p, _pf, _pf]
_lib.qref_quantize_uint8.argtypes = [_p, _sz, _f, _f, _p, _pf, _pf]
_lib.qref_minmax_f32.argtypes = [_p, _sz, _pf, _pf]
_lib.qref_minmax_i32.argtypes = [_p, _sz, ctypes.POINTER(ctypes.c_int32),
                                 ctypes.POINTER(ctypes.c_int32)]
_lib.qref_requantize.argtypes = [_p, _sz, _f, _f, _f, _p, _pf, _pf]
_lib.qref_requantize_actual_range.argtypes = [_p, _sz, _f, _f]
_lib.qref_requantize_actual_range.restype = _f
_lib.qref_dequantize_int8.argtypes = [_p, _sz, _f, _f, _p]
_lib.qref_dequantize_uint8.argtypes = [_p, _sz, _f, _f, _p]
_lib.qref_range_for_multiplication.argtypes = [_f, _f, _f, _f, _pf, _pf]
_lib.qref_bias_i8_to_i32.argtypes = [_p, _sz, _f, _f, _f, _f, _p]
_lib.qref_fc.argtypes = [_p, _p, _p, _i, _i, _i, _p]
_lib.qref_conv_nchw.argtypes = [_p, _p, _p] + [_i] * 13 + [_p]
_lib.qref_relu_i8.argtypes = [_p, _sz, _p]
_lib.qref_pool_nchw.argtypes = [_p, _i] + [_i] * 12 + [_i, _i, _p]
_lib.qref_elemwise_add.argtypes = [_p, _i, _p, _i, _sz, _f, _f, _f, _f, _i, _i, _f, _f, _p, _pf,
                                   _pf]
_lib.qref_broadcast_add.argtypes = _lib.qref_elemwise_add.argtypes
_lib.qref_concat_rescale.argtypes = [_p, _i, _sz, _f, _f, _f, _f, _i, _p]
_lib.qref_elemwise_mul.argtypes = [_p, _p, _sz, _f, _f, _f, _f, _i, _f, _f, _p, _pf, _pf]
_lib.qref_quantize_asym.argtypes = [_p, _sz, _f, _f, _p, _pf, _pf]
_lib.qref_batch_norm.argtypes = [_p, _i, _sz, _sz, _sz, _p, _p, _p, _p, _f, _f, ctypes.c_double,
                                 _f, _f, _i, _p, _pf, _pf]


def _c(a, dtype):
    a = np.ascontiguousarray(a, dtype=dtype)
    return a


def _ptr(a):
    return a.ctypes.data_as(ctypes.c_void_p)


def num_threads():
    return int(_lib.qref_num_threads())


def minmax_f32(x):
    x = _c(x, np.float32)
    mn, mx = _f(), _f()
    _lib.qref_minmax_f32(_ptr(x), x.size, ctypes.byref(mn), ctypes.byref(mx))
    return np.float32(mn.value), np.float32(mx.value)


def minmax_i32(x):
    x = _c(x, np.int32)
    mn, mx = ctypes.c_int32(), ctypes.c_int32()
    _lib.qref_minmax_i32(_ptr(x), x.size, ctypes.byref(mn), ctypes.byref(mx))
    return int(mn.value), int(mx.value)


def quantize_v2(x, out_type="int8", min_calib_range=None, max_calib_range=None):
    """_contrib_quantize_v2 on fp32 data -> (q, min, max); out_type 'auto' follows
    GetQuantizeOutputType (quantization_utils.h:201-220)."""
    x = _c(x, np.float32)
    calibrated = min_calib_range is not None and max_calib_range is not None
    if out_type == "auto":
        out_type = "uint8" if (calibrated and min_calib_range >= 0.0) else "int8"
    if calibrated:
        lo, hi = np.float32(min_calib_range), np.float32(max_calib_range)
    else:
        lo, hi = minmax_f32(x)
    omin, omax = _f(), _f()
    if out_type == "int8":
        q = np.empty(x.shape, np.int8)
        _lib.qref_quantize_int8(_ptr(x), x.size, lo, hi, _ptr(q), ctypes.byref(omin),
                                ctypes.byref(omax))
    elif out_type == "uint8":
        q = np.empty(x.shape, np.uint8)
        _lib.qref_quantize_uint8(_ptr(x), x.size, lo, hi, _ptr(q), ctypes.byref(omin),
                                 ctypes.byref(omax))
    else:
        raise ValueError(out_type)
    return q, np.float32(omin.value), np.float32(omax.value)


def quantize(x, min_range, max_range, out_type="int8"):
    """v1 _contrib_quantize (quantize-inl.h:50-88): ranges are inputs."""
    return quantize_v2(x, out_type, float(min_range), float(max_range))


def requantize(x, min_range, max_range, min_calib_range=None, max_calib_range=None):
    x = _c(x, np.int32)
    imin, imax = np.float32(min_range), np.float32(max_range)
    if min_calib_range is not None and max_calib_range is not None:
        rr = np.float32(max(abs(np.float32(min_calib_range)), abs(np.float32(max_calib_range))))
    else:
        rr = np.float32(_lib.qref_requantize_actual_range(_ptr(x), x.size, imin, imax))
    q = np.empty(x.shape, np.int8)
    omin, omax = _f(), _f()
    _lib.qref_requantize(_ptr(x), x.size, imin, imax, rr, _ptr(q), ctypes.byref(omin),
                         ctypes.byref(omax))
    return q, np.float32(omin.value), np.float32(omax.value)


def dequantize(q, min_range, max_range):
    q = np.ascontiguousarray(q)
    out = np.empty(q.shape, np.float32)
    if q.dtype == np.int8:
        _lib.qref_dequantize_int8(_ptr(q), q.size, np.float32(min_range), np.float32(max_range),
                                  _ptr(out))
    elif q.dtype == np.uint8:
        _lib.qref_dequantize_uint8(_ptr(q), q.size, np.float32(min_range),
                                   np.float32(max_range), _ptr(out))
    else:
        raise TypeError(q.dtype)
    return out


def range_for_multiplication(min_a, max_a, min_b, max_b):
    mn, mx = _f(), _f()
    _lib.qref_range_for_multiplication(np.float32(min_a), np.float32(max_a), np.float32(min_b),
                                       np.float32(max_b), ctypes.byref(mn), ctypes.byref(mx))
    return np.float32(mn.value), np.float32(mx.value)


def bias_i8_to_i32(bias, min_out, max_out, min_bias, max_bias):
    bias = _c(bias, np.int8)
    out = np.empty(bias.shape, np.int32)
    _lib.qref_bias_i8_to_i32(_ptr(bias), bias.size, np.float32(min_out), np.float32(max_out),
                             np.float32(min_bias), np.float32(max_bias), _ptr(out))
    return out


def fc_int32(data, weight, bias32=None):
    """Raw exact contraction: data int8 [M,K], weight int8 [N,K], bias32 int32 [N]."""
    data = _c(data, np.int8)
    weight = _c(weight, np.int8)
    M, K = data.shape
    N, K2 = weight.shape
    assert K == K2
    out = np.empty((M, N), np.int32)
    b = None
    if bias32 is not None:
        b = _c(bias32, np.int32)
        assert b.shape == (N,)
    _lib.qref_fc(_ptr(data), _ptr(weight), _ptr(b) if b is not None else None, M, N, K,
                 _ptr(out))
    return out


def quantized_fully_connected(data, weight, bias, min_data, max_data, min_weight, max_weight,
                              min_bias=None, max_bias=None, flatten=True):
    """_contrib_quantized_fully_connected -> (int32 out, min_out, max_out)."""
    data = _c(data, np.int8)
    weight = _c(weight, np.int8)
    if flatten:
        d2 = data.reshape(data.shape[0], int(np.prod(data.shape[1:], dtype=np.int64)))
    else:
        d2 = data.reshape(int(np.prod(data.shape[:-1], dtype=np.int64)), data.shape[-1])
    mn, mx = range_for_multiplication(min_data, max_data, min_weight, max_weight)
    b32 = None
    if bias is not None:
        b32 = bias_i8_to_i32(bias, mn, mx, min_bias, max_bias)
    out = fc_int32(d2, weight, b32)
    if not flatten:
        out = out.reshape(data.shape[:-1] + (weight.shape[0],))
    return out, mn, mx


def conv_int32_nchw(data, weight, bias32=None, stride=(1, 1), pad=(0, 0), dilate=(1, 1)):
    data = _c(data, np.int8)
    weight = _c(weight, np.int8)
    N, C, H, W = data.shape
    O, C2, KH, KW = weight.shape
    assert C == C2
    OH = (H + 2 * pad[0] - (dilate[0] * (KH - 1) + 1)) // stride[0] + 1
    OW = (W + 2 * pad[1] - (dilate[1] * (KW - 1) + 1)) // stride[1] + 1
    out = np.empty((N, O, OH, OW), np.int32)
    b = None
    if bias32 is not None:
        b = _c(bias32, np.int32)
    _lib.qref_conv_nchw(_ptr(data), _ptr(weight), _ptr(b) if b is not None else None, N, C, H,
                        W, O, KH, KW, stride[0], stride[1], pad[0], pad[1], dilate[0], dilate[1],
                        _ptr(out))
    return out


def quantized_conv(data, weight, bias, min_data, max_data, min_weight, max_weight,
                   min_bias=None, max_bias=None, stride=(1, 1), pad=(0, 0), dilate=(1, 1)):
    """_contrib_quantized_conv (NCHW) -> (int32 out, min_out, max_out)."""
    mn, mx = range_for_multiplication(min_data, max_data, min_weight, max_weight)
    b32 = None
    if bias is not None:
        b32 = bias_i8_to_i32(bias, mn, mx, min_bias, max_bias)
    return conv_int32_nchw(data, weight, b32, stride, pad, dilate), mn, mx


def relu_i8(q):
    q = _c(q, np.int8)
    out = np.empty_like(q)
    _lib.qref_relu_i8(_ptr(q), q.size, _ptr(out))
    return out


def pooling_output_hw(H, W, kernel, stride, pad, global_pool=False, convention="valid"):
    """Output extents of QuantizedPoolingShape (quantized_pooling.cc:82-121)."""
    if global_pool:
        return 1, 1
    out = []
    for size, k, s, p in ((H, kernel[0], stride[0], pad[0]), (W, kernel[1], stride[1], pad[1])):
        if k > size + 2 * p:
            raise ValueError("kernel size (%d) exceeds input (%d padded to %d)"
                             % (k, size, size + 2 * p))
        if convention == "valid":
            out.append(1 + (size + 2 * p - k) // s)
        elif convention == "full":
            # 1 + int(ceil(float(x) / s)) evaluated in binary32 as the reference does
            out.append(1 + int(np.ceil(np.float32(size + 2 * p - k) / np.float32(s))))
        else:
            raise ValueError("pooling_convention %r is not supported" % convention)
    return out[0], out[1]


def quantized_pooling(data, min_data, max_data, kernel=(1, 1), pool_type="max", stride=(1, 1),
                      pad=(0, 0), global_pool=False, convention="valid",
                      count_include_pad=True):
    """_contrib_quantized_pooling on NCHW int8/uint8 -> (out, min, max)."""
    if data.dtype not in (np.int8, np.uint8):
        raise TypeError("quantized_pooling takes int8 or uint8")
    if pool_type not in ("max", "avg"):
        raise ValueError("QuantizedPoolingOp only supports pool_type=max/avg for now")
    d = _c(data, data.dtype)
    N, C, H, W = d.shape
    if global_pool:
        kernel, stride, pad = (H, W), (1, 1), pad
    OH, OW = pooling_output_hw(H, W, kernel, stride, pad, global_pool, convention)
    out = np.empty((N, C, OH, OW), dtype=d.dtype)
    _lib.qref_pool_nchw(_ptr(d), int(d.dtype == np.uint8), N, C, H, W, kernel[0], kernel[1],
                        stride[0], stride[1], pad[0], pad[1], OH, OW, int(pool_type == "avg"),
                        int(bool(count_include_pad)), _ptr(out))
    return out, np.float32(min_data), np.float32(max_data)


def quantized_flatten(data, min_data, max_data):
    """_contrib_quantized_flatten (quantized_flatten-inl.h:39-110): a reshape to
    (d0, prod(rest)); the ranges pass through."""
    d = np.ascontiguousarray(data)
    return d.reshape(d.shape[0], -1).copy(), np.float32(min_data), np.float32(max_data)


def quantized_elemwise_add(lhs, rhs, lhs_min, lhs_max, rhs_min, rhs_max, min_calib_range=None,
                           max_calib_range=None):
    """_contrib_quantized_elemwise_add on operands of one shape -> (out, min, max); int32
    without calibration, else the inputs' type (int8 when they differ)
    (quantized_elemwise_add.cc:50-78)."""
    for x in (lhs, rhs):
        if x.dtype not in (np.int8, np.uint8):
            raise TypeError("quantized_elemwise_add takes int8 or uint8")
    if lhs.shape != rhs.shape:
        raise ValueError("operands must have one shape")
    a, b = _c(lhs, lhs.dtype), _c(rhs, rhs.dtype)
    calibrated = min_calib_range is not None and max_calib_range is not None
    if not calibrated:
        out_dtype, kind = np.int32, 0
    elif a.dtype == b.dtype:
        out_dtype, kind = a.dtype, (1 if a.dtype == np.int8 else 2)
    else:
        out_dtype, kind = np.int8, 1
    out = np.empty(a.shape, dtype=out_dtype)
    omin, omax = ctypes.c_float(), ctypes.c_float()
    _lib.qref_elemwise_add(_ptr(a), int(a.dtype == np.uint8), _ptr(b), int(b.dtype == np.uint8),
                           a.size, lhs_min, lhs_max, rhs_min, rhs_max, kind, int(calibrated),
                           min_calib_range if calibrated else 0.0,
                           max_calib_range if calibrated else 0.0, _ptr(out),
                           ctypes.byref(omin), ctypes.byref(omax))
    return out, np.float32(omin.value), np.float32(omax.value)


def quantized_npi_add(lhs, rhs, lhs_min, lhs_max, rhs_min, rhs_max, min_calib_range=None,
                      max_calib_range=None):
    """_contrib_quantized_npi_add -> (out, min, max): operands of one shape take the plain sum;
    others are stretched by numpy's rules and summed at their own scales
    (dnnl_quantized_elemwise_add.cc:183-257)."""
    if lhs.shape == rhs.shape:
        return quantized_elemwise_add(lhs, rhs, lhs_min, lhs_max, rhs_min, rhs_max,
                                      min_calib_range, max_calib_range)
    for x in (lhs, rhs):
        if x.dtype not in (np.int8, np.uint8):
            raise TypeError("quantized_npi_add takes int8 or uint8")
    a, b = np.broadcast_arrays(lhs, rhs)
    a, b = np.ascontiguousarray(a), np.ascontiguousarray(b)
    calibrated = min_calib_range is not None and max_calib_range is not None
    if not calibrated:
        out_dtype, kind = np.int32, 0
    elif a.dtype == b.dtype:
        out_dtype, kind = a.dtype, (1 if a.dtype == np.int8 else 2)
    else:
        out_dtype, kind = np.int8, 1
    out = np.empty(a.shape, dtype=out_dtype)
    omin, omax = ctypes.c_float(), ctypes.c_float()
    _lib.qref_broadcast_add(_ptr(a), int(a.dtype == np.uint8), _ptr(b), int(b.dtype == np.uint8),
                            a.size, lhs_min, lhs_max, rhs_min, rhs_max, kind, int(calibrated),
                            min_calib_range if calibrated else 0.0,
                            max_calib_range if calibrated else 0.0, _ptr(out),
                            ctypes.byref(omin), ctypes.byref(omax))
    return out, np.float32(omin.value), np.float32(omax.value)


def quantized_concat(arrays, mins, maxs, dim=1):
    """_contrib_quantized_concat -> (out, min, max): the output range is the hull of the
    input ranges and 0 (dnnl_quantized_concat.cc:53-67), the type int8 as soon as one
    input is int8 (quantized_concat.cc:83-103)."""
    if not arrays or len(arrays) != len(mins) or len(arrays) != len(maxs):
        raise ValueError("one range per input")
    for x in arrays:
        if x.dtype not in (np.int8, np.uint8):
            raise TypeError("quantized_concat takes int8 or uint8")
    out_dtype = np.int8 if any(x.dtype == np.int8 for x in arrays) else np.uint8
    omin, omax = np.float32(0.0), np.float32(0.0)
    for lo, hi in zip(mins, maxs):
        if np.float32(lo) < omin:
            omin = np.float32(lo)
        if np.float32(hi) > omax:
            omax = np.float32(hi)
    parts = []
    for x, lo, hi in zip(arrays, mins, maxs):
        x = _c(x, x.dtype)
        y = np.empty(x.shape, dtype=out_dtype)
        _lib.qref_concat_rescale(_ptr(x), int(x.dtype == np.uint8), x.size, lo, hi, omin, omax,
                                 int(out_dtype == np.uint8), _ptr(y))
        parts.append(y)
    return np.concatenate(parts, axis=dim), omin, omax


def quantized_elemwise_mul(lhs, rhs, lhs_min, lhs_max, rhs_min, rhs_max, min_calib_range=None,
                           max_calib_range=None, enable_float_output=False):
    """_contrib_quantized_elemwise_mul on int8 operands of one shape
    (quantized_elemwise_mul.cc:62-206): float32 output alone with enable_float_output, else
    (out, min, max) with out int8 when both calibration bounds are given and int32 when not."""
    if lhs.dtype != np.int8 or rhs.dtype != np.int8:
        raise TypeError("quantized_elemwise_mul takes int8")
    if lhs.shape != rhs.shape:
        raise ValueError("operands must have one shape")
    a, b = _c(lhs, np.int8), _c(rhs, np.int8)
    calibrated = min_calib_range is not None and max_calib_range is not None
    if enable_float_output:
        out_dtype, kind = np.float32, 2
    elif calibrated:
        out_dtype, kind = np.int8, 1
    else:
        out_dtype, kind = np.int32, 0
    out = np.empty(a.shape, dtype=out_dtype)
    omin, omax = ctypes.c_float(), ctypes.c_float()
    _lib.qref_elemwise_mul(_ptr(a), _ptr(b), a.size, lhs_min, lhs_max, rhs_min, rhs_max, kind,
                           min_calib_range if calibrated else 0.0,
                           max_calib_range if calibrated else 0.0, _ptr(out), ctypes.byref(omin),
                           ctypes.byref(omax))
    if enable_float_output:
        return out
    return out, np.float32(omin.value), np.float32(omax.value)


def quantized_embedding(data, weight, min_weight, max_weight):
    """_contrib_quantized_embedding -> (out, min, max): rows of the int8 table taken at
    int64(data) clipped to [0, input_dim - 1] (indexing_op.cc:44-58), the table's range
    passed through (quantized_indexing_op.cc:118-121)."""
    if weight.dtype != np.int8 or weight.ndim != 2:
        raise TypeError("the table is a 2-D int8 array")
    idx = np.asarray(data)
    with np.errstate(invalid="ignore"):
        j = np.trunc(idx).astype(np.int64) if idx.dtype.kind == "f" else idx.astype(np.int64)
    j = np.clip(j, 0, weight.shape[0] - 1)
    return weight[j.reshape(-1)].reshape(idx.shape + (weight.shape[1],)).copy(), \
        np.float32(min_weight), np.float32(max_weight)


def quantized_reshape(data, min_data, max_data, shape):
    """_contrib_quantized_reshape (quantized_reshape.cc:31-46): the data under another
    shape, the range passed through.  `shape` is the inferred output shape."""
    return np.ascontiguousarray(data).reshape(shape).copy(), np.float32(min_data), \
        np.float32(max_data)


def quantized_transpose(data, min_data, max_data, axes=None):
    """_contrib_quantized_transpose (quantized_transpose.cc:49-104): numpy's transpose, the
    range passed through."""
    return np.array(np.transpose(data, axes), order="C", copy=True), np.float32(min_data), \
        np.float32(max_data)


def quantize_asym(data, min_calib_range=None, max_calib_range=None):
    """_contrib_quantize_asym -> (out uint8, scale, shift) (quantize_asym-inl.h:78-160)."""
    d = np.ascontiguousarray(data)
    if d.dtype == np.uint8:
        return d.copy(), np.float32(1.0), np.float32(0.0)
    if d.dtype == np.int8:
        return (d.astype(np.int16) + 128).astype(np.uint8), np.float32(1.0), np.float32(128.0)
    if d.dtype != np.float32:
        raise TypeError("quantize_asym takes float32, int8 or uint8")
    if min_calib_range is None or max_calib_range is None:
        min_calib_range, max_calib_range = minmax_f32(d)
    out = np.empty(d.shape, dtype=np.uint8)
    scale, shift = ctypes.c_float(), ctypes.c_float()
    _lib.qref_quantize_asym(_ptr(d), d.size, min_calib_range, max_calib_range, _ptr(out),
                            ctypes.byref(scale), ctypes.byref(shift))
    return out, np.float32(scale.value), np.float32(shift.value)


def quantized_batch_norm(data, gamma, beta, moving_mean, moving_var, min_data, max_data,
                         min_calib_range, max_calib_range, eps=1e-3, axis=1, relu=False):
    """_contrib_quantized_batch_norm / _relu -> (out int8, min, max); the output range is the
    calibrated one, which the operator requires (dnnl_quantized_batch_norm.cc:76-85)."""
    if data.dtype not in (np.int8, np.uint8):
        raise TypeError("quantized_batch_norm takes int8 or uint8 data")
    if min_calib_range is None or max_calib_range is None:
        raise ValueError("min_calib_range or max_calib_range is not available")
    d = np.ascontiguousarray(data)
    axis = axis + d.ndim if axis < 0 else axis
    channels = d.shape[axis]
    outer = int(np.prod(d.shape[:axis], dtype=np.int64))
    inner = int(np.prod(d.shape[axis + 1:], dtype=np.int64))
    vec = [_c(v, np.float32) for v in (gamma, beta, moving_mean, moving_var)]
    for v in vec:
        if v.shape != (channels,):
            raise ValueError("per-channel parameters must have shape (%d,)" % channels)
    out = np.empty(d.shape, dtype=np.int8)
    omin, omax = ctypes.c_float(), ctypes.c_float()
    _lib.qref_batch_norm(_ptr(d), int(d.dtype == np.uint8), outer, channels, inner, _ptr(vec[0]),
                         _ptr(vec[1]), _ptr(vec[2]), _ptr(vec[3]), min_data, max_data,
                         float(eps), min_calib_range, max_calib_range, int(relu), _ptr(out),
                         ctypes.byref(omin), ctypes.byref(omax))
    return out, np.float32(omin.value), np.float32(omax.value)
