"""The reference's imperative operator names: `mxnet_amd.contrib.quantize_v2(...)`
reads like `mx.nd.contrib.quantize_v2(...)` (and the `_npx_*` aliases like
`mx.npx.requantize`).  Same positional tensors, same keyword attributes, same
outputs; everything runs through the C++ operator host."""
from .operator import invoke


def quantize(data, min_range, max_range, out_type="uint8"):
    return invoke("_contrib_quantize", data, min_range, max_range, out_type=out_type)


def quantize_v2(data, out_type="int8", min_calib_range=None, max_calib_range=None):
    return invoke("_contrib_quantize_v2", data, out_type=out_type,
                  min_calib_range=min_calib_range, max_calib_range=max_calib_range)


def requantize(data, min_range, max_range, out_type="int8", min_calib_range=None,
               max_calib_range=None):
    return invoke("_contrib_requantize", data, min_range, max_range, out_type=out_type,
                  min_calib_range=min_calib_range, max_calib_range=max_calib_range)


def dequantize(data, min_range, max_range, out_type="float32"):
    return invoke("_contrib_dequantize", data, min_range, max_range, out_type=out_type)


def quantized_fully_connected(data, weight, bias=None, min_data=None, max_data=None,
                              min_weight=None, max_weight=None, min_bias=None, max_bias=None,
                              num_hidden=None, no_bias=False, flatten=True):
    ins = [data, weight] + ([] if no_bias else [bias]) + [min_data, max_data, min_weight,
                                                          max_weight]
    if not no_bias:
        ins += [min_bias, max_bias]
    return invoke("_contrib_quantized_fully_connected", *ins, num_hidden=num_hidden,
                  no_bias=no_bias, flatten=flatten)


def quantized_conv(data, weight, bias=None, min_data=None, max_data=None, min_weight=None,
                   max_weight=None, min_bias=None, max_bias=None, kernel=None, stride=None,
                   dilate=None, pad=None, num_filter=None, num_group=1, no_bias=False,
                   layout=None):
    ins = [data, weight] + ([] if no_bias else [bias]) + [min_data, max_data, min_weight,
                                                          max_weight]
    if not no_bias:
        ins += [min_bias, max_bias]
    return invoke("_contrib_quantized_conv", *ins, kernel=kernel, stride=stride, dilate=dilate,
                  pad=pad, num_filter=num_filter, num_group=num_group, no_bias=no_bias,
                  layout=layout)


def quantized_act(data, min_data, max_data, act_type="relu"):
    return invoke("_contrib_quantized_act", data, min_data, max_data, act_type=act_type)


def quantized_pooling(data, min_data, max_data, kernel=None, pool_type="max", global_pool=False,
                      cudnn_off=False, pooling_convention="valid", stride=None, pad=None,
                      count_include_pad=None, layout=None):
    attrs = {"pool_type": pool_type, "global_pool": global_pool, "cudnn_off": cudnn_off,
             "pooling_convention": pooling_convention}
    for key, value in (("kernel", kernel), ("stride", stride), ("pad", pad),
                       ("count_include_pad", count_include_pad), ("layout", layout)):
        if value is not None:
            attrs[key] = value
    return invoke("_contrib_quantized_pooling", data, min_data, max_data, **attrs)


def quantized_flatten(data, min_data, max_data):
    return invoke("_contrib_quantized_flatten", data, min_data, max_data)


def quantized_elemwise_add(lhs, rhs, lhs_min, lhs_max, rhs_min, rhs_max, min_calib_range=None,
                           max_calib_range=None):
    return invoke("_contrib_quantized_elemwise_add", lhs, rhs, lhs_min, lhs_max, rhs_min,
                  rhs_max, min_calib_range=min_calib_range, max_calib_range=max_calib_range)


def quantized_npi_add(lhs, rhs, lhs_min, lhs_max, rhs_min, rhs_max, min_calib_range=None,
                      max_calib_range=None):
    """_contrib_quantized_npi_add: the quantized sum under numpy broadcasting."""
    return invoke("_contrib_quantized_npi_add", lhs, rhs, lhs_min, lhs_max, rhs_min, rhs_max,
                  min_calib_range=min_calib_range, max_calib_range=max_calib_range)


def quantized_concat(*data, num_args=None, dim=1):
    """`data` is arg0..argN-1 followed by (arg0_min, arg0_max, ..., argN-1_min, argN-1_max)."""
    if num_args is None:
        num_args = len(data) // 3
    return invoke("_contrib_quantized_concat", *data, num_args=num_args, dim=dim)


def quantized_elemwise_mul(lhs, rhs, lhs_min, lhs_max, rhs_min, rhs_max, min_calib_range=None,
                           max_calib_range=None, enable_float_output=False):
    return invoke("_contrib_quantized_elemwise_mul", lhs, rhs, lhs_min, lhs_max, rhs_min,
                  rhs_max, min_calib_range=min_calib_range, max_calib_range=max_calib_range,
                  enable_float_output=enable_float_output)


def quantized_embedding(data, weight, min_weight, max_weight, input_dim=None, output_dim=None,
                        dtype="float32", sparse_grad=False):
    return invoke("_contrib_quantized_embedding", data, weight, min_weight, max_weight,
                  input_dim=input_dim, output_dim=output_dim, dtype=dtype,
                  sparse_grad=sparse_grad)


def quantized_reshape(data, min_data, max_data, shape=(), reverse=False):
    return invoke("_contrib_quantized_reshape", data, min_data, max_data, shape=shape,
                  reverse=reverse)


def quantized_transpose(data, min_data, max_data, axes=()):
    return invoke("_contrib_quantized_transpose", data, min_data, max_data, axes=axes)


def npx_quantized_reshape(data, min_data, max_data, newshape, reverse=False, order="C"):
    """_npx_quantized_reshape: numpy-namespace reshape, newshape with -1 ... -6."""
    return invoke("_npx_quantized_reshape", data, min_data, max_data, newshape=newshape,
                  reverse=reverse, order=order)


def npx_quantized_transpose(data, min_data, max_data, axes=None):
    """_npx_quantized_transpose: axes None reverses; negative axes count from the end."""
    return invoke("_npx_quantized_transpose", data, min_data, max_data, axes=axes)


def quantize_asym(data, min_calib_range=None, max_calib_range=None):
    return invoke("_contrib_quantize_asym", data, min_calib_range=min_calib_range,
                  max_calib_range=max_calib_range)


def quantized_batch_norm(data, gamma, beta, moving_mean, moving_var, min_data, max_data,
                         eps=1e-3, momentum=0.9, fix_gamma=True, use_global_stats=False,
                         axis=1, min_calib_range=None, max_calib_range=None, relu=False):
    """_contrib_quantized_batch_norm, or _contrib_quantized_batch_norm_relu with relu=True."""
    return invoke("_contrib_quantized_batch_norm_relu" if relu else
                  "_contrib_quantized_batch_norm", data, gamma, beta, moving_mean, moving_var,
                  min_data, max_data, eps=eps, momentum=momentum, fix_gamma=fix_gamma,
                  use_global_stats=use_global_stats, axis=axis, min_calib_range=min_calib_range,
                  max_calib_range=max_calib_range)
