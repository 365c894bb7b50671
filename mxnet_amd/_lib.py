"""ctypes binding of libmxq_hip.so.  There is no fallback: if the library is
missing or a symbol is absent the import raises."""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libmxq_hip.so")

# element type codes = mshadow::TypeFlag
FLOAT32, UINT8, INT32, INT8 = 0, 3, 4, 5


class MXQError(RuntimeError):
    """A C-ABI call returned non-zero; carries mxq_last_error()."""


if not os.path.exists(LIB_PATH):
    raise ImportError(
        "libmxq_hip.so is not built: run `python -c 'import __graft_entry__ as g; g.build()'` "
        "(or python mxnet_amd/build.py) first; there is no CPU fallback")

lib = ctypes.CDLL(LIB_PATH)

_p = ctypes.c_void_p
_sz = ctypes.c_size_t
_i = ctypes.c_int
_f = ctypes.c_float

# every symbol include/mxq.h declares, with its signature
SIGNATURES = {
    "mxq_last_error": (ctypes.c_char_p, []),
    "mxq_abi_version": (_i, []),
    "mxq_quantize_v2_workspace": (_sz, [_sz]),
    "mxq_quantize_v2": (_i, [_p, _p, _p, _p, _p, _sz, _i, _i, _f, _f, _p, _sz]),
    "mxq_quantize_v2_noalloc": (_i, [_p, _p, _p, _p, _p, _sz, _i, _i, _f, _f]),
    "mxq_quantize": (_i, [_p, _p, _p, _p, _p, _p, _p, _sz, _i]),
    "mxq_quantize_v2_passthrough": (_i, [_p, _p, _p, _p, _p, _sz, _i, _i, _f, _f]),
    "mxq_requantize_workspace": (_sz, [_sz]),
    "mxq_requantize": (_i, [_p, _p, _p, _p, _p, _p, _p, _sz, _i, _f, _f, _p, _sz]),
    "mxq_dequantize": (_i, [_p, _p, _i, _p, _p, _p, _sz]),
    "mxq_quantized_relu": (_i, [_p, _p, _p, _p, _p, _p, _p, _sz]),
    "mxq_quantized_pooling_nchw": (_i, [_p, _p, _i] + [_i] * 12 + [_i, _i, _p, _p, _p, _p, _p]),
    "mxq_quantized_flatten": (_i, [_p, _p, _p, _p, _p, _p, _p, _sz]),
    "mxq_quantized_elemwise_add": (_i, [_p, _p, _i, _p, _i, _p, _p, _p, _p, _p, _i, _p, _p, _sz,
                                        _i, _f, _f]),
    "mxq_quantized_broadcast_add": (_i, [_p, _p, _i, _i, _p, _p, _i, _i, _p, _p, _p, _p, _p, _p,
                                         _i, _p, _p, _i, _f, _f]),
    "mxq_quantized_elemwise_mul": (_i, [_p, _p, _p, _p, _p, _p, _p, _p, _i, _p, _p, _sz, _i, _f,
                                        _f]),
    "mxq_quantized_embedding": (_i, [_p, _p, _i, _p, _p, _p, _p, _p, _p, _sz, ctypes.c_int64,
                                     ctypes.c_int64]),
    "mxq_quantized_transpose": (_i, [_p, _p, _p, _p, _p, _p, _p, _i, _p, _p]),
    "mxq_quantize_asym_workspace": (_sz, [_sz]),
    "mxq_quantize_asym": (_i, [_p, _p, _i, _p, _p, _p, _sz, _i, _f, _f, _p, _sz]),
    "mxq_quantized_batch_norm_workspace": (_sz, [ctypes.c_int64]),
    "mxq_quantized_batch_norm": (_i, [_p, _p, _i] + [_p] * 6 + [_p, _p, _p] +
                                 [ctypes.c_int64] * 3 + [ctypes.c_double, _f, _f, _i, _p, _sz]),
    "mxq_quantized_concat": (_i, [_p, _i, _p, _p, _p, _p, _p, ctypes.c_int64, ctypes.c_int64, _p,
                                  _i, _p, _p]),
    "mxq_quantized_fc_workspace": (_sz, [_i, _i, _i, _i]),
    "mxq_quantized_fc": (_i, [_p, _p, _p, _p, _i, _i, _i] + [_p] * 6 + [_p, _p, _p, _p, _p, _p,
                              _i, _f, _f, _p, _sz]),
    "mxq_quantized_fc_f32": (_i, [_p, _p, _p, _p, _i, _i, _i] + [_p] * 6 + [_p, _p, _p, _p, _p,
                                  _i, _f, _f, _p, _sz]),
    "mxq_quantized_fc_sum": (_i, [_p, _p, _p, _p, _i, _i, _i] + [_p] * 6 + [_p, _p, _p] +
                             [_p, _p, _p, _p, _p, _f, _f, _f, _f, _i, _p, _sz]),
    "mxq_quantized_conv_workspace": (_sz, [_i] * 14),
    "mxq_quantized_conv_nhwc": (_i, [_p, _p, _p, _p] + [_i] * 13 + [_p] * 6 +
                                [_p, _p, _p, _p, _p, _p, _i, _f, _f, _p, _sz]),
    "mxq_quantized_conv_nhwc_out_nchw": (_i, [_p, _p, _p, _p] + [_i] * 13 + [_p] * 6 +
                                         [_p, _p, _p, _p, _sz]),
    "mxq_quantized_conv_nchw_workspace": (_sz, [_i] * 14),
    "mxq_quantized_conv_nchw": (_i, [_p, _p, _p, _p] + [_i] * 13 + [_p] * 6 +
                                [_p, _p, _p, _p, _sz]),
    "mxq_nchw_to_nhwc_i8": (_i, [_p, _p, _p, _i, _i, _i, _i]),
    "mxq_nchw_to_nhwc_pad_i8": (_i, [_p, _p, _p, _i, _i, _i, _i, _i]),
    "mxq_nchw_to_s2d_nhwc_i8": (_i, [_p, _p, _p, _i, _i, _i, _i, _i, _i, _i]),
    "mxq_nhwc_to_nchw": (_i, [_p, _p, _p, _i, _i, _i, _i, _i]),
}

for _name, (_res, _args) in SIGNATURES.items():
    _fn = getattr(lib, _name)  # AttributeError if the library lacks the symbol
    _fn.restype = _res
    _fn.argtypes = _args

# test-only twins of the FC and convolution entry points (tests/mxq_test_hooks.h, not part
# of include/mxq.h): the same arguments followed by the tile configuration, the split-K
# factor and, for the FC, the streaming kernel's work-groups per CU (0 = choose)
TEST_HOOKS = {
    "mxq_test_quantized_fc": (_i, SIGNATURES["mxq_quantized_fc"][1] + [_i, _i, _i]),
    "mxq_test_quantized_fc_sum": (_i, SIGNATURES["mxq_quantized_fc_sum"][1] + [_i, _i, _i]),
    "mxq_test_quantized_fc_f32": (_i, SIGNATURES["mxq_quantized_fc_f32"][1] + [_i, _i]),
    "mxq_test_quantized_conv_nhwc": (_i, SIGNATURES["mxq_quantized_conv_nhwc"][1] + [_i, _i]),
    "mxq_test_quantized_conv_nchw": (_i, SIGNATURES["mxq_quantized_conv_nchw"][1] + [_i]),
}
for _name, (_res, _args) in TEST_HOOKS.items():
    _fn = getattr(lib, _name)
    _fn.restype = _res
    _fn.argtypes = _args


def last_error():
    return lib.mxq_last_error().decode()


def check(rc):
    if rc != 0:
        raise MXQError(last_error())
