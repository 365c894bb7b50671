"""mxnet_amd: MI355X (gfx950) implementation of MXNet's INT8 quantized-inference
operators (_contrib_quantize_v2, _contrib_requantize, _contrib_dequantize,
_contrib_quantized_fully_connected, _contrib_quantized_conv).

The compute lives in libmxq_hip.so (hand-written HIP behind a C ABI, declared in
include/mxq.h).  This package is the host-side mirror of the reference operator
interface; torch is used only to own device memory and streams."""
from . import _lib  # noqa: F401  (fails loudly if the HIP library is missing)
from . import capi  # noqa: F401
from . import operator  # noqa: F401  (loads the C++ operator host, libmxq_ops.so)
from . import contrib  # noqa: F401

__all__ = ["capi", "operator", "contrib"]
