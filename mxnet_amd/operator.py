"""Imperative operator invocation through the C++ operator host (libmxq_ops.so):
the registry with the reference's operator names, attribute parsing, shape/type
inference and FCompute<gpu>.  `invoke()` does what `mx.nd.contrib.<op>(...)` does
in MXNet: attributes are stringified into the node dict exactly as MXNet's frontend
does, outputs are allocated from the inferred shapes/types, the registered gpu
function runs on the current stream.  Torch only owns the device memory."""
import ctypes
import os

import torch

from . import _lib  # loads libmxq_hip.so first (libmxq_ops.so links against it)

_HERE = os.path.dirname(os.path.abspath(__file__))
OPS_LIB_PATH = os.path.join(_HERE, "libmxq_ops.so")
if not os.path.exists(OPS_LIB_PATH):
    raise ImportError("libmxq_ops.so is not built: run __graft_entry__.build() first")

MAX_NDIM = 8


class Blob(ctypes.Structure):
    _fields_ = [("data", ctypes.c_void_p), ("ndim", ctypes.c_int),
                ("shape", ctypes.c_int64 * MAX_NDIM), ("dtype", ctypes.c_int)]


ops = ctypes.CDLL(OPS_LIB_PATH)
_p, _i, _sz = ctypes.c_void_p, ctypes.c_int, ctypes.c_size_t
_pi = ctypes.POINTER(ctypes.c_int)
_pl = ctypes.POINTER(ctypes.c_int64)
_pb = ctypes.POINTER(Blob)
_pps = ctypes.POINTER(ctypes.c_char_p)
OPS_SIGNATURES = {
    "mxq_ops_last_error": (ctypes.c_char_p, []),
    "mxq_op_count": (_i, []),
    "mxq_op_name": (ctypes.c_char_p, [_i]),
    "mxq_op_has_attr": (_i, [ctypes.c_char_p, ctypes.c_char_p]),
    "mxq_node_create": (_i, [ctypes.c_char_p, ctypes.c_char_p, _i, _pps, _pps,
                             ctypes.POINTER(_p)]),
    "mxq_node_free": (_i, [_p]),
    "mxq_node_num_inputs": (_i, [_p, _pi]),
    "mxq_node_num_outputs": (_i, [_p, _pi]),
    "mxq_node_input_names": (_i, [_p, _pps]),
    "mxq_node_output_names": (_i, [_p, _pps]),
    "mxq_node_gradient_names": (_i, [_p, _pps]),
    "mxq_node_infer_shape": (_i, [_p, _i, _pi, _pl, _i, _pi, _pl]),
    "mxq_node_infer_type": (_i, [_p, _i, _pi, _i, _pi]),
    "mxq_node_temp_bytes": (_i, [_p, _i, _pb, _i, _pb, ctypes.POINTER(_sz)]),
    "mxq_node_forward": (_i, [_p, _p, _i, _i, _pb, _i, _pb, _p, _sz]),
    "mxq_quantize_symbol": (_i, [ctypes.c_char_p, _i, _i, _pps, _i, _pps, _i, _pps,
                                 ctypes.c_char_p, ctypes.c_char_p, ctypes.c_char_p, _pps, _pi,
                                 ctypes.POINTER(_pps)]),
    "mxq_set_calib_table": (_i, [ctypes.c_char_p, _i, _pps, ctypes.POINTER(ctypes.c_float),
                                 ctypes.POINTER(ctypes.c_float), _pps]),
    "mxq_symbol_normalize": (_i, [ctypes.c_char_p, _pps]),
    "mxq_ndlist_load": (_i, [ctypes.c_char_p, ctypes.POINTER(_p), _pi, _pi]),
    "mxq_ndlist_get": (_i, [_p, _i, _pps, _pi, _pi, _pi, ctypes.POINTER(_pl),
                            ctypes.POINTER(_p), ctypes.POINTER(_sz)]),
    "mxq_ndlist_free": (_i, [_p]),
    "mxq_ndlist_save": (_i, [ctypes.c_char_p, _i, _pps, _pb, _i]),
    "mxq_calibrate_entropy": (_i, [ctypes.POINTER(ctypes.c_float), ctypes.POINTER(ctypes.c_float),
                                   _sz, _i, ctypes.POINTER(ctypes.c_float),
                                   ctypes.POINTER(ctypes.c_float)]),
}
for _name, (_res, _args) in OPS_SIGNATURES.items():
    _fn = getattr(ops, _name)
    _fn.restype = _res
    _fn.argtypes = _args

# mshadow::TypeFlag <-> torch dtype
_FLAG_OF = {torch.float32: 0, torch.float64: 1, torch.float16: 2, torch.uint8: 3,
            torch.int32: 4, torch.int8: 5, torch.int64: 6, torch.bool: 7, torch.bfloat16: 12}
_DTYPE_OF = {v: k for k, v in _FLAG_OF.items()}


class MXNetError(RuntimeError):
    """What MXNet raises when an operator's CHECK fails (dmlc::Error)."""


def _check(rc):
    if rc != 0:
        raise MXNetError(ops.mxq_ops_last_error().decode())


def list_operators():
    return [ops.mxq_op_name(i).decode() for i in range(ops.mxq_op_count())]


def has_attr(op, key):
    return bool(ops.mxq_op_has_attr(op.encode(), key.encode()))


def _attr_str(v):
    """Python value -> the string MXNet's frontend puts in the node dict."""
    if v is None:
        return "None"
    if isinstance(v, bool):
        return "True" if v else "False"
    if isinstance(v, (tuple, list)):
        return "(" + ", ".join(str(int(x)) for x in v) + ("," if len(v) == 1 else "") + ")"
    if isinstance(v, float):
        return repr(v)
    return str(v)


class Node:
    """One operator node: op + attribute dict (nnvm::NodeAttrs) and, for stateful
    operators, its OpStatePtr."""

    def __init__(self, op, name="", **attrs):
        self.op = op
        self.attrs = {k: _attr_str(v) for k, v in attrs.items()}
        keys = (ctypes.c_char_p * len(self.attrs))(*[k.encode() for k in self.attrs])
        vals = (ctypes.c_char_p * len(self.attrs))(*[v.encode() for v in self.attrs.values()])
        h = _p()
        _check(ops.mxq_node_create(op.encode(), name.encode(), len(self.attrs), keys, vals,
                                   ctypes.byref(h)))
        self._h = h

    def __del__(self):
        h = getattr(self, "_h", None)
        if h and ops is not None:
            ops.mxq_node_free(h)
            self._h = None

    @property
    def num_inputs(self):
        n = _i()
        _check(ops.mxq_node_num_inputs(self._h, ctypes.byref(n)))
        return n.value

    @property
    def num_outputs(self):
        n = _i()
        _check(ops.mxq_node_num_outputs(self._h, ctypes.byref(n)))
        return n.value

    def list_inputs(self):
        s = ctypes.c_char_p()
        _check(ops.mxq_node_input_names(self._h, ctypes.byref(s)))
        return s.value.decode().split(",") if s.value else []

    def list_outputs(self):
        s = ctypes.c_char_p()
        _check(ops.mxq_node_output_names(self._h, ctypes.byref(s)))
        return s.value.decode().split(",") if s.value else []

    def gradient_nodes(self):
        """(operator, node name) of the gradient node FGradient makes for every input."""
        s = ctypes.c_char_p()
        _check(ops.mxq_node_gradient_names(self._h, ctypes.byref(s)))
        return [tuple(x.split(":", 1)) for x in s.value.decode().split(",")] if s.value else []

    def infer_shape(self, in_shapes, out_shapes=None):
        """Shapes are tuples or None (unknown).  Returns (in_shapes, out_shapes)."""
        nin, nout = len(in_shapes), self.num_outputs
        out_shapes = out_shapes or [None] * nout

        def pack(shapes):
            nd = (ctypes.c_int * len(shapes))()
            dims = (ctypes.c_int64 * (len(shapes) * MAX_NDIM))()
            for i, s in enumerate(shapes):
                if s is None:
                    nd[i] = -1
                else:
                    nd[i] = len(s)
                    for d, x in enumerate(s):
                        dims[i * MAX_NDIM + d] = x
            return nd, dims

        def unpack(nd, dims, n):
            return [None if nd[i] < 0 else tuple(dims[i * MAX_NDIM + d] for d in range(nd[i]))
                    for i in range(n)]

        ind, idims = pack(in_shapes)
        ond, odims = pack(out_shapes)
        _check(ops.mxq_node_infer_shape(self._h, nin, ind, idims, nout, ond, odims))
        return unpack(ind, idims, nin), unpack(ond, odims, nout)

    def infer_type(self, in_types, out_types=None):
        """Types are torch dtypes or None.  Returns (in_types, out_types)."""
        nin, nout = len(in_types), self.num_outputs
        out_types = out_types or [None] * nout
        it = (ctypes.c_int * nin)(*[-1 if t is None else _FLAG_OF[t] for t in in_types])
        ot = (ctypes.c_int * nout)(*[-1 if t is None else _FLAG_OF[t] for t in out_types])
        _check(ops.mxq_node_infer_type(self._h, nin, it, nout, ot))
        return ([None if x < 0 else _DTYPE_OF[x] for x in it],
                [None if x < 0 else _DTYPE_OF[x] for x in ot])

    def __call__(self, *inputs):
        inputs = [x for x in inputs if x is not None]
        if len(inputs) != self.num_inputs:
            raise MXNetError("%s expects %d inputs %s, got %d" % (
                self.op, self.num_inputs, self.list_inputs(), len(inputs)))
        for x in inputs:
            if not (x.is_cuda and x.is_contiguous()):
                raise MXNetError("inputs must be contiguous device tensors")
        dev = inputs[0].device
        _, out_shapes = self.infer_shape([tuple(x.shape) for x in inputs])
        _, out_types = self.infer_type([x.dtype for x in inputs])
        outputs = [torch.empty(s, dtype=t, device=dev) for s, t in zip(out_shapes, out_types)]

        def blobs(ts):
            arr = (Blob * len(ts))()
            for b, t in zip(arr, ts):
                b.data = t.data_ptr()
                b.ndim = t.dim()
                for d, x in enumerate(t.shape):
                    b.shape[d] = x
                b.dtype = _FLAG_OF[t.dtype]
            return arr

        bi, bo = blobs(inputs), blobs(outputs)
        nbytes = _sz()
        _check(ops.mxq_node_temp_bytes(self._h, len(inputs), bi, len(outputs), bo,
                                       ctypes.byref(nbytes)))
        temp = None
        if nbytes.value:
            temp = torch.empty(nbytes.value, dtype=torch.uint8, device=dev)
        stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
        _check(ops.mxq_node_forward(self._h, stream, dev.index or 0, len(inputs), bi,
                                    len(outputs), bo,
                                    ctypes.c_void_p(temp.data_ptr()) if temp is not None else None,
                                    nbytes.value))
        return outputs[0] if len(outputs) == 1 else tuple(outputs)


def invoke(op, *inputs, **attrs):
    """mx.nd.contrib-style call: tensors positionally, attributes by keyword."""
    attrs = {k: v for k, v in attrs.items() if v is not None}
    return Node(op, **attrs)(*inputs)
