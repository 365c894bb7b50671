"""`mx.nd.save` / `mx.nd.load` and the symbolic checkpoint helpers over the reference's
NDArray list format (python/mxnet/ndarray/utils.py:149-273, python/mxnet/model.py:
save_checkpoint / load_checkpoint; the bytes are src/ndarray/ndarray.cc:1856-2146, read
and written by libmxq_ops.so).  Arrays are torch CPU tensors."""
import ctypes

import numpy as np
import torch

from . import operator as _operator
from .operator import Blob
from .symbol import Symbol

# mshadow type flag <-> numpy dtype (bfloat16, flag 12, has no numpy dtype: torch only)
_NP_OF_FLAG = {0: np.float32, 1: np.float64, 2: np.float16, 3: np.uint8, 4: np.int32, 5: np.int8,
               6: np.int64, 7: np.bool_, 8: np.int16, 9: np.uint16, 10: np.uint32, 11: np.uint64}
_FLAG_OF_TORCH = {torch.float32: 0, torch.float64: 1, torch.float16: 2, torch.uint8: 3,
                  torch.int32: 4, torch.int8: 5, torch.int64: 6, torch.bool: 7, torch.int16: 8,
                  torch.bfloat16: 12}


def load(fname):
    """dict name -> tensor when the file carries names, else a list (empty NDArrays come
    back as None)."""
    handle, count, has_names = ctypes.c_void_p(), ctypes.c_int(), ctypes.c_int()
    _operator._check(_operator.ops.mxq_ndlist_load(fname.encode(), ctypes.byref(handle),
                                                   ctypes.byref(count), ctypes.byref(has_names)))
    try:
        arrays, names = [], []
        for i in range(count.value):
            name, none, dtype, ndim = (ctypes.c_char_p(), ctypes.c_int(), ctypes.c_int(),
                                       ctypes.c_int())
            shape = ctypes.POINTER(ctypes.c_int64)()
            data, nbytes = ctypes.c_void_p(), ctypes.c_size_t()
            _operator._check(_operator.ops.mxq_ndlist_get(
                handle, i, ctypes.byref(name), ctypes.byref(none), ctypes.byref(dtype),
                ctypes.byref(ndim), ctypes.byref(shape), ctypes.byref(data),
                ctypes.byref(nbytes)))
            names.append(name.value.decode())
            if none.value:
                arrays.append(None)
                continue
            dims = tuple(shape[d] for d in range(ndim.value))
            raw = ctypes.string_at(data, nbytes.value) if nbytes.value else b""
            if dtype.value == 12:
                t = torch.frombuffer(bytearray(raw), dtype=torch.bfloat16).reshape(dims) \
                    if raw else torch.empty(dims, dtype=torch.bfloat16)
            else:
                a = np.frombuffer(raw, dtype=_NP_OF_FLAG[dtype.value]).reshape(dims).copy()
                if a.dtype in (np.uint16, np.uint32, np.uint64):
                    a = a.astype(np.int64)  # torch has no unsigned types beyond uint8
                t = torch.from_numpy(a)
            arrays.append(t)
    finally:
        _operator.ops.mxq_ndlist_free(handle)
    return dict(zip(names, arrays)) if has_names.value else arrays


def save(fname, data, np_shape=False):
    """data: a tensor, a list of tensors or a dict name -> tensor (mx.nd.save).  np_shape
    writes the records `npx.save` / Gluon's save_parameters write (zero-dimensional and
    zero-size arrays allowed)."""
    if isinstance(data, torch.Tensor):
        data = [data]
    names = None
    if isinstance(data, dict):
        names = list(data.keys())
        data = list(data.values())
    tensors = [(t if isinstance(t, torch.Tensor) else torch.as_tensor(t)).detach().cpu()
               .contiguous() for t in data]
    blobs = (Blob * len(tensors))()
    for b, t in zip(blobs, tensors):
        if t.dtype not in _FLAG_OF_TORCH:
            raise TypeError("cannot save dtype %s" % t.dtype)
        if t.dim() > 8:
            raise ValueError("at most 8 dimensions")
        b.data = t.data_ptr()
        b.ndim = t.dim()
        for d, x in enumerate(t.shape):
            b.shape[d] = x
        b.dtype = _FLAG_OF_TORCH[t.dtype]
    cnames = (ctypes.c_char_p * len(tensors))(*[n.encode() for n in names]) if names is not None \
        else None
    _operator._check(_operator.ops.mxq_ndlist_save(fname.encode(), len(tensors), cnames, blobs,
                                                   int(bool(np_shape))))


def save_checkpoint(prefix, epoch, symbol, arg_params, aux_params):
    """`prefix-symbol.json` + `prefix-%04d.params` with `arg:` / `aux:` key prefixes."""
    if symbol is not None:
        with open("%s-symbol.json" % prefix, "w") as f:
            f.write(symbol.tojson())
    save_dict = {("arg:%s" % k): v for k, v in arg_params.items()}
    save_dict.update({("aux:%s" % k): v for k, v in aux_params.items()})
    save("%s-%04d.params" % (prefix, epoch), save_dict)


def load_params(prefix, epoch):
    arg_params, aux_params = {}, {}
    for k, v in load("%s-%04d.params" % (prefix, epoch)).items():
        tp, name = k.split(":", 1)
        if tp == "arg":
            arg_params[name] = v
        elif tp == "aux":
            aux_params[name] = v
    return arg_params, aux_params


def load_checkpoint(prefix, epoch):
    with open("%s-symbol.json" % prefix) as f:
        symbol = Symbol.fromjson(f.read())
    arg_params, aux_params = load_params(prefix, epoch)
    return symbol, arg_params, aux_params
