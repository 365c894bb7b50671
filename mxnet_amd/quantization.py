"""Model quantization driver: the counterpart of `mxnet.contrib.quantization`
(python/mxnet/contrib/quantization.py) for symbols held as JSON.

Same functions, arguments and naming conventions:
  _quantize_symbol              :105-176   -> mxq_quantize_symbol (QuantizeGraph pass)
  _calibrate_quantized_sym      :339-361   -> mxq_set_calib_table
  _quantize_params              :50-102    offline int8 weights/biases via _contrib_quantize
  CalibrationCollector, _LayerOutputMinMaxCollector (:311-336),
  _LayerHistogramCollector      :210-308   entropy thresholds via mxq_calibrate_entropy
  quantize_model                :423-568   symbol + params in, calibrated int8 symbol + params out
The float network that calibration observes runs through `executor.Executor`.
"""
import ctypes

import numpy as np
import torch

from . import operator as _operator
from .executor import Executor
from .symbol import Symbol

_DEV_TYPE = {"cpu": 1, "gpu": 2}


def _c_strs(strings):
    return (ctypes.c_char_p * len(strings))(*[s.encode() for s in strings])


def _quantize_symbol(sym, device="gpu", excluded_symbols=None, excluded_operators=None,
                     offline_params=None, quantized_dtype="int8", quantize_mode="smart",
                     quantize_granularity="tensor-wise"):
    """FP32 symbol -> (INT8 symbol, names of the tensors to calibrate)."""
    excluded_symbols = list(excluded_symbols or [])
    excluded_operators = list(excluded_operators or [])
    offline_params = list(offline_params or [])
    out = ctypes.c_char_p()
    n = ctypes.c_int()
    names = ctypes.POINTER(ctypes.c_char_p)()
    _operator._check(_operator.ops.mxq_quantize_symbol(
        sym.tojson().encode(), _DEV_TYPE[device], len(excluded_symbols),
        _c_strs(excluded_symbols), len(excluded_operators), _c_strs(excluded_operators),
        len(offline_params), _c_strs(offline_params), quantized_dtype.encode(),
        quantize_mode.encode(), quantize_granularity.encode(), ctypes.byref(out), ctypes.byref(n),
        ctypes.byref(names)))
    calib_layers = [names[i].decode() for i in range(n.value)]
    return Symbol.fromjson(out.value.decode()), calib_layers


def _calibrate_quantized_sym(qsym, min_max_dict):
    """Writes the thresholds into the min_calib_range / max_calib_range attributes of the
    quantize / requantize nodes they belong to."""
    if min_max_dict is None or len(min_max_dict) == 0:
        return qsym
    names = list(min_max_dict.keys())
    mins = (ctypes.c_float * len(names))(*[float(min_max_dict[k][0]) for k in names])
    maxs = (ctypes.c_float * len(names))(*[float(min_max_dict[k][1]) for k in names])
    out = ctypes.c_char_p()
    _operator._check(_operator.ops.mxq_set_calib_table(qsym.tojson().encode(), len(names),
                                                       _c_strs(names), mins, maxs,
                                                       ctypes.byref(out)))
    return Symbol.fromjson(out.value.decode())


def _own_range_int8(tensor):
    """int8 values and the (min, max) scalars of a float parameter quantized over its own
    range by the v1 quantize operator."""
    from . import contrib
    t = tensor if isinstance(tensor, torch.Tensor) else torch.as_tensor(tensor)
    t = t.cuda().to(torch.float32).contiguous()
    bounds = [f().reshape(1).to(torch.float32) for f in (t.min, t.max)]
    return contrib.quantize(t, bounds[0], bounds[1], out_type="int8")


def _quantize_params(qsym, params, min_max_dict):
    """Parameters of the quantized symbol, keyed by its argument names: `<p>_quantize`
    (int8, the parameter's own range) with `<p>_quantize_min` / `_max` for weights and
    biases, parameters of nodes that stayed float as they are, and one-element `<x>_min` /
    `<x>_max` tensors for the entries of `min_max_dict`
    (python/mxnet/contrib/quantization.py:85-123)."""
    result = {}
    for arg in qsym.list_arguments():
        stem, _, tail = arg.rpartition("_")
        if tail == "quantize" and stem.endswith(("weight", "bias")):
            q, lo, hi = _own_range_int8(params[stem])
            result.update({arg: q, arg + "_min": lo, arg + "_max": hi})
        elif arg in params:
            result[arg] = params[arg]
        elif tail in ("min", "max") and stem in min_max_dict:
            bound = min_max_dict[stem][1 if tail == "max" else 0]
            result[arg] = torch.tensor([bound], dtype=torch.float32)
    return result


class CalibrationCollector:
    """Base of the collectors hooked into the float network: `collect(name, op_name,
    arr)` sees tensors, `post_collect()` returns {name: (min, max)}."""

    def __init__(self):
        self.include_layers = None
        self.min_max_dict = {}

    def collect(self, name, op_name, arr):
        raise NotImplementedError

    def post_collect(self):
        return self.min_max_dict


def _to_numpy(arr):
    return arr.detach().cpu().numpy() if isinstance(arr, torch.Tensor) else np.asarray(arr)


class _LayerOutputMinMaxCollector(CalibrationCollector):
    """calib_mode='naive': running min / max of every calibrated tensor."""

    def __init__(self, quantized_dtype, include_layers=None, logger=None):
        super().__init__()
        self.quantized_dtype = quantized_dtype
        self.include_layers = include_layers
        self.logger = logger

    def collect(self, name, op_name, arr):
        if name not in self.include_layers:
            return
        arr = _to_numpy(arr)
        lo, hi = np.min(arr), np.max(arr)
        if name in self.min_max_dict:
            cur = self.min_max_dict[name]
            self.min_max_dict[name] = (min(cur[0], lo), max(cur[1], hi))
        else:
            self.min_max_dict[name] = (lo, hi)


def calibrate_entropy(hist, hist_edges, num_quantized_bins=255):
    """_contrib_calibrate_entropy: (threshold, divergence)."""
    hist = np.ascontiguousarray(hist, dtype=np.float32)
    edges = np.ascontiguousarray(hist_edges, dtype=np.float32)
    if edges.size != hist.size + 1:
        raise ValueError("hist_edges needs one more entry than hist")
    th, div = ctypes.c_float(), ctypes.c_float()
    fp = ctypes.POINTER(ctypes.c_float)
    _operator._check(_operator.ops.mxq_calibrate_entropy(
        hist.ctypes.data_as(fp), edges.ctypes.data_as(fp), hist.size, int(num_quantized_bins),
        ctypes.byref(th), ctypes.byref(div)))
    return np.float32(th.value), np.float32(div.value)


class _SymmetricHistogram:
    """Counts of a tensor's values over [-th, th] in equal bins, growable by whole bins on
    both sides so that what was counted keeps its bins when a later batch reaches further
    out.  `lo` / `hi` are the extreme values seen."""

    def __init__(self, counts, th, lo, hi):
        self.counts, self.th, self.lo, self.hi = counts, th, lo, hi

    @classmethod
    def of(cls, arr, bins):
        lo, hi = np.min(arr), np.max(arr)
        th = max(abs(lo), abs(hi))
        return cls(np.histogram(arr, bins=bins, range=(-th, th))[0], th, lo, hi)

    @classmethod
    def from_tuple(cls, t):
        return cls(t[0], t[4], t[2], t[3])

    def as_tuple(self):
        edges = np.linspace(-self.th, self.th, len(self.counts) + 1)
        return (self.counts, edges, self.lo, self.hi, self.th)

    def absorb(self, arr, lo, hi, reach):
        """Count one more batch (`reach` = max |value| of it)."""
        if reach > self.th:
            width = 2 * self.th / len(self.counts)
            margin = int((reach - self.th) // width + 1)
            self.counts = np.pad(self.counts, margin)
            self.th = margin * width + self.th
        batch = np.histogram(arr, bins=len(self.counts), range=(-self.th, self.th))[0]
        self.counts = self.counts + batch
        self.lo, self.hi = min(self.lo, lo), max(self.hi, hi)
        return self


class _LayerHistogramCollector(CalibrationCollector):
    """calib_mode='entropy': a symmetric histogram per calibrated tensor, grown over the
    batches, then the KL-optimal threshold of each
    (python/mxnet/contrib/quantization.py:269-361).  `hist_dict[name]` is the reference's
    tuple (hist, edges, min, max, threshold)."""

    def __init__(self, quantized_dtype, num_bins=8001, include_layers=None, logger=None):
        super().__init__()
        self.hist_dict = {}
        self.num_bins = num_bins
        self.include_layers = include_layers
        self.logger = logger
        self.quantized_dtype = quantized_dtype

    def collect(self, name, op_name, arr):
        if name not in self.include_layers:
            return
        arr = _to_numpy(arr)
        seen = self.hist_dict.get(name)
        if seen is None:
            self.hist_dict[name] = _SymmetricHistogram.of(arr, self.num_bins).as_tuple()
        else:
            lo, hi = np.min(arr), np.max(arr)
            self.hist_dict[name] = self.combine_histogram(seen, arr, lo, hi,
                                                          max(abs(lo), abs(hi)))

    def post_collect(self):
        return self.get_optimal_thresholds(self.hist_dict, self.quantized_dtype,
                                           logger=self.logger)

    @staticmethod
    def combine_histogram(old_hist, arr, new_min, new_max, new_th):
        return _SymmetricHistogram.from_tuple(old_hist).absorb(
            arr, new_min, new_max, new_th).as_tuple()

    @staticmethod
    def get_optimal_threshold(hist_data, quantized_dtype, num_quantized_bins=255):
        (hist, hist_edges, min_val, max_val, _) = hist_data
        assert len(hist) % 2 == 1
        if min_val >= 0 and quantized_dtype in ["auto", "uint8"]:
            # all levels sit on the positive side: twice the resolution
            num_quantized_bins = num_quantized_bins * 2 + 1
        threshold, divergence = calibrate_entropy(hist, hist_edges, num_quantized_bins)
        return min_val, max_val, threshold, divergence

    @staticmethod
    def get_optimal_thresholds(hist_dict, quantized_dtype, num_quantized_bins=255, logger=None):
        th_dict = {}
        for name in list(hist_dict.keys()):
            min_val, max_val, th, divergence = _LayerHistogramCollector.get_optimal_threshold(
                hist_dict[name], quantized_dtype, num_quantized_bins=num_quantized_bins)
            if min_val >= 0 and quantized_dtype in ["auto", "uint8"]:
                th_dict[name] = (0, th)
            else:
                th_dict[name] = (-th, th)
            del hist_dict[name]
            if logger:
                logger.debug("layer=%s, min_val=%s, max_val=%s, th=%s, divergence=%s",
                             name, min_val, max_val, th, divergence)
        return th_dict


def _collect_layer_statistics(executor, calib_data, collector, data_names,
                              num_calib_batches=None, logger=None):
    """Runs the float network over the calibration batches with the collector hooked in.
    A batch is a tensor (one input) or a list / tuple of tensors in data_names order."""
    executor.register_op_hook(collector.collect, monitor_all=True)
    num_batches = 0
    for batch in calib_data:
        if not isinstance(batch, (list, tuple)):
            batch = [batch]
        executor.forward(**{n: b for n, b in zip(data_names, batch)})
        num_batches += 1
        if num_calib_batches is not None and num_batches >= num_calib_batches:
            break
    if logger is not None:
        logger.info("Collected statistics from %d batches", num_batches)
    return num_batches


def quantize_model(sym, arg_params, aux_params, data_names=("data",), device="gpu",
                   excluded_sym_names=None, excluded_op_names=None, calib_mode="entropy",
                   calib_data=None, num_calib_batches=None, quantized_dtype="int8",
                   quantize_mode="smart", quantize_granularity="tensor-wise", logger=None):
    """FP32 symbol + parameters -> (quantized symbol, quantized arg_params, aux_params)."""
    excluded_sym_names = excluded_sym_names or []
    if not isinstance(excluded_sym_names, list):
        raise ValueError("excluded_sym_names must be a list of strings representing the names of "
                         "the symbols that will not be quantized, while received type %s"
                         % type(excluded_sym_names))
    excluded_op_names = excluded_op_names or []
    if not isinstance(excluded_op_names, list):
        raise ValueError("excluded_op_names must be a list of strings representing the names of "
                         "the operators that will not be quantized, while received type %s"
                         % type(excluded_op_names))
    if quantized_dtype not in ("int8", "uint8", "auto"):
        raise ValueError("unknown quantized_dtype %s received, expected `int8`, `uint8` or `auto`"
                         % quantized_dtype)
    if quantize_granularity not in ("tensor-wise", "channel-wise"):
        raise ValueError("unkonwn quantize_granularity %s received, expected `tensor-wise` or "
                         "`channel-wise`." % quantize_granularity)
    qsym, calib_layers = _quantize_symbol(sym, device, excluded_symbols=excluded_sym_names,
                                          excluded_operators=excluded_op_names,
                                          offline_params=list(arg_params.keys()),
                                          quantized_dtype=quantized_dtype,
                                          quantize_mode=quantize_mode,
                                          quantize_granularity=quantize_granularity)
    min_max_dict = {}
    if calib_mode is not None and calib_mode != "none":
        if calib_data is None:
            raise ValueError("calib_data must be provided when calib_mode=%s" % calib_mode)
        params = dict(arg_params)
        params.update(aux_params)
        executor = Executor(sym, params)
        if calib_mode == "entropy":
            collector = _LayerHistogramCollector(quantized_dtype=quantized_dtype,
                                                 include_layers=calib_layers, logger=logger)
        elif calib_mode == "naive":
            collector = _LayerOutputMinMaxCollector(quantized_dtype=quantized_dtype,
                                                    include_layers=calib_layers, logger=logger)
        else:
            raise ValueError("unknown calibration mode %s received, expected `none`, `naive`, or "
                             "`entropy`" % calib_mode)
        _collect_layer_statistics(executor, calib_data, collector, list(data_names),
                                  num_calib_batches, logger)
        min_max_dict = collector.post_collect()
        qsym = _calibrate_quantized_sym(qsym, min_max_dict)
    qarg_params = _quantize_params(qsym, arg_params, min_max_dict)
    return qsym, qarg_params, aux_params


def quantize_graph(sym, arg_params, aux_params, device="gpu", excluded_sym_names=None,
                   excluded_op_names=None, calib_mode="entropy", quantized_dtype="int8",
                   quantize_mode="full", quantize_granularity="tensor-wise",
                   LayerOutputCollector=None, logger=None):
    """The two-step form of quantize_model (python/mxnet/contrib/quantization.py:613-738):
    returns (qsym, qarg_params, aux_params, collector, calib_layers).  The caller feeds the
    collector (e.g. `Executor.register_op_hook(collector.collect)` over calibration batches)
    and then calls `calib_graph`."""
    excluded_sym_names = excluded_sym_names or []
    if not isinstance(excluded_sym_names, list):
        raise ValueError("excluded_sym_names must be a list of strings representing the names of "
                         "the symbols that will not be quantized, while received type %s"
                         % type(excluded_sym_names))
    if quantized_dtype not in ("int8", "uint8", "auto"):
        raise ValueError("unknown quantized_dtype %s received, expected `int8`, `uint8` or `auto`"
                         % quantized_dtype)
    if quantize_granularity not in ("tensor-wise", "channel-wise"):
        raise ValueError("unkonwn quantize_granularity %s received, expected `tensor-wise` or "
                         "`channel-wise`." % quantize_granularity)
    qsym, calib_layers = _quantize_symbol(sym, device, excluded_symbols=excluded_sym_names,
                                          excluded_operators=excluded_op_names,
                                          offline_params=list(arg_params.keys()),
                                          quantized_dtype=quantized_dtype,
                                          quantize_mode=quantize_mode,
                                          quantize_granularity=quantize_granularity)
    collector = None
    if calib_mode is not None and calib_mode != "none":
        if calib_mode == "entropy":
            collector = _LayerHistogramCollector(quantized_dtype=quantized_dtype,
                                                 include_layers=calib_layers, logger=logger)
        elif calib_mode == "naive":
            collector = _LayerOutputMinMaxCollector(quantized_dtype=quantized_dtype,
                                                    include_layers=calib_layers, logger=logger)
        elif calib_mode == "custom" and LayerOutputCollector is not None:
            if not isinstance(LayerOutputCollector, CalibrationCollector):
                raise ValueError("LayerOutputCollecotr must be a subclass of a "
                                 "CalibrationCollector class, but it is %s"
                                 % LayerOutputCollector.__class__)
            collector = LayerOutputCollector
            # the names of the tensors that need calibration, unless the collector brings its own
            if getattr(collector, "include_layers", None) is None:
                collector.include_layers = calib_layers
        else:
            raise ValueError("unknown calibration mode %s received, expected `none`, `naive`, "
                             "`entropy` or `custom`" % calib_mode)
    qarg_params = _quantize_params(qsym, arg_params, min_max_dict={})
    return qsym, qarg_params, aux_params, collector, calib_layers


def calib_graph(qsym, arg_params, aux_params, collector, calib_mode="entropy", logger=None):
    """Second step (python/mxnet/contrib/quantization.py:740-796): the collector's thresholds
    onto the quantized symbol, the parameters quantized against it.  `arg_params` are the
    FP32 parameters."""
    if calib_mode is not None and calib_mode != "none":
        if calib_mode in ("entropy", "naive", "custom"):
            min_max_dict = collector.post_collect()
        else:
            raise ValueError("unknown calibration mode %s received, expected `none`, `naive`, "
                             "`entropy` or `custom`" % calib_mode)
        qsym = _calibrate_quantized_sym(qsym, min_max_dict)
    else:
        raise ValueError("Please set calibration mode to naive, entropy or custom (with custom "
                         "CalibrationCollector)")
    qarg_params = _quantize_params(qsym, arg_params, min_max_dict)
    return qsym, qarg_params, aux_params
