"""A minimal symbol executor for calibration runs and end-to-end checks.

It walks a symbol in depth-first post-order and evaluates each node on the GPU: the
`_contrib_*` operators through the C++ operator host (FCompute<gpu> of this package),
the float operators of the surrounding network through torch.  The reference runs
symbols through CachedOp / the graph executor (src/imperative/cached_op.cc), which is
outside this package; this is only the harness the calibration collectors hook into,
the way `SymbolBlock.register_op_hook(collector.collect, monitor_all=True)` does in
`_collect_layer_statistics` (python/mxnet/contrib/quantization.py:364-380): the callback
sees every operator output as `<node>_<output name>` and, with monitor_all, every
operator input as `<node>_<argument name>`; operators without registered names get
the decimal output index and `input<i>` (src/common/utils.cc:53-107).
"""
import torch

from . import operator as _operator


def _tuple(text, n=2, default=None):
    if text is None:
        return default
    t = text.strip().strip("()[]")
    vals = tuple(int(x) for x in t.split(",") if x.strip())
    return vals if vals else default


def _bool(text, default=False):
    if text is None:
        return default
    return text.strip().lower() in ("true", "1")


def _convolution(a, data, weight, bias=None):
    kernel = _tuple(a.get("kernel"))
    return torch.nn.functional.conv2d(data, weight, bias, stride=_tuple(a.get("stride"), default=(1, 1)),
                                      padding=_tuple(a.get("pad"), default=(0, 0)),
                                      dilation=_tuple(a.get("dilate"), default=(1, 1)),
                                      groups=int(a.get("num_group", "1")))


def _fully_connected(a, data, weight, bias=None):
    if _bool(a.get("flatten"), True):
        data = data.reshape(data.shape[0], -1)
    return torch.nn.functional.linear(data, weight, bias)


def _activation(a, data):
    return {"relu": torch.relu, "sigmoid": torch.sigmoid, "tanh": torch.tanh,
            "softrelu": torch.nn.functional.softplus,
            "softsign": torch.nn.functional.softsign}[a["act_type"]](data)


def _pooling(a, data):
    pool_type = a.get("pool_type", "max")
    if _bool(a.get("global_pool")):
        return data.amax(dim=(2, 3), keepdim=True) if pool_type == "max" else \
            data.mean(dim=(2, 3), keepdim=True)
    kernel = _tuple(a.get("kernel"))
    stride = _tuple(a.get("stride"), default=(1, 1))
    pad = _tuple(a.get("pad"), default=(0, 0))
    ceil = a.get("pooling_convention", "valid") == "full"
    if pool_type == "max":
        return torch.nn.functional.max_pool2d(data, kernel, stride, pad, ceil_mode=ceil)
    if pool_type == "avg":
        return torch.nn.functional.avg_pool2d(
            data, kernel, stride, pad, ceil_mode=ceil,
            count_include_pad=_bool(a.get("count_include_pad"), True))
    raise NotImplementedError("Pooling pool_type=%s" % pool_type)


def _batch_norm(a, data, gamma, beta, mean, var):
    if _bool(a.get("fix_gamma"), True):
        gamma = torch.ones_like(gamma)
    eps = float(a.get("eps", "0.001"))
    shape = [1, -1] + [1] * (data.dim() - 2)
    return (data - mean.reshape(shape)) / torch.sqrt(var.reshape(shape) + eps) * \
        gamma.reshape(shape) + beta.reshape(shape)


def _shape_attr(value):
    text = str(value).strip()
    if text in ("", "None", "()", "[]"):
        return ()
    return tuple(int(v) for v in text.strip("()[] ").split(",") if v.strip())


def _reshape(a, x):
    """`Reshape` for the plain target shapes (positive extents, 0 = keep, one -1); the
    other special values are resolved by the operator host for the quantized twin only."""
    shape = list(_shape_attr(a.get("shape", "()")))
    if any(v < -1 for v in shape) or _bool(a.get("reverse"), False):
        raise NotImplementedError("Reshape special values -2/-3/-4 in the float executor")
    shape = [x.shape[i] if v == 0 else v for i, v in enumerate(shape)]
    return x.reshape(shape)


def _transpose(a, x):
    axes = _shape_attr(a.get("axes", "()"))
    return x.permute(*(axes if axes else reversed(range(x.dim())))).contiguous()


def _embedding(a, idx, weight):
    j = idx.to(torch.int64).clamp(0, weight.shape[0] - 1)
    return weight[j]


_FLOAT_OPS = {
    "Convolution": _convolution,
    "FullyConnected": _fully_connected,
    "Activation": _activation,
    "Pooling": _pooling,
    "BatchNorm": _batch_norm,
    "Flatten": lambda a, x: x.reshape(x.shape[0], -1),
    "flatten": lambda a, x: x.reshape(x.shape[0], -1),
    "softmax": lambda a, x: torch.softmax(x, dim=int(a.get("axis", "-1"))),
    "SoftmaxOutput": lambda a, x, label=None: torch.softmax(x, dim=1),
    "Dropout": lambda a, x: x,
    "elemwise_add": lambda a, x, y: x + y,
    "_plus": lambda a, x, y: x + y,
    "elemwise_mul": lambda a, x, y: x * y,
    "Embedding": _embedding,
    "Reshape": _reshape,
    "reshape": _reshape,
    "transpose": _transpose,
    "Concat": lambda a, *xs: torch.cat(xs, dim=int(a.get("dim", "1"))),
    "concat": lambda a, *xs: torch.cat(xs, dim=int(a.get("dim", "1"))),
}


class Executor:
    """`Executor(symbol, params).forward(data=...)` -> list of outputs (torch tensors on
    the GPU).  `params` maps variable names to tensors."""

    def __init__(self, symbol, params, device="cuda"):
        self.symbol = symbol
        self.device = device
        self.params = {k: (v if isinstance(v, torch.Tensor) else torch.as_tensor(v)).to(device)
                       for k, v in params.items()}
        self.monitor = None
        self.monitor_all = False
        self._nodes = {}

    def register_op_hook(self, callback, monitor_all=False):
        """callback(name, op_name, array) as in Block.register_op_hook."""
        self.monitor = callback
        self.monitor_all = monitor_all

    def _op_node(self, i, op, name, attrs):
        node = self._nodes.get(i)
        if node is None:
            node = self._nodes[i] = _operator.Node(op, name, **attrs)
        return node

    def forward(self, **feed):
        values = []
        nodes = self.symbol.nodes()
        for i, (op, name, attrs, inputs) in enumerate(nodes):
            if op == "null":
                if name in feed:
                    v = feed[name]
                    v = (v if isinstance(v, torch.Tensor) else torch.as_tensor(v)).to(self.device)
                elif name in self.params:
                    v = self.params[name]
                else:
                    raise KeyError("no value for variable %r" % name)
                values.append([v])
                continue
            args = [values[j][k] for j, k in inputs]
            if op.startswith("_contrib_") or op.startswith("_npx_"):
                node = self._op_node(i, op, name, attrs)
                out = node(*[a.contiguous() for a in args])
                outs = list(out) if isinstance(out, (tuple, list)) else [out]
                in_names, out_names = node.list_inputs(), node.list_outputs()
            else:
                fn = _FLOAT_OPS.get(op)
                if fn is None:
                    raise NotImplementedError("the harness executor has no float operator %r" % op)
                out = fn(attrs, *args)
                outs = list(out) if isinstance(out, (tuple, list)) else [out]
                try:
                    probe = self._op_node(i, op, name, attrs)
                    in_names, out_names = probe.list_inputs(), probe.list_outputs()
                except _operator.MXNetError:
                    in_names, out_names = [], []
            values.append(outs)
            if self.monitor is not None:
                if self.monitor_all:
                    for k, arr in enumerate(args):
                        arg = in_names[k] if k < len(in_names) else "input%d" % k
                        self.monitor("%s_%s" % (name, arg), op, arr)
                for k, arr in enumerate(outs):
                    out_name = out_names[k] if k < len(out_names) else str(k)
                    self.monitor("%s_%s" % (name, out_name), op, arr)
        return [values[j][k] for j, k in self.symbol.heads()]
