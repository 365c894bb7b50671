"""Symbols as text: a thin composer / inspector over the NNVM symbol JSON.

The reference's `mx.sym` builds an nnvm::Symbol in C++ and serialises it with `tojson()`;
the graph passes of this package (include/mxq_ops.h) take and return that JSON, so a
symbol here *is* its JSON plus a few of the queries `python/mxnet/symbol/symbol.py`
offers (list_arguments :1068, list_outputs :1094, list_auxiliary_states :1140, attr_dict
:748, tojson :1432, get_internals :912).  Composition follows the reference's rules: a
missing operator argument becomes a variable named `<node>_<argument>`
(nnvm Symbol::Compose), node names default to `<op lower-case><counter>`.
"""
import ctypes
import json

from . import operator as _operator

# inputs an operator mutates: they are auxiliary states, not arguments
# (FMutateInputs, src/operator/nn/batch_norm.cc:641-644)
_MUTATED_INPUTS = {"BatchNorm": (3, 4)}

_name_counters = {}


def _auto_name(op):
    hint = op.lower().lstrip("_")
    n = _name_counters.get(hint, 0)
    _name_counters[hint] = n + 1
    return "%s%d" % (hint, n)


def _attr_str(v):
    if isinstance(v, bool):
        return "True" if v else "False"
    if isinstance(v, (tuple, list)):
        return "(" + ", ".join(str(x) for x in v) + ")"
    return str(v)


class _Node:
    __slots__ = ("op", "name", "attrs", "inputs")

    def __init__(self, op, name, attrs, inputs):
        self.op, self.name, self.attrs = op, name, attrs
        self.inputs = inputs  # list of (_Node, output index, version)


class Symbol:
    """A list of heads, each (node, output index, version); nodes refer to their inputs
    by object, so symbols share sub-graphs the way nnvm symbols do."""

    def __init__(self, heads):
        self._heads = list(heads)

    # ---- construction -------------------------------------------------------------
    @staticmethod
    def fromjson(text):
        g = json.loads(text)
        nodes = []

        def entry(e):
            if not 0 <= e[0] < len(nodes):
                raise _operator.MXNetError("symbol JSON: entry refers to a later or missing node")
            return (nodes[e[0]], e[1], e[2] if len(e) > 2 else 0)

        for n in g["nodes"]:
            attrs = {}
            for key in ("param", "attr", "attrs"):
                attrs.update(n.get(key, {}))
            nodes.append(_Node(n["op"], n["name"], attrs, [entry(e) for e in n.get("inputs", [])]))
        return Symbol([entry(e) for e in g["heads"]])

    def tojson(self):
        """The normalised JSON: reachable nodes in depth-first post-order."""
        order = self._post_order()
        pos = {id(n): i for i, n in enumerate(order)}
        raw = {"nodes": [dict(op=n.op, name=n.name,
                              inputs=[[pos[id(m)], k, v] for m, k, v in n.inputs],
                              **({"attrs": n.attrs} if n.attrs else {})) for n in order],
               "arg_nodes": [i for i, n in enumerate(order) if n.op == "null"],
               "heads": [[pos[id(m)], k, v] for m, k, v in self._heads]}
        out = ctypes.c_char_p()
        _operator._check(_operator.ops.mxq_symbol_normalize(json.dumps(raw).encode(),
                                                            ctypes.byref(out)))
        return out.value.decode()

    def __getitem__(self, index):
        if isinstance(index, str):
            index = self.list_outputs().index(index)
        return Symbol([self._heads[index]])

    def __len__(self):
        return len(self._heads)

    # ---- queries ----------------------------------------------------------------------
    def _post_order(self):
        order, seen = [], set()
        for head, _, _ in self._heads:
            if id(head) in seen:
                continue
            seen.add(id(head))
            stack = [(head, 0)]
            while stack:
                node, i = stack.pop()
                if i < len(node.inputs):
                    stack.append((node, i + 1))
                    nxt = node.inputs[i][0]
                    if id(nxt) not in seen:
                        seen.add(id(nxt))
                        stack.append((nxt, 0))
                else:
                    order.append(node)
        return order

    def _aux_ids(self):
        aux = set()
        for n in self._post_order():
            for i in _MUTATED_INPUTS.get(n.op, ()):
                if i < len(n.inputs):
                    aux.add(id(n.inputs[i][0]))
        return aux

    def list_arguments(self):
        aux = self._aux_ids()
        return [n.name for n in self._post_order() if n.op == "null" and id(n) not in aux]

    def list_auxiliary_states(self):
        aux = self._aux_ids()
        return [n.name for n in self._post_order() if n.op == "null" and id(n) in aux]

    def list_inputs(self):
        return [n.name for n in self._post_order() if n.op == "null"]

    @staticmethod
    def _output_names(n):
        """Registered output names, nnvm's defaults for operators unknown here."""
        try:
            probe = _operator.Node(n.op, **n.attrs)
            names = probe.list_outputs()
            if names:
                return names
            count = probe.num_outputs
        except _operator.MXNetError:
            count = 1
        return ["output"] if count == 1 else ["output%d" % k for k in range(count)]

    def list_outputs(self):
        out = []
        for n, index, _ in self._heads:
            out.append(n.name if n.op == "null" else
                       "%s_%s" % (n.name, self._output_names(n)[index]))
        return out

    def attr_dict(self):
        return {n.name: dict(n.attrs) for n in self._post_order() if n.attrs}

    def get_internals(self):
        heads = []
        for n in self._post_order():
            count = 1 if n.op == "null" else len(self._output_names(n))
            heads.extend((n, k, 0) for k in range(count))
        return Symbol(heads)

    def nodes(self):
        """(op, name, attrs, inputs) of the reachable nodes in post-order, inputs as
        (position in this list, output index)."""
        order = self._post_order()
        pos = {id(n): i for i, n in enumerate(order)}
        return [(n.op, n.name, dict(n.attrs), [(pos[id(m)], k) for m, k, _ in n.inputs])
                for n in order]

    def heads(self):
        pos = {id(n): i for i, n in enumerate(self._post_order())}
        return [(pos[id(n)], k) for n, k, _ in self._heads]


def Variable(name, **attrs):
    return Symbol([(_Node("null", name, {k: _attr_str(v) for k, v in attrs.items()}, []), 0, 0)])


var = Variable


def Group(symbols):
    heads = []
    for s in symbols:
        heads.extend(s._heads)
    return Symbol(heads)


def create(op, *args, name=None, **kwargs):
    """`mx.sym.<op>(*args, name=..., **attrs)`: positional and keyword symbol arguments
    fill the operator's named inputs; the rest become `<name>_<argument>` variables."""
    sym_kwargs = {k: v for k, v in kwargs.items() if isinstance(v, Symbol)}
    attrs = {k: _attr_str(v) for k, v in kwargs.items()
             if not isinstance(v, Symbol) and v is not None}
    name = name or _auto_name(op)
    given = list(args)
    try:
        probe = _operator.Node(op, **attrs)
        arg_names = probe.list_inputs()
        if not arg_names:  # nnvm's default names
            n = probe.num_inputs
            arg_names = ["data"] if n == 1 else ["arg%d" % i for i in range(n)]
    except _operator.MXNetError as e:
        if "not registered" not in str(e):
            raise
        # an operator this build knows nothing about: positional inputs only
        arg_names = ["arg%d" % i for i in range(len(given))]
    if len(given) > len(arg_names):
        raise TypeError("%s takes %d inputs, got %d" % (op, len(arg_names), len(given)))
    bound = {arg_names[i]: s for i, s in enumerate(given)}
    for k, s in sym_kwargs.items():
        if k not in arg_names:
            raise TypeError("%s has no input named %r" % (op, k))
        bound[k] = s
    inputs = []
    for arg in arg_names:
        s = bound.get(arg)
        if s is None:
            s = Variable("%s_%s" % (name, arg))
        if len(s._heads) != 1:
            raise TypeError("an operator input must be a single-output symbol")
        inputs.append(s._heads[0])
    return Symbol([(_Node(op, name, attrs, inputs), 0, 0)])


def _make(op):
    def f(*args, **kwargs):
        return create(op, *args, **kwargs)
    f.__name__ = op
    return f


Convolution = _make("Convolution")
FullyConnected = _make("FullyConnected")
Activation = _make("Activation")
Pooling = _make("Pooling")
Flatten = _make("Flatten")
BatchNorm = _make("BatchNorm")
softmax = _make("softmax")
SoftmaxOutput = _make("SoftmaxOutput")
Dropout = _make("Dropout")
elemwise_add = _make("elemwise_add")
elemwise_mul = _make("elemwise_mul")
Embedding = _make("Embedding")
Reshape = _make("Reshape")
reshape = Reshape
transpose = _make("transpose")


def Concat(*args, name=None, dim=1, **kwargs):
    """`mx.sym.Concat(a, b, ..., dim=1)`: num_args is the number of symbols given
    (the operator's key_var_num_args)."""
    return create("Concat", *args, name=name, num_args=len(args), dim=dim, **kwargs)


concat = Concat
