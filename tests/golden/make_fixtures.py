"""Writes tests/golden/operator_vectors.npz: small seeded input/output vectors of every
operator on the path, produced by the CPU oracle (whose arithmetic is pinned separately by
the exact-rational and known-answer tests).  The file is data only: operator name, its
attributes as JSON, the input arrays in the operator's argument order (range scalars as
float32 arrays of shape (1,)) and the expected outputs.

Two consumers: a CPU test replays the oracle against the file (a change of the oracle's
results then shows up as a diff of a committed file), a GPU test runs the operators through
the operator host and compares with the file.

    python tests/golden/make_fixtures.py          # rewrites the file
"""
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PATH = os.path.join(HERE, "operator_vectors.npz")


def s(v):
    return np.array([v], np.float32)


def _i8(rng, shape, lo=-127, hi=127):
    return rng.integers(lo, hi + 1, size=shape, dtype=np.int8)


def _u8(rng, shape):
    return rng.integers(0, 256, size=shape, dtype=np.uint8)


def _outliers(rng, n, laplace=False, mag=50.0):
    x = rng.laplace(0.0, 1.0, n).astype(np.float32) if laplace else \
        rng.standard_normal(n, dtype=np.float32)
    idx = rng.choice(n, size=max(1, n // 500), replace=False)
    x[idx] = mag * rng.choice(np.array([-1.0, 1.0], np.float32), size=idx.size)
    return x


def cases():
    """[(operator, attrs, inputs)] — seeded, sizes chosen with ragged tails."""
    rng = np.random.default_rng(20240607)
    out = []
    x = _outliers(rng, 1031)
    out.append(("_contrib_quantize_v2", dict(out_type="int8", min_calib_range=-4.0,
                                             max_calib_range=4.0), [x]))
    out.append(("_contrib_quantize_v2", dict(out_type="int8", min_calib_range=-50.0,
                                             max_calib_range=50.0), [x]))
    y = _outliers(rng, 1031, laplace=True)
    out.append(("_contrib_quantize_v2", dict(out_type="int8"), [y]))
    out.append(("_contrib_quantize_v2", dict(out_type="uint8", min_calib_range=float(y.min()),
                                             max_calib_range=float(y.max())), [y]))
    out.append(("_contrib_quantize_v2", dict(out_type="auto", min_calib_range=0.0,
                                             max_calib_range=7.5), [np.abs(y) / 8]))
    out.append(("_contrib_quantize", dict(out_type="int8"), [x, s(x.min()), s(x.max())]))
    q32 = rng.integers(-1000, 1001, size=(13, 37), dtype=np.int32) * 1000003
    out.append(("_contrib_requantize", dict(min_calib_range=-134.349, max_calib_range=523.43),
                [q32, s(-1010.0), s(1020.0)]))
    out.append(("_contrib_requantize", dict(), [q32, s(-1010.0), s(1020.0)]))
    out.append(("_contrib_dequantize", dict(), [_i8(rng, (1031,), -128), s(-2.5), s(3.25)]))
    out.append(("_contrib_dequantize", dict(), [_u8(rng, (1031,)), s(0.5), s(3.25)]))
    # fully connected: ragged in every dimension, with and without bias, flatten of 4-D data
    d, w, b = _i8(rng, (33, 80)), _i8(rng, (100, 80)), _i8(rng, (100,))
    out.append(("_contrib_quantized_fully_connected", dict(num_hidden=100, no_bias=False),
                [d, w, b, s(-1.0), s(1.0), s(-0.08), s(0.08), s(-0.5), s(0.5)]))
    d4, w4 = _i8(rng, (8, 111, 2, 2)), _i8(rng, (10, 444))
    out.append(("_contrib_quantized_fully_connected", dict(num_hidden=10, no_bias=True),
                [d4, w4, s(-3.0), s(2.0), s(-0.3), s(0.2)]))
    # convolution: 3x3 stride 2 pad 1 with bias; a 4-channel case as in the reference's test; 1x1
    cd, cw, cb = _i8(rng, (2, 16, 9, 9)), _i8(rng, (24, 16, 3, 3)), _i8(rng, (24,))
    out.append(("_contrib_quantized_conv",
                dict(kernel=(3, 3), stride=(2, 2), pad=(1, 1), num_filter=24, no_bias=False),
                [cd, cw, cb, s(-1.0), s(1.0), s(-0.1), s(0.1), s(-0.4), s(0.4)]))
    cd4, cw4 = _i8(rng, (1, 4, 12, 12)), _i8(rng, (16, 4, 3, 3))
    out.append(("_contrib_quantized_conv",
                dict(kernel=(3, 3), pad=(1, 1), num_filter=16, no_bias=True),
                [cd4, cw4, s(-1.0), s(1.0), s(-0.1), s(0.1)]))
    c1, w1 = _i8(rng, (1, 32, 7, 7)), _i8(rng, (16, 32, 1, 1))
    out.append(("_contrib_quantized_conv", dict(kernel=(1, 1), num_filter=16, no_bias=True),
                [c1, w1, s(-2.0), s(2.0), s(-0.2), s(0.2)]))
    out.append(("_contrib_quantized_act", dict(act_type="relu"),
                [_i8(rng, (5, 77), -128), s(-1.5), s(1.0)]))
    p = _i8(rng, (2, 5, 13, 11), -128)
    out.append(("_contrib_quantized_pooling",
                dict(kernel=(3, 3), stride=(2, 2), pad=(1, 1), pool_type="max"),
                [p, s(-1.0), s(1.0)]))
    out.append(("_contrib_quantized_pooling",
                dict(kernel=(3, 3), stride=(2, 2), pool_type="avg", pooling_convention="full"),
                [p.view(np.uint8), s(0.0), s(1.0)]))
    out.append(("_contrib_quantized_pooling", dict(kernel=(1, 1), global_pool=True,
                                                   pool_type="avg"), [p, s(-1.0), s(1.0)]))
    out.append(("_contrib_quantized_flatten", dict(), [p, s(-1.0), s(1.0)]))
    a, b2 = _i8(rng, (3, 133), -128), _i8(rng, (3, 133), -128)
    out.append(("_contrib_quantized_elemwise_add", dict(),
                [a, b2, s(-1.0), s(2.0), s(-3.0), s(0.5)]))
    out.append(("_contrib_quantized_elemwise_add", dict(min_calib_range=-3.5,
                                                        max_calib_range=3.0),
                [a, b2.view(np.uint8), s(-1.0), s(2.0), s(0.0), s(2.5)]))
    out.append(("_contrib_quantized_concat", dict(num_args=3, dim=1),
                [a, b2.view(np.uint8), a[:, :17], s(-1.0), s(1.0), s(0.0), s(2.0), s(-0.5),
                 s(3.0)]))
    out.append(("_contrib_quantized_elemwise_mul", dict(),
                [a, b2, s(-1.0), s(2.0), s(-3.0), s(0.5)]))
    out.append(("_contrib_quantized_elemwise_mul", dict(min_calib_range=-4.0,
                                                        max_calib_range=5.0),
                [a, b2, s(-1.0), s(2.0), s(-3.0), s(0.5)]))
    out.append(("_contrib_quantized_elemwise_mul", dict(enable_float_output=True),
                [a, b2, s(-1.0), s(2.0), s(-3.0), s(0.5)]))
    table = _i8(rng, (50, 24), -128)
    ids = rng.integers(-3, 55, size=(4, 9)).astype(np.float32)
    out.append(("_contrib_quantized_embedding", dict(input_dim=50, output_dim=24),
                [ids, table, s(-0.7), s(0.9)]))
    t = _i8(rng, (3, 5, 4, 16), -128)
    out.append(("_contrib_quantized_transpose", dict(axes=(0, 2, 1, 3)), [t, s(-1.0), s(1.0)]))
    out.append(("_contrib_quantized_transpose", dict(axes=(3, 1, 0, 2)), [t, s(-1.0), s(1.0)]))
    out.append(("_contrib_quantized_reshape", dict(shape=(0, -3, -1)), [t, s(-1.0), s(1.0)]))
    out.append(("_contrib_quantize_asym", dict(min_calib_range=-6.0, max_calib_range=6.0),
                [x[:528].reshape(16, 33)]))
    out.append(("_contrib_quantize_asym", dict(), [y[:528].reshape(16, 33)]))
    C = 6
    bn = [rng.uniform(0.5, 2.0, C).astype(np.float32), rng.normal(0, 0.5, C).astype(np.float32),
          rng.normal(0, 0.3, C).astype(np.float32), rng.uniform(0.3, 2.0, C).astype(np.float32)]
    bd = _i8(rng, (3, C, 5, 16), -128)
    out.append(("_contrib_quantized_batch_norm", dict(eps=2e-5, min_calib_range=-6.5,
                                                      max_calib_range=7.25),
                [bd] + bn + [s(-2.7), s(3.1)]))
    out.append(("_contrib_quantized_batch_norm_relu", dict(eps=1e-3, min_calib_range=-6.5,
                                                           max_calib_range=7.25),
                [bd.view(np.uint8)] + bn + [s(0.0), s(3.1)]))
    out.append(("_npx_quantized_transpose", dict(axes=(-1, 0, -2, 1)), [t, s(-1.0), s(1.0)]))
    out.append(("_npx_quantized_reshape", dict(newshape=(-2, -5, -6, 4, -1)),
                [t, s(-1.0), s(1.0)]))
    out.append(("_contrib_quantized_npi_add", dict(),
                [bd, _u8(rng, (C, 1, 16)), s(-1.0), s(2.0), s(0.0), s(2.5)]))
    out.append(("_contrib_quantized_npi_add", dict(min_calib_range=-3.5, max_calib_range=3.0),
                [bd, _i8(rng, (1, C, 5, 1), -128), s(-1.0), s(2.0), s(-0.5), s(2.5)]))
    return out


def run_oracle(op, attrs, ins):
    """The oracle's answer for one case, as the operator's list of outputs."""
    import oracle
    f = lambda a: float(a[0])
    cal = (attrs.get("min_calib_range"), attrs.get("max_calib_range"))
    if op == "_contrib_quantize_v2":
        res = oracle.quantize_v2(ins[0], attrs["out_type"], *cal)
    elif op == "_contrib_quantize":
        res = oracle.quantize(ins[0], f(ins[1]), f(ins[2]), attrs["out_type"])
    elif op == "_contrib_requantize":
        res = oracle.requantize(ins[0], f(ins[1]), f(ins[2]), *cal)
    elif op == "_contrib_dequantize":
        return [oracle.dequantize(ins[0], f(ins[1]), f(ins[2]))]
    elif op == "_contrib_quantized_fully_connected":
        nb = attrs["no_bias"]
        r = [f(v) for v in ins[(2 if nb else 3):]]
        res = oracle.quantized_fully_connected(ins[0], ins[1], None if nb else ins[2], *r)
    elif op == "_contrib_quantized_conv":
        nb = attrs["no_bias"]
        r = [f(v) for v in ins[(2 if nb else 3):]] + ([None, None] if nb else [])
        res = oracle.quantized_conv(ins[0], ins[1], None if nb else ins[2], *r,
                                    stride=tuple(attrs.get("stride", (1, 1))),
                                    pad=tuple(attrs.get("pad", (0, 0))))
    elif op == "_contrib_quantized_act":
        return [oracle.relu_i8(ins[0]), ins[1], ins[2]]
    elif op == "_contrib_quantized_pooling":
        res = oracle.quantized_pooling(
            ins[0], f(ins[1]), f(ins[2]), kernel=tuple(attrs["kernel"]),
            pool_type=attrs["pool_type"], stride=tuple(attrs.get("stride", (1, 1))),
            pad=tuple(attrs.get("pad", (0, 0))), global_pool=attrs.get("global_pool", False),
            convention=attrs.get("pooling_convention", "valid"))
    elif op == "_contrib_quantized_flatten":
        res = oracle.quantized_flatten(ins[0], f(ins[1]), f(ins[2]))
    elif op == "_contrib_quantized_elemwise_add":
        res = oracle.quantized_elemwise_add(ins[0], ins[1], *[f(v) for v in ins[2:]], *cal)
    elif op == "_contrib_quantized_npi_add":
        res = oracle.quantized_npi_add(ins[0], ins[1], *[f(v) for v in ins[2:]], *cal)
    elif op == "_contrib_quantized_concat":
        n = attrs["num_args"]
        res = oracle.quantized_concat(ins[:n], [f(v) for v in ins[n::2]],
                                      [f(v) for v in ins[n + 1::2]], dim=attrs["dim"])
    elif op == "_contrib_quantized_elemwise_mul":
        res = oracle.quantized_elemwise_mul(ins[0], ins[1], *[f(v) for v in ins[2:]], *cal,
                                            enable_float_output=attrs.get("enable_float_output",
                                                                          False))
        if attrs.get("enable_float_output", False):
            return [res]
    elif op == "_contrib_quantized_embedding":
        res = oracle.quantized_embedding(ins[0], ins[1], f(ins[2]), f(ins[3]))
    elif op == "_contrib_quantized_transpose":
        res = oracle.quantized_transpose(ins[0], f(ins[1]), f(ins[2]), tuple(attrs["axes"]))
    elif op == "_contrib_quantized_reshape":
        # (0, -3, -1) on (3, 5, 4, 16): keep, merge two, infer the rest
        assert tuple(attrs["shape"]) == (0, -3, -1) and ins[0].shape == (3, 5, 4, 16)
        res = oracle.quantized_reshape(ins[0], f(ins[1]), f(ins[2]), (3, 20, 16))
    elif op == "_npx_quantized_transpose":
        res = oracle.quantized_transpose(ins[0], f(ins[1]), f(ins[2]), tuple(attrs["axes"]))
    elif op == "_npx_quantized_reshape":
        # (-2, -5, -6, 4, -1) on (3, 5, 4, 16): copy, merge two, split the last into 4 x 4
        assert tuple(attrs["newshape"]) == (-2, -5, -6, 4, -1) and ins[0].shape == (3, 5, 4, 16)
        res = oracle.quantized_reshape(ins[0], f(ins[1]), f(ins[2]), (3, 20, 4, 4))
    elif op == "_contrib_quantize_asym":
        res = oracle.quantize_asym(ins[0], *cal)
    elif op in ("_contrib_quantized_batch_norm", "_contrib_quantized_batch_norm_relu"):
        res = oracle.quantized_batch_norm(*ins[:5], f(ins[5]), f(ins[6]), *cal, eps=attrs["eps"],
                                          relu=op.endswith("_relu"))
    else:
        raise KeyError(op)
    return [np.asarray(v, np.float32).reshape(1) if np.ndim(v) == 0 else v for v in res]


def load(path=PATH):
    """[(operator, attrs, inputs, outputs)] from the committed file."""
    z = np.load(path, allow_pickle=False)
    index = json.loads(str(z["index"]))
    out = []
    for i, item in enumerate(index):
        ins = [z["c%d_in%d" % (i, j)] for j in range(item["n_in"])]
        outs = [z["c%d_out%d" % (i, j)] for j in range(item["n_out"])]
        out.append((item["op"], item["attrs"], ins, outs))
    return out


def main():
    arrays, index = {}, []
    for i, (op, attrs, ins) in enumerate(cases()):
        outs = run_oracle(op, attrs, ins)
        for j, a in enumerate(ins):
            arrays["c%d_in%d" % (i, j)] = a
        for j, a in enumerate(outs):
            arrays["c%d_out%d" % (i, j)] = np.asarray(a)
        index.append({"op": op, "attrs": attrs, "n_in": len(ins), "n_out": len(outs)})
    arrays["index"] = np.array(json.dumps(index))
    np.savez_compressed(PATH, **arrays)
    print("%d cases, %d bytes -> %s" % (len(index), os.path.getsize(PATH), PATH))


if __name__ == "__main__":
    main()
