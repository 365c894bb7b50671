"""quantize_model end to end on the GPU: float symbol + parameters -> calibrated int8
symbol + offline-quantized parameters -> executed through the registered operators.
Follows the reference's test_quantize_model (tests/python/quantization/test_quantization.py
:1172-1312: parameter names and types of the quantized model, calibration attributes on the
requantize nodes) and adds what the reference cannot check without a model zoo: the int8
network's output against the float network's, and the quantized prefix of the graph against
the CPU oracle, bit for bit."""
import numpy as np
import pytest
import torch

import oracle

pytestmark = pytest.mark.gpu


def build():
    from mxnet_amd import symbol as S
    data = S.Variable("data")
    conv = S.Convolution(data, kernel=(3, 3), pad=(1, 1), num_filter=16, name="conv")
    bn = S.BatchNorm(data=conv, eps=2e-05, fix_gamma=False, momentum=0.9,
                     use_global_stats=False, name="bn")
    act = S.Activation(data=bn, act_type="relu", name="relu")
    pool = S.Pooling(act, kernel=(4, 4), stride=(4, 4), pool_type="avg", name="pool")
    flat = S.Flatten(pool, name="flat")
    fc = S.FullyConnected(flat, num_hidden=10, flatten=True, name="fc")
    return S.softmax(fc, name="softmax")


def params(rng):
    arg = {"conv_weight": rng.normal(0, 0.2, (16, 4, 3, 3)), "conv_bias": rng.normal(0, 0.1, 16),
           "bn_gamma": rng.uniform(0.5, 1.5, 16), "bn_beta": rng.normal(0, 0.1, 16),
           "fc_weight": rng.normal(0, 0.1, (10, 16 * 2 * 2)), "fc_bias": rng.normal(0, 0.1, 10)}
    aux = {"bn_moving_mean": rng.normal(0, 0.1, 16), "bn_moving_var": rng.uniform(0.5, 1.5, 16)}
    f = lambda d: {k: torch.tensor(v, dtype=torch.float32) for k, v in d.items()}
    return f(arg), f(aux)


@pytest.mark.parametrize("calib_mode", ["naive", "entropy"])
@pytest.mark.parametrize("quantize_mode", ["full", "smart"])
def test_quantize_model_runs_and_tracks_the_float_network(calib_mode, quantize_mode):
    from mxnet_amd import quantization as Q
    from mxnet_amd.executor import Executor
    rng = np.random.default_rng(0)
    sym = build()
    arg, aux = params(rng)
    calib = [torch.tensor(rng.normal(0, 1, (16, 4, 8, 8)), dtype=torch.float32) for _ in range(3)]
    qsym, qarg, qaux = Q.quantize_model(sym, arg, aux, calib_mode=calib_mode, calib_data=calib,
                                        num_calib_batches=3, quantize_mode=quantize_mode)
    # parameters: int8 weights and biases with fp32 (1,) ranges; float ones untouched
    for name in ["conv_weight_quantize", "conv_bias_quantize", "fc_weight_quantize",
                 "fc_bias_quantize"]:
        assert qarg[name].dtype == torch.int8
        assert qarg[name + "_min"].shape == (1,) and qarg[name + "_min"].dtype == torch.float32
        assert qarg[name + "_min"].item() == -qarg[name + "_max"].item()
    assert qarg["conv_weight_quantize"].shape == (16, 4, 3, 3)
    assert torch.equal(qarg["bn_gamma"], arg["bn_gamma"]) and "conv_weight" not in qarg
    assert set(qsym.list_arguments()) - {"data"} == set(qarg.keys())
    # every requantize / quantize node got its calibrated range
    attrs = qsym.attr_dict()
    calibrated = [n for n in attrs if n.startswith("requantize_") or n.endswith("_quantize")]
    assert "requantize_conv" in calibrated and "requantize_fc" in calibrated
    for n in calibrated:
        assert "min_calib_range" in attrs[n] and "max_calib_range" in attrs[n]
        assert float(attrs[n]["min_calib_range"]) < float(attrs[n]["max_calib_range"])
    # the offline weights are exactly the oracle's v1 quantize of the float weights
    w = arg["conv_weight"].numpy()
    ref, rmin, rmax = oracle.quantize(w, w.min(), w.max(), "int8")
    np.testing.assert_array_equal(qarg["conv_weight_quantize"].cpu().numpy(), ref)
    assert qarg["conv_weight_quantize_max"].item() == rmax
    # run both networks on fresh data
    x = torch.tensor(rng.normal(0, 1, (32, 4, 8, 8)), dtype=torch.float32)
    fp = Executor(sym, {**arg, **aux}).forward(data=x)[0]
    q = Executor(qsym, {**qarg, **qaux}).forward(data=x)[0]
    assert q.shape == fp.shape == (32, 10) and q.dtype == torch.float32
    err = (q - fp).abs().max().item()
    assert err < 0.06, err
    assert (q.argmax(1) == fp.argmax(1)).float().mean().item() >= 0.85


def test_quantized_prefix_matches_the_oracle_bit_for_bit():
    """data -> quantize_v2 -> quantized_conv -> requantize -> dequantize against the
    oracle's functions with the same calibrated attributes."""
    from mxnet_amd import quantization as Q
    from mxnet_amd.executor import Executor
    rng = np.random.default_rng(1)
    sym = build()
    arg, aux = params(rng)
    calib = [torch.tensor(rng.normal(0, 1, (8, 4, 8, 8)), dtype=torch.float32)]
    qsym, qarg, qaux = Q.quantize_model(sym, arg, aux, calib_mode="naive", calib_data=calib,
                                        quantize_mode="full")
    internals = qsym.get_internals()
    head = internals["conv_dequantize_output"]
    x = rng.normal(0, 1, (5, 4, 8, 8)).astype(np.float32)
    got = Executor(head, {**qarg, **qaux}).forward(data=torch.from_numpy(x))[0].cpu().numpy()
    attrs = qsym.attr_dict()
    a = attrs["conv_data_quantize"]
    qd, dmin, dmax = oracle.quantize_v2(x, "int8", float(a["min_calib_range"]),
                                        float(a["max_calib_range"]))
    wq = qarg["conv_weight_quantize"].cpu().numpy()
    bq = qarg["conv_bias_quantize"].cpu().numpy()
    acc, omin, omax = oracle.quantized_conv(
        qd, wq, bq, dmin, dmax, qarg["conv_weight_quantize_min"].item(),
        qarg["conv_weight_quantize_max"].item(), qarg["conv_bias_quantize_min"].item(),
        qarg["conv_bias_quantize_max"].item(), stride=(1, 1), pad=(1, 1))
    r = attrs["requantize_conv"]
    q8, rmin, rmax = oracle.requantize(acc, omin, omax, float(r["min_calib_range"]),
                                       float(r["max_calib_range"]))
    want = oracle.dequantize(q8, rmin, rmax)
    np.testing.assert_array_equal(got, want)


def test_calibration_sees_every_requested_tensor():
    from mxnet_amd import quantization as Q
    from mxnet_amd.executor import Executor
    rng = np.random.default_rng(2)
    sym = build()
    arg, aux = params(rng)
    qsym, calib_layers = Q._quantize_symbol(sym, "gpu", offline_params=list(arg.keys()),
                                            quantize_mode="full")
    seen = []
    ex = Executor(sym, {**arg, **aux})
    ex.register_op_hook(lambda name, op, arr: seen.append(name), monitor_all=True)
    ex.forward(data=torch.tensor(rng.normal(0, 1, (2, 4, 8, 8)), dtype=torch.float32))
    assert set(calib_layers) <= set(seen)
    assert "conv_data" in seen and "conv_output" in seen and "bn_output" in seen


def build_residual():
    from mxnet_amd import symbol as S
    data = S.Variable("data")
    c1 = S.Convolution(data, kernel=(3, 3), pad=(1, 1), num_filter=16, name="conv1")
    r1 = S.Activation(c1, act_type="relu", name="relu1")
    c2 = S.Convolution(r1, kernel=(3, 3), pad=(1, 1), num_filter=16, name="conv2")
    add = S.elemwise_add(c2, r1, name="add")
    r2 = S.Activation(add, act_type="relu", name="relu2")
    c3 = S.Convolution(r2, kernel=(1, 1), num_filter=8, name="conv3")
    cat = S.Concat(c3, r1, name="cat")
    pool = S.Pooling(cat, kernel=(8, 8), global_pool=True, pool_type="avg", name="pool")
    flat = S.Flatten(pool, name="flat")
    return S.FullyConnected(flat, num_hidden=10, name="fc")


def test_residual_block_with_concat_stays_int8_end_to_end():
    """A residual sum and a concatenation between quantized convolutions: the int8 graph
    runs through _contrib_quantized_elemwise_add / _contrib_quantized_concat, tracks the
    float network, and the sum's output equals the oracle's on the tensors that reach it."""
    from mxnet_amd import quantization as Q
    from mxnet_amd.executor import Executor
    rng = np.random.default_rng(7)
    sym = build_residual()
    f = lambda v: torch.tensor(v, dtype=torch.float32)
    arg = {"conv1_weight": f(rng.normal(0, 0.2, (16, 4, 3, 3))), "conv1_bias": f(rng.normal(0, 0.1, 16)),
           "conv2_weight": f(rng.normal(0, 0.1, (16, 16, 3, 3))), "conv2_bias": f(rng.normal(0, 0.1, 16)),
           "conv3_weight": f(rng.normal(0, 0.2, (8, 16, 1, 1))), "conv3_bias": f(rng.normal(0, 0.1, 8)),
           "fc_weight": f(rng.normal(0, 0.2, (10, 24))), "fc_bias": f(rng.normal(0, 0.1, 10))}
    calib = [f(rng.normal(0, 1, (16, 4, 8, 8))) for _ in range(3)]
    qsym, qarg, qaux = Q.quantize_model(sym, arg, {}, calib_mode="naive", calib_data=calib,
                                        num_calib_batches=3, quantize_mode="full")
    ops = [op for op, _, _, _ in qsym.nodes() if op != "null"]
    assert ops.count("_contrib_quantized_elemwise_add") == 1
    assert ops.count("_contrib_quantized_concat") == 1
    # int8 from the first quantize to the last dequantize
    assert ops.count("_contrib_quantize_v2") == 1 and ops.count("_contrib_dequantize") == 1
    attrs = qsym.attr_dict()
    assert "min_calib_range" in attrs["requantize_add"]
    x = f(rng.normal(0, 1, (32, 4, 8, 8)))
    fp = Executor(sym, arg).forward(data=x)[0]
    q = Executor(qsym, {**qarg, **qaux}).forward(data=x)[0]
    assert q.shape == fp.shape == (32, 10)
    scale = fp.abs().max().item()
    assert (q - fp).abs().max().item() < 0.08 * scale
    # the sum itself against the oracle, on the operands the graph feeds it
    internals = qsym.get_internals()
    from mxnet_amd import symbol as S
    probe = S.Group([internals["requantize_conv2_output0"], internals["requantize_conv2_output1"],
                     internals["requantize_conv2_output2"], internals["quantized_relu1_output"],
                     internals["quantized_relu1_min_output"], internals["quantized_relu1_max_output"],
                     internals["quantized_add_output"], internals["quantized_add_min_output"],
                     internals["quantized_add_max_output"]])
    a, amin, amax, b, bmin, bmax, s, smin, smax = [
        t.cpu().numpy() for t in Executor(probe, {**qarg, **qaux}).forward(data=x)]
    ref, rmin, rmax = oracle.quantized_elemwise_add(a, b, amin[0], amax[0], bmin[0], bmax[0])
    np.testing.assert_array_equal(s, ref)
    assert smin[0] == rmin and smax[0] == rmax


def build_attention_like():
    from mxnet_amd import symbol as S
    d = S.Variable("data")
    emb = S.Embedding(d, input_dim=200, output_dim=32, name="emb")
    fc1 = S.FullyConnected(emb, num_hidden=32, flatten=False, name="fc1")
    rs = S.Reshape(fc1, shape=(0, 0, 4, 8), name="rs")
    tr = S.transpose(rs, axes=(0, 2, 1, 3), name="tr")
    mul = S.elemwise_mul(tr, tr, name="mul")
    return S.FullyConnected(mul, num_hidden=10, name="fc2")


def test_embedding_transpose_mul_network_stays_int8_end_to_end():
    """Token ids -> int8 embedding rows -> FC -> reshape -> transpose -> element-wise product
    -> FC, all through the quantized operators; tracks the float network, and the byte movers'
    outputs equal the oracle's on the tensors that reach them."""
    from mxnet_amd import quantization as Q
    from mxnet_amd import symbol as S
    from mxnet_amd.executor import Executor
    rng = np.random.default_rng(17)
    sym = build_attention_like()
    f = lambda v: torch.tensor(v, dtype=torch.float32)
    arg = {"emb_weight": f(rng.normal(0, 1.0, (200, 32))),
           "fc1_weight": f(rng.normal(0, 0.2, (32, 32))), "fc1_bias": f(rng.normal(0, 0.1, 32)),
           "fc2_weight": f(rng.normal(0, 0.05, (10, 4 * 12 * 8))), "fc2_bias": f(rng.normal(0, 0.1, 10))}
    calib = [f(rng.integers(0, 200, (16, 12))) for _ in range(3)]
    qsym, qarg, qaux = Q.quantize_model(sym, arg, {}, calib_mode="naive", calib_data=calib,
                                        num_calib_batches=3, quantize_mode="full")
    ops = [op for op, _, _, _ in qsym.nodes() if op != "null"]
    for name in ["_contrib_quantized_embedding", "_contrib_quantized_reshape",
                 "_contrib_quantized_transpose", "_contrib_quantized_elemwise_mul"]:
        assert ops.count(name) == 1
    assert "_contrib_quantize_v2" not in ops and ops.count("_contrib_dequantize") == 1
    assert qarg["emb_weight_quantize"].dtype == torch.int8
    attrs = qsym.attr_dict()
    assert "min_calib_range" in attrs["requantize_mul"]
    x = f(rng.integers(0, 200, (32, 12)))
    fp = Executor(sym, arg).forward(data=x)[0]
    q = Executor(qsym, {**qarg, **qaux}).forward(data=x)[0]
    assert q.shape == fp.shape == (32, 10)
    assert (q - fp).abs().max().item() < 0.1 * fp.abs().max().item()
    internals = qsym.get_internals()
    names = ["quantized_emb_output", "requantize_fc1_output0", "requantize_fc1_output1",
             "requantize_fc1_output2", "quantized_rs_output", "quantized_tr_output",
             "quantized_tr_min_output", "quantized_tr_max_output", "quantized_mul_output0",
             "quantized_mul_output1", "quantized_mul_output2"]
    emb, h, hmin, hmax, rs, tr, trmin, trmax, mul, mulmin, mulmax = [
        t.cpu().numpy() for t in Executor(S.Group([internals[n] for n in names]),
                                          {**qarg, **qaux}).forward(data=x)]
    w8 = qarg["emb_weight_quantize"].cpu().numpy()
    np.testing.assert_array_equal(emb, w8[x.cpu().numpy().astype(np.int64)])
    np.testing.assert_array_equal(rs, h.reshape(32, 12, 4, 8))
    ref, rmin, rmax = oracle.quantized_transpose(rs, hmin[0], hmax[0], (0, 2, 1, 3))
    np.testing.assert_array_equal(tr, ref)
    assert (trmin[0], trmax[0]) == (rmin, rmax)
    ref, rmin, rmax = oracle.quantized_elemwise_mul(tr, tr, trmin[0], trmax[0], trmin[0], trmax[0])
    np.testing.assert_array_equal(mul, ref)
    assert (mulmin[0], mulmax[0]) == (rmin, rmax)


@pytest.mark.parametrize("calib_mode", ["naive", "entropy"])
def test_quantize_graph_then_calib_graph_equals_quantize_model(calib_mode):
    """The two-step API (python/mxnet/contrib/quantization.py:613-796): quantize_graph hands
    back a collector, the caller runs calibration batches through the float network with the
    collector as the monitor callback, calib_graph finishes; symbol and parameters are those of
    the one-step quantize_model on the same batches."""
    from mxnet_amd import quantization as Q
    from mxnet_amd.executor import Executor
    rng = np.random.default_rng(3)
    sym = build()
    arg, aux = params(rng)
    calib = [torch.tensor(rng.normal(0, 1, (8, 4, 8, 8)), dtype=torch.float32) for _ in range(2)]
    want_sym, want_arg, _ = Q.quantize_model(sym, arg, aux, calib_mode=calib_mode,
                                             calib_data=calib, num_calib_batches=2,
                                             quantize_mode="full")
    qsym, qarg, qaux, collector, calib_layers = Q.quantize_graph(
        sym, arg, aux, calib_mode=calib_mode, quantize_mode="full")
    assert collector.include_layers == calib_layers and qaux is aux
    assert "min_calib_range" not in qsym.tojson()
    ex = Executor(sym, {**arg, **aux})
    ex.register_op_hook(collector.collect, monitor_all=True)
    for batch in calib:
        ex.forward(data=batch)
    csym, carg, caux = Q.calib_graph(qsym, arg, aux, collector, calib_mode=calib_mode)
    assert csym.tojson() == want_sym.tojson()
    assert set(carg.keys()) == set(want_arg.keys())
    for k in carg:
        assert torch.equal(carg[k].cpu(), want_arg[k].cpu()), k
    with pytest.raises(ValueError, match="calibration mode"):
        Q.calib_graph(qsym, arg, aux, collector, calib_mode="none")

    class Custom(Q.CalibrationCollector):
        def collect(self, name, op_name, arr):
            if name in self.include_layers:
                self.min_max_dict[name] = (-1.0, 1.0)

    custom = Custom()
    _, _, _, got, layers = Q.quantize_graph(sym, arg, aux, calib_mode="custom",
                                            LayerOutputCollector=custom)
    assert got is custom and custom.include_layers == layers
    with pytest.raises(ValueError, match="CalibrationCollector"):
        Q.quantize_graph(sym, arg, aux, calib_mode="custom", LayerOutputCollector=object())
    assert Q.quantize_graph(sym, arg, aux, calib_mode="none")[3] is None
    with pytest.raises(ValueError, match="quantized_dtype"):
        Q.quantize_graph(sym, arg, aux, quantized_dtype="int4")
