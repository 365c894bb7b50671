"""The QuantizeGraph / SetCalibTable passes, the symbol JSON reader/writer and entropy
calibration on the CPU (no kernel runs).  Expectations come from the reference's pass
(src/operator/quantization/quantize_graph_pass.cc) worked by hand on small graphs and from
its own tests (tests/python/quantization/test_quantization.py:1092-1115 test_quantize_params,
:1365-1399 test_quantize_sym_with_calib, :1451-1493 the optimal-threshold tests)."""
import json

import numpy as np
import pytest

from mxnet_amd import quantization as Q
from mxnet_amd import symbol as S
from mxnet_amd.operator import MXNetError


def fp32_sym():
    # get_fp32_sym of test_quantize_sym_with_calib
    data = S.Variable("data")
    conv = S.Convolution(data, kernel=(1, 1), num_filter=16, name="conv")
    bn = S.BatchNorm(data=conv, eps=2e-05, fix_gamma=False, momentum=0.9,
                     use_global_stats=False, name="bn")
    act = S.Activation(data=bn, act_type="relu", name="relu")
    pool = S.Pooling(act, kernel=(4, 4), pool_type="avg", name="pool")
    fc = S.FullyConnected(pool, num_hidden=10, flatten=True, name="fc")
    return S.softmax(fc, name="softmax")


def offline_of(sym):
    return [n for n in sym.list_arguments() if not n.startswith("data") and not n.endswith("label")]


def ops_of(sym):
    return [(op, name) for op, name, _, _ in sym.nodes() if op != "null"]


def node(sym, name):
    nodes = sym.nodes()
    for op, n, attrs, inputs in nodes:
        if n == name:
            return op, attrs, [(nodes[j][1], k) for j, k in inputs]
    raise KeyError(name)


def test_symbol_composition_and_json_round_trip():
    sym = fp32_sym()
    assert sym.list_arguments() == ["data", "conv_weight", "conv_bias", "bn_gamma", "bn_beta",
                                    "fc_weight", "fc_bias"]
    assert sym.list_auxiliary_states() == ["bn_moving_mean", "bn_moving_var"]
    assert sym.list_outputs() == ["softmax_output"]
    text = sym.tojson()
    g = json.loads(text)
    assert [n["name"] for n in g["nodes"]][:4] == ["data", "conv_weight", "conv_bias", "conv"]
    assert g["nodes"][3]["attrs"] == {"kernel": "(1, 1)", "num_filter": "16"}
    assert g["nodes"][3]["inputs"] == [[0, 0, 0], [1, 0, 0], [2, 0, 0]]
    assert g["arg_nodes"] == [i for i, n in enumerate(g["nodes"]) if n["op"] == "null"]
    # BatchNorm has three outputs: node_row_ptr advances by 3 over it
    bn = [n["name"] for n in g["nodes"]].index("bn")
    assert g["node_row_ptr"][bn + 1] - g["node_row_ptr"][bn] == 3
    assert g["heads"] == [[len(g["nodes"]) - 1, 0, 0]]
    assert S.Symbol.fromjson(text).tojson() == text
    # files written by old versions keep attributes under "param" / "attr"
    old = json.loads(text)
    for n in old["nodes"]:
        if "attrs" in n:
            n["param"] = n.pop("attrs")
    assert S.Symbol.fromjson(json.dumps(old)).tojson() == text
    with pytest.raises(MXNetError, match="symbol JSON"):
        S.Symbol.fromjson('{"nodes": [], "heads": [[3, 0, 0]]}').tojson()


def test_quantize_full_mode_graph():
    sym = fp32_sym()
    qsym, calib = Q._quantize_symbol(sym, "gpu", offline_params=offline_of(sym),
                                     quantize_mode="full")
    assert ops_of(qsym) == [
        ("_contrib_quantize_v2", "conv_data_quantize"),
        ("_contrib_quantized_conv", "quantized_conv"),
        ("_contrib_requantize", "requantize_conv"),
        ("_contrib_dequantize", "conv_dequantize"),
        ("BatchNorm", "bn"),
        ("_contrib_quantize_v2", "bn_output_quantize"),
        ("_contrib_quantized_act", "quantized_relu"),
        ("_contrib_quantized_pooling", "quantized_pool"),
        ("_contrib_quantized_fully_connected", "quantized_fc"),
        ("_contrib_requantize", "requantize_fc"),
        ("_contrib_dequantize", "fc_dequantize"),
        ("softmax", "softmax")]
    # data inputs first, then (min, max) per input in input order
    op, attrs, inputs = node(qsym, "quantized_conv")
    assert attrs == {"kernel": "(1, 1)", "num_filter": "16"}
    assert inputs == [("conv_data_quantize", 0), ("conv_weight_quantize", 0),
                      ("conv_bias_quantize", 0), ("conv_data_quantize", 1),
                      ("conv_data_quantize", 2), ("conv_weight_quantize_min", 0),
                      ("conv_weight_quantize_max", 0), ("conv_bias_quantize_min", 0),
                      ("conv_bias_quantize_max", 0)]
    assert node(qsym, "requantize_conv")[1:] == ({"out_type": "int8"},
                                                 [("quantized_conv", 0), ("quantized_conv", 1),
                                                  ("quantized_conv", 2)])
    assert node(qsym, "conv_dequantize")[2] == [("requantize_conv", 0), ("requantize_conv", 1),
                                                ("requantize_conv", 2)]
    assert node(qsym, "bn")[2][0] == ("conv_dequantize", 0)
    # int8 flows from relu through pooling into the FC without leaving int8
    assert node(qsym, "quantized_relu")[2] == [("bn_output_quantize", 0),
                                               ("bn_output_quantize", 1),
                                               ("bn_output_quantize", 2)]
    assert node(qsym, "quantized_pool")[2] == [("quantized_relu", 0), ("quantized_relu", 1),
                                               ("quantized_relu", 2)]
    assert node(qsym, "quantized_fc")[2][:5] == [("quantized_pool", 0), ("fc_weight_quantize", 0),
                                                 ("fc_bias_quantize", 0), ("quantized_pool", 1),
                                                 ("quantized_pool", 2)]
    assert node(qsym, "softmax")[2] == [("fc_dequantize", 0)]
    assert calib == ["conv_data", "conv_output", "bn_output", "fc_output"]
    assert qsym.list_outputs() == ["softmax_output"]


def test_quantize_smart_mode_keeps_isolated_supporting_ops_float():
    sym = fp32_sym()
    qsym, calib = Q._quantize_symbol(sym, "gpu", offline_params=offline_of(sym),
                                     quantize_mode="smart")
    names = [n for _, n in ops_of(qsym)]
    # relu and pool sit between a float BatchNorm and the FC: int8 does not reach them
    # from a must-quantize producer, so they stay float
    assert names == ["conv_data_quantize", "quantized_conv", "requantize_conv",
                     "conv_dequantize", "bn", "relu", "pool", "pool_output_quantize",
                     "quantized_fc", "requantize_fc", "fc_dequantize", "softmax"]
    assert calib == ["conv_data", "conv_output", "pool_output", "fc_output"]
    # conv -> relu -> conv: the relu is between two must-quantize nodes and goes int8
    d = S.Variable("data")
    c1 = S.Convolution(d, kernel=(3, 3), num_filter=8, name="c1")
    r = S.Activation(c1, act_type="relu", name="r")
    c2 = S.Convolution(r, kernel=(3, 3), num_filter=8, name="c2")
    q2, calib2 = Q._quantize_symbol(c2, "gpu", offline_params=offline_of(c2),
                                    quantize_mode="smart")
    assert [n for _, n in ops_of(q2)] == ["c1_data_quantize", "quantized_c1", "requantize_c1",
                                          "quantized_r", "quantized_c2", "requantize_c2",
                                          "c2_dequantize"]
    assert node(q2, "quantized_c2")[2][0] == ("quantized_r", 0)
    assert node(q2, "quantized_c2")[2][3:5] == [("quantized_r", 1), ("quantized_r", 2)]
    assert calib2 == ["c1_data", "c1_output", "c2_output"]
    assert q2.list_outputs() == ["c2_dequantize_output"]
    with pytest.raises(MXNetError, match="unrecognized quantize mode"):
        Q._quantize_symbol(c2, "gpu", quantize_mode="clever")


def test_exclusions_and_device():
    sym = fp32_sym()
    off = offline_of(sym)
    # the reference's GPU build has no quantized relu / flatten kernels; excluding the
    # float operators reproduces its graph
    qsym, calib = Q._quantize_symbol(sym, "gpu", offline_params=off, quantize_mode="full",
                                     excluded_operators=["Activation", "Flatten"])
    assert [n for _, n in ops_of(qsym)] == [
        "conv_data_quantize", "quantized_conv", "requantize_conv", "conv_dequantize", "bn",
        "relu", "relu_output_quantize", "quantized_pool", "quantized_fc", "requantize_fc",
        "fc_dequantize", "softmax"]
    assert calib == ["conv_data", "conv_output", "relu_output", "fc_output"]
    qsym, _ = Q._quantize_symbol(sym, "gpu", offline_params=off, quantize_mode="full",
                                 excluded_symbols=["conv"])
    assert ("Convolution", "conv") in ops_of(qsym)
    assert "conv_weight" in qsym.list_arguments()
    # no quantized operator has a cpu kernel in this build: nothing is replaced
    qsym, calib = Q._quantize_symbol(sym, "cpu", offline_params=off, quantize_mode="full")
    assert ops_of(qsym) == ops_of(sym) and calib == []
    # non-relu activations and sum pooling have no quantized counterpart
    d = S.Variable("data")
    t = S.Activation(S.Convolution(d, kernel=(1, 1), num_filter=4, name="c"), act_type="tanh",
                     name="t")
    qsym, _ = Q._quantize_symbol(t, "gpu", quantize_mode="full")
    assert ops_of(qsym)[-2:] == [("_contrib_dequantize", "c_dequantize"), ("Activation", "t")]
    with pytest.raises(MXNetError, match="channel-wise"):
        Q._quantize_symbol(sym, "gpu", quantize_granularity="channel-wise")


def test_weights_quantized_online_when_not_offline():
    d = S.Variable("data")
    fc = S.FullyConnected(d, num_hidden=4, no_bias=True, name="fc")
    qsym, calib = Q._quantize_symbol(fc, "gpu", quantize_mode="full")
    assert [n for _, n in ops_of(qsym)] == ["fc_data_quantize", "fc_weight_quantize",
                                            "quantized_fc", "requantize_fc", "fc_dequantize"]
    assert node(qsym, "fc_weight_quantize")[2] == [("fc_weight", 0)]
    assert node(qsym, "quantized_fc")[2] == [("fc_data_quantize", 0), ("fc_weight_quantize", 0),
                                             ("fc_data_quantize", 1), ("fc_data_quantize", 2),
                                             ("fc_weight_quantize", 1), ("fc_weight_quantize", 2)]
    assert calib == ["fc_data", "fc_weight", "fc_output"]


def test_shared_float_producer_gets_one_quantize_node():
    d = S.Variable("data")
    bn = S.BatchNorm(d, name="bn")
    a = S.FullyConnected(bn, num_hidden=4, no_bias=True, name="a")
    b = S.FullyConnected(bn, num_hidden=4, no_bias=True, name="b")
    out = S.elemwise_add(a, b, name="sum")
    qsym, calib = Q._quantize_symbol(out, "gpu", offline_params=["a_weight", "b_weight"],
                                     quantize_mode="full", excluded_operators=["elemwise_add"])
    names = [n for _, n in ops_of(qsym)]
    assert names.count("bn_output_quantize") == 1
    assert node(qsym, "quantized_a")[2][0] == ("bn_output_quantize", 0)
    assert node(qsym, "quantized_b")[2][0] == ("bn_output_quantize", 0)
    assert node(qsym, "sum")[2] == [("a_dequantize", 0), ("b_dequantize", 0)]
    assert calib == ["bn_output", "a_output", "b_output"]
    # with the sum quantized as well the graph leaves int8 only at its head
    qsym, calib = Q._quantize_symbol(out, "gpu", offline_params=["a_weight", "b_weight"],
                                     quantize_mode="full")
    assert [n for _, n in ops_of(qsym)][-3:] == ["quantized_sum", "requantize_sum",
                                                 "sum_dequantize"]
    assert node(qsym, "quantized_sum")[2][:2] == [("requantize_a", 0), ("requantize_b", 0)]
    assert calib == ["bn_output", "a_output", "b_output", "sum_output"]


def test_quantize_params_names():
    # test_quantize_params: conv + bn, every non-data argument offline
    data = S.Variable("data")
    conv = S.Convolution(data, kernel=(1, 1), num_filter=2048, name="conv")
    sym = S.BatchNorm(data=conv, eps=2e-05, fix_gamma=False, momentum=0.9,
                      use_global_stats=False, name="bn")
    qsym, _ = Q._quantize_symbol(sym, "gpu", offline_params=offline_of(sym), quantize_mode="full")
    args = qsym.list_arguments()
    assert [a for a in args if a.startswith("conv")] == [
        "conv_weight_quantize", "conv_bias_quantize", "conv_weight_quantize_min",
        "conv_weight_quantize_max", "conv_bias_quantize_min", "conv_bias_quantize_max"]
    assert [a for a in args if a.startswith("bn")] == ["bn_gamma", "bn_beta"]


def test_set_calib_table():
    # test_quantize_sym_with_calib
    sym = fp32_sym()
    qsym, _ = Q._quantize_symbol(sym, "gpu", offline_params=offline_of(sym), quantize_mode="full")
    rng = np.random.default_rng(0)
    table = {"conv_output": (rng.uniform(100.0, 200.0), rng.uniform(100.0, 200.0)),
             "fc_output": (rng.uniform(100.0, 200.0), rng.uniform(100.0, 200.0)),
             "conv_data": (-1.5, 2.5), "bn_output": (-0.25, 7.0), "unused_output": (0.0, 1.0)}
    cqsym = Q._calibrate_quantized_sym(qsym, table)
    attrs = cqsym.attr_dict()
    for name, key in [("requantize_conv", "conv_output"), ("requantize_fc", "fc_output"),
                      ("conv_data_quantize", "conv_data"), ("bn_output_quantize", "bn_output")]:
        np.testing.assert_allclose(float(attrs[name]["min_calib_range"]), table[key][0],
                                   rtol=1e-6, atol=1e-6)
        np.testing.assert_allclose(float(attrs[name]["max_calib_range"]), table[key][1],
                                   rtol=1e-3, atol=1e-4)
    # std::to_string(float) spelling, as the operators' parsers receive it
    assert attrs["conv_data_quantize"]["min_calib_range"] == "-1.500000"
    assert ops_of(cqsym) == ops_of(qsym)
    assert Q._calibrate_quantized_sym(qsym, {}) is qsym


def test_optimal_threshold_adversarial_case():
    # all mass in the last bin: the threshold must be the maximum
    hist = [0] * 998 + [1000]
    min_val, max_val = -2, 2
    edges = [(max_val - min_val) / 999 * i + min_val for i in range(999)] + [max_val]
    hist_data = (hist, edges, min_val, max_val, max_val)
    for dtype in ["uint8", "int8", "auto"]:
        res = Q._LayerHistogramCollector.get_optimal_threshold(hist_data, dtype,
                                                               num_quantized_bins=5)
        assert abs(res[2] - 2) < 1e-5


def test_get_optimal_thresholds_uniform():
    # uniform data: the best threshold is (close to) the largest magnitude
    rng = np.random.default_rng(3)
    for dtype in ["uint8", "int8", "auto"]:
        arr = rng.uniform(-10.532, 11.3432, size=(8, 3, 23, 23))
        lo, hi = arr.min(), arr.max()
        th = max(abs(lo), abs(hi))
        hist, edges = np.histogram(arr, bins=8001, range=(-th, th))
        out = Q._LayerHistogramCollector.get_optimal_thresholds(
            {"layer1": (hist, edges, lo, hi, th)}, dtype)
        assert out["layer1"][0] == -out["layer1"][1]
        np.testing.assert_allclose(out["layer1"][1], th, rtol=1e-2, atol=1e-4)


def kl_threshold_numpy(hist, edges, nq):
    """Independent float64 evaluation of the same search with scipy's entropy."""
    from scipy.stats import entropy
    hist = np.asarray(hist, dtype=np.float64)
    nb = hist.size
    zero = nb // 2
    best = (np.inf, None)

    def smooth(p, eps=0.0001):
        z = p == 0
        nz = p.size - z.sum()
        if nz == 0:
            return None
        eps1 = eps * z.sum() / nz
        if eps1 >= 1:
            return None
        return p + eps * z - eps1 * (~z)

    for i in range(nq // 2, zero + 1):
        start, stop = zero - i, zero + i + 1
        sliced = hist[start:stop].copy()
        p = sliced.copy()
        p[0] = hist[:start + 1].sum()
        p[-1] = hist[stop - 1:].sum()
        sliced[0] = 0  # the reference leaves the first kept bin out of the merged levels
        merged = sliced.size // nq
        q = np.zeros_like(sliced)
        for j in range(nq):
            lo = j * merged
            hi = sliced.size if j == nq - 1 else (j + 1) * merged
            level = sliced[lo:hi].sum()
            nonempty = (sliced[lo:hi] != 0).sum()
            if nonempty:
                q[lo:hi] = np.where(p[lo:hi] != 0, level / nonempty, 0)
        ps, qs = smooth(p), smooth(q)
        d = np.inf if qs is None else entropy(ps, qs)
        if d < best[0]:
            best = (d, edges[stop])
    return best[1], best[0]


def test_entropy_against_float64_search():
    rng = np.random.default_rng(7)
    arr = np.concatenate([rng.standard_normal(200000), rng.uniform(-9, 9, 300)])
    th = np.abs(arr).max()
    for bins, nq in [(2001, 255), (801, 127)]:
        hist, edges = np.histogram(arr, bins=bins, range=(-th, th))
        got_th, got_div = Q.calibrate_entropy(hist, edges, nq)
        want_th, want_div = kl_threshold_numpy(hist, edges, nq)
        # binary32 vs binary64 accumulation: the divergence agrees to a few digits and the
        # chosen threshold is the same candidate or a neighbour with an equal divergence
        np.testing.assert_allclose(got_div, want_div, rtol=2e-3)
        step = edges[1] - edges[0]
        assert abs(got_th - want_th) <= 2 * step + 1e-6


def test_histogram_collector_merges_batches():
    c = Q._LayerHistogramCollector("int8", num_bins=11, include_layers=["x"])
    import torch
    c.collect("x", "op", torch.tensor([-1.0, 0.0, 0.5, 1.0]))
    c.collect("ignored", "op", torch.tensor([100.0]))
    hist, edges, lo, hi, th = c.hist_dict["x"]
    assert hist.sum() == 4 and th == 1.0 and len(hist) == 11
    c.collect("x", "op", torch.tensor([0.25, -0.25]))        # inside the old range
    assert c.hist_dict["x"][0].sum() == 6 and c.hist_dict["x"][4] == 1.0
    c.collect("x", "op", torch.tensor([2.0, -0.1]))          # widens by whole old bins
    hist, edges, lo, hi, th = c.hist_dict["x"]
    assert hist.sum() == 8 and len(hist) % 2 == 1 and th >= 2.0 and (lo, hi) == (-1.0, 2.0)
    old_step = 2.0 / 11
    np.testing.assert_allclose(edges[1] - edges[0], old_step, rtol=1e-5)
    assert "ignored" not in c.hist_dict
    m = Q._LayerOutputMinMaxCollector("int8", include_layers=["x"])
    m.collect("x", "op", torch.tensor([-1.0, 3.0]))
    m.collect("x", "op", torch.tensor([-2.0, 1.0]))
    assert m.post_collect() == {"x": (-2.0, 3.0)}


def test_merged_histogram_equals_one_histogram_of_all_batches():
    """Bins of width 1 with values on a quarter grid: every edge is exact in binary, so
    growing by whole bins and counting batch by batch must give exactly the counts of one
    histogram of everything over the final range (quantization.py:295-329 of the
    reference)."""
    rng = np.random.default_rng(3)
    grid = lambda reach, n: (rng.integers(-4 * reach, 4 * reach, n) + 0.5) / 4.0
    first = np.concatenate([grid(2, 50), [2.5]]).astype(np.float32)      # th 2.5, 5 bins
    inside = grid(2, 30).astype(np.float32)
    beyond = np.concatenate([grid(4, 40), [-4.25]]).astype(np.float32)   # reach 4.25
    h = Q._LayerHistogramCollector("int8", num_bins=5, include_layers=["t"])
    for batch in (first, inside, beyond):
        h.collect("t", "op", batch)
    hist, edges, lo, hi, th = h.hist_dict["t"]
    # margin = floor((4.25 - 2.5) / 1) + 1 = 2 bins a side
    assert th == 4.5 and len(hist) == 9
    everything = np.concatenate([first, inside, beyond])
    want, want_edges = np.histogram(everything, bins=9, range=(-4.5, 4.5))
    # the first batch's own maximum (2.5) sat on the closed top edge of its histogram and
    # keeps that bin; counted in one go it would open the next one
    want[6] += 1
    want[7] -= 1
    np.testing.assert_array_equal(hist, want)
    np.testing.assert_array_equal(edges, want_edges)
    assert lo == everything.min() and hi == everything.max()
    # the static form the reference's callers use gives the same tuple
    t = Q._LayerHistogramCollector.combine_histogram(
        (np.array([1, 2, 3]), np.linspace(-1.5, 1.5, 4), -1.25, 1.25, 1.5),
        np.array([2.75, -0.25]), -0.25, 2.75, 2.75)
    np.testing.assert_array_equal(t[0], [0, 0, 1, 3, 3, 0, 1])
    assert t[2:] == (-1.25, 2.75, 3.5)


def test_residual_add_and_concat_stay_int8():
    """elemwise_add (quantized_elemwise_add.cc:124-133, FNeedRequantize) and Concat
    (quantized_concat.cc:143-152): data inputs first, then one (min, max) pair per input in
    input order, as quantize_graph_pass.cc wires every quantized operator."""
    d = S.Variable("data")
    c1 = S.Convolution(d, kernel=(3, 3), pad=(1, 1), num_filter=16, name="conv1")
    r1 = S.Activation(c1, act_type="relu", name="relu1")
    c2 = S.Convolution(r1, kernel=(3, 3), pad=(1, 1), num_filter=16, name="conv2")
    add = S.elemwise_add(c2, r1, name="add")
    c3 = S.Convolution(add, kernel=(1, 1), num_filter=8, name="conv3")
    cat = S.Concat(c3, r1, name="cat")
    fc = S.FullyConnected(cat, num_hidden=10, name="fc")
    assert node(fc, "cat")[1] == {"dim": "1", "num_args": "2"}
    qsym, calib = Q._quantize_symbol(fc, "gpu", offline_params=offline_of(fc),
                                     quantize_mode="full")
    assert [o for o in ops_of(qsym) if o[0] != "_contrib_quantized_conv"] == [
        ("_contrib_quantize_v2", "conv1_data_quantize"),
        ("_contrib_requantize", "requantize_conv1"),
        ("_contrib_quantized_act", "quantized_relu1"),
        ("_contrib_requantize", "requantize_conv2"),
        ("_contrib_quantized_elemwise_add", "quantized_add"),
        ("_contrib_requantize", "requantize_add"),
        ("_contrib_requantize", "requantize_conv3"),
        ("_contrib_quantized_concat", "quantized_cat"),
        ("_contrib_quantized_fully_connected", "quantized_fc"),
        ("_contrib_requantize", "requantize_fc"),
        ("_contrib_dequantize", "fc_dequantize")]
    assert node(qsym, "quantized_add")[2] == [
        ("requantize_conv2", 0), ("quantized_relu1", 0), ("requantize_conv2", 1),
        ("requantize_conv2", 2), ("quantized_relu1", 1), ("quantized_relu1", 2)]
    assert node(qsym, "requantize_add")[2] == [("quantized_add", 0), ("quantized_add", 1),
                                               ("quantized_add", 2)]
    assert node(qsym, "quantized_cat")[1:] == (
        {"dim": "1", "num_args": "2"},
        [("requantize_conv3", 0), ("quantized_relu1", 0), ("requantize_conv3", 1),
         ("requantize_conv3", 2), ("quantized_relu1", 1), ("quantized_relu1", 2)])
    assert node(qsym, "quantized_fc")[2][0] == ("quantized_cat", 0)
    assert calib == ["conv1_data", "conv1_output", "conv2_output", "add_output", "conv3_output",
                     "fc_output"]
    # the calibrated range of the sum lands on its requantize node
    cq = Q._calibrate_quantized_sym(qsym, {"add_output": (-3.0, 5.0)})
    assert node(cq, "requantize_add")[1] == {"out_type": "int8", "min_calib_range": "-3",
                                             "max_calib_range": "5"} or \
        float(node(cq, "requantize_add")[1]["max_calib_range"]) == 5.0
    # the reference's GPU registry has neither operator: excluding them reproduces its graph
    gsym, _ = Q._quantize_symbol(fc, "gpu", offline_params=offline_of(fc), quantize_mode="full",
                                 excluded_operators=["elemwise_add", "Concat"])
    names = [n for _, n in ops_of(gsym)]
    assert "add" in names and "cat" in names and "quantized_add" not in names


def attention_like():
    d = S.Variable("data")
    emb = S.Embedding(d, input_dim=100, output_dim=16, name="emb")
    fc1 = S.FullyConnected(emb, num_hidden=16, flatten=False, name="fc1")
    rs = S.Reshape(fc1, shape=(0, 0, 4, 4), name="rs")
    tr = S.transpose(rs, axes=(0, 2, 1, 3), name="tr")
    mul = S.elemwise_mul(tr, tr, name="mul")
    return S.FullyConnected(mul, num_hidden=8, name="fc2")


def test_embedding_reshape_transpose_and_mul_stay_int8():
    """Embedding (quantized_indexing_op.cc:162-190: its indices are never quantized, its table
    is quantized offline), Reshape (quantized_reshape.cc:119-127), transpose
    (quantized_transpose.cc:106-115) and elemwise_mul (quantized_elemwise_mul.cc:247-256,
    FNeedRequantize) between two fully-connected layers."""
    sym = attention_like()
    offline = [n for n in sym.list_arguments() if n != "data"]
    assert offline == ["emb_weight", "fc1_weight", "fc1_bias", "fc2_weight", "fc2_bias"]
    qsym, calib = Q._quantize_symbol(sym, "gpu", offline_params=offline, quantize_mode="full")
    assert ops_of(qsym) == [
        ("_contrib_quantized_embedding", "quantized_emb"),
        ("_contrib_quantized_fully_connected", "quantized_fc1"),
        ("_contrib_requantize", "requantize_fc1"),
        ("_contrib_quantized_reshape", "quantized_rs"),
        ("_contrib_quantized_transpose", "quantized_tr"),
        ("_contrib_quantized_elemwise_mul", "quantized_mul"),
        ("_contrib_requantize", "requantize_mul"),
        ("_contrib_quantized_fully_connected", "quantized_fc2"),
        ("_contrib_requantize", "requantize_fc2"),
        ("_contrib_dequantize", "fc2_dequantize")]
    # token ids go in as they are; the table and its range are the offline-quantized variables
    assert node(qsym, "quantized_emb")[1:] == (
        {"input_dim": "100", "output_dim": "16"},
        [("data", 0), ("emb_weight_quantize", 0), ("emb_weight_quantize_min", 0),
         ("emb_weight_quantize_max", 0)])
    assert node(qsym, "quantized_fc1")[2][0] == ("quantized_emb", 0)
    assert node(qsym, "quantized_fc1")[2][3:5] == [("quantized_emb", 1), ("quantized_emb", 2)]
    assert node(qsym, "quantized_rs")[1:] == (
        {"shape": "(0, 0, 4, 4)"},
        [("requantize_fc1", 0), ("requantize_fc1", 1), ("requantize_fc1", 2)])
    assert node(qsym, "quantized_tr")[1:] == (
        {"axes": "(0, 2, 1, 3)"},
        [("quantized_rs", 0), ("quantized_rs", 1), ("quantized_rs", 2)])
    assert node(qsym, "quantized_mul")[2] == [
        ("quantized_tr", 0), ("quantized_tr", 0), ("quantized_tr", 1), ("quantized_tr", 2),
        ("quantized_tr", 1), ("quantized_tr", 2)]
    # elemwise_mul registers no output names, float or quantized: its tensor is "<name>_0"
    # (common::GetOutputName, src/common/utils.h) on both sides of the calibration table
    assert calib == ["fc1_output", "mul_0", "fc2_output"]
    cq = Q._calibrate_quantized_sym(qsym, {"mul_0": (-3.0, 5.0), "mul_output": (-9.0, 9.0)})
    assert float(node(cq, "requantize_mul")[1]["max_calib_range"]) == 5.0
    assert "emb_weight_quantize" in qsym.list_arguments() and "emb_weight" not in \
        qsym.list_arguments()
    # an int32 Embedding table is not a float32 one: the node stays as it is
    d = S.Variable("data")
    e32 = S.Embedding(d, input_dim=10, output_dim=4, dtype="int32", name="emb")
    fc = S.FullyConnected(e32, num_hidden=3, name="fc")
    names = [n for _, n in ops_of(Q._quantize_symbol(fc, "gpu", offline_params=["fc_weight",
                                                                               "fc_bias"],
                                                     quantize_mode="full")[0])]
    assert "emb" in names and "quantized_emb" not in names



def test_numpy_namespace_reshape_and_transpose_take_their_quantized_twins():
    """quantized_reshape.cc:125-126 (_npx_reshape -> _npx_quantized_reshape) and
    quantized_transpose.cc:118-127 (_npi_transpose -> _npx_quantized_transpose); both keep
    the float node's attribute dictionary."""
    d = S.Variable("data")
    fc1 = S.FullyConnected(d, num_hidden=16, flatten=False, name="fc1")
    rs = S.create("_npx_reshape", fc1, name="rs", newshape=(-2, -2, -6, 4, -1))
    tr = S.create("_npi_transpose", rs, name="tr", axes=(0, -2, 1, -1))
    fc2 = S.FullyConnected(tr, num_hidden=8, flatten=False, name="fc2")
    offline = [n for n in fc2.list_arguments() if n != "data"]
    qsym, calib = Q._quantize_symbol(fc2, "gpu", offline_params=offline, quantize_mode="full")
    assert ops_of(qsym) == [
        ("_contrib_quantize_v2", "fc1_data_quantize"),
        ("_contrib_quantized_fully_connected", "quantized_fc1"),
        ("_contrib_requantize", "requantize_fc1"),
        ("_npx_quantized_reshape", "quantized_rs"),
        ("_npx_quantized_transpose", "quantized_tr"),
        ("_contrib_quantized_fully_connected", "quantized_fc2"),
        ("_contrib_requantize", "requantize_fc2"),
        ("_contrib_dequantize", "fc2_dequantize")]
    assert node(qsym, "quantized_rs")[1:] == (
        {"newshape": "(-2, -2, -6, 4, -1)"},
        [("requantize_fc1", 0), ("requantize_fc1", 1), ("requantize_fc1", 2)])
    assert node(qsym, "quantized_tr")[1:] == (
        {"axes": "(0, -2, 1, -1)"},
        [("quantized_rs", 0), ("quantized_rs", 1), ("quantized_rs", 2)])
    assert calib == ["fc1_data", "fc1_output", "fc2_output"]
