"""The C++ operator host on the CPU: registry contents, attribute parsing, shape and
type inference (no kernel is launched).  Expected values are read off the reference's
registrations and inference functions (src/operator/quantization/*.cc, *-inl.h)."""
import numpy as np
import pytest
import torch

from mxnet_amd import operator as op
from mxnet_amd.operator import MXNetError, Node

F32, I8, U8, I32 = torch.float32, torch.int8, torch.uint8, torch.int32


def test_registry_names_aliases_and_gpu_attributes():
    names = op.list_operators()
    for n in ["_contrib_quantize_v2", "_contrib_requantize", "_contrib_dequantize",
              "_contrib_quantized_fully_connected", "_contrib_quantized_conv",
              "_contrib_quantize", "_contrib_quantized_act"]:
        assert n in names
    # stateless operators carry FCompute<gpu>, the two stateful ones FStatefulCompute<gpu>
    for n in ["_contrib_requantize", "_contrib_quantized_fully_connected",
              "_contrib_quantized_conv", "_contrib_quantize", "_contrib_quantized_act"]:
        assert op.has_attr(n, "FCompute<gpu>") and not op.has_attr(n, "FStatefulCompute<gpu>")
    for n in ["_contrib_quantize_v2", "_contrib_dequantize"]:
        assert op.has_attr(n, "FStatefulCompute<gpu>") and op.has_attr(n, "FCreateOpState")
        assert not op.has_attr(n, "FCompute<gpu>")
    for n in ["_contrib_quantized_fully_connected", "_contrib_quantized_conv"]:
        assert op.has_attr(n, "FNeedRequantize") and op.has_attr(n, "FResourceRequest")
    for n in ["_contrib_quantize_v2", "_contrib_requantize"]:
        assert op.has_attr(n, "FNeedCalibrateInput")
    # aliases resolve to the same operator
    for alias, name in [("_npx_contrib_quantize_v2", "_contrib_quantize_v2"),
                        ("_npx_requantize", "_contrib_requantize"),
                        ("_npx_quantized_fully_connected", "_contrib_quantized_fully_connected"),
                        ("_npx_quantized_conv", "_contrib_quantized_conv"),
                        ("_npx_quantized_act", "_contrib_quantized_act")]:
        assert op.has_attr(alias, "FInferShape")
    with pytest.raises(MXNetError, match="not registered"):
        Node("_contrib_does_not_exist")


def test_inference_only_operators_have_zero_gradients():
    """FGradient = MakeZeroGradNodes on the five operators (quantize_v2.cc:108, requantize.cc:94,
    dequantize.cc:95, quantized_fully_connected.cc:362, quantized_conv.cc:221): one zeros_like
    node per input, named as operator_common.h:430-444 names them."""
    for n in ["_contrib_quantize_v2", "_contrib_requantize", "_contrib_dequantize",
              "_contrib_quantized_fully_connected", "_contrib_quantized_conv"]:
        assert op.has_attr(n, "FGradient")
    q = Node("_contrib_quantize_v2", name="q0", out_type="int8")
    assert q.gradient_nodes() == [("zeros_like", "q0_backward")]
    fc = Node("_contrib_quantized_fully_connected", name="fc1", num_hidden=8, no_bias=True)
    assert fc.gradient_nodes() == [("zeros_like", "fc1_in%d_backward" % i) for i in range(6)]
    conv = Node("_contrib_quantized_conv", name="c", kernel=(1, 1), num_filter=8)
    assert len(conv.gradient_nodes()) == 9 and conv.gradient_nodes()[8][1] == "c_in8_backward"
    assert Node("_contrib_quantized_act", act_type="relu").gradient_nodes() == []


def test_input_output_names():
    n = Node("_contrib_quantized_fully_connected", num_hidden=8)
    assert n.num_inputs == 9 and n.num_outputs == 3
    assert n.list_inputs() == ["data", "weight", "bias", "min_data", "max_data", "min_weight",
                               "max_weight", "min_bias", "max_bias"]
    assert n.list_outputs() == ["output", "min_output", "max_output"]
    n = Node("_contrib_quantized_conv", kernel=(3, 3), num_filter=8, no_bias=True)
    assert n.num_inputs == 6
    assert n.list_inputs() == ["data", "weight", "min_data", "max_data", "min_weight",
                               "max_weight"]
    assert Node("_contrib_requantize").list_inputs() == ["data", "min_range", "max_range"]
    assert Node("_contrib_quantize_v2").list_inputs() == ["data"]
    assert Node("_contrib_dequantize").num_outputs == 1


def test_attribute_parsing():
    # defaults: out_type int8 for quantize_v2 and requantize, uint8 for v1 quantize
    assert Node("_contrib_quantize_v2").infer_type([F32])[1][0] == I8
    assert Node("_contrib_requantize").infer_type([I32, F32, F32])[1][0] == I8
    assert Node("_contrib_quantize").infer_type([F32, F32, F32])[1][0] == U8
    # auto: uint8 iff calibrated with a non-negative minimum (quantization_utils.h:201-220)
    assert Node("_contrib_quantize_v2", out_type="auto", min_calib_range=0.0,
                max_calib_range=1.0).infer_type([F32])[1][0] == U8
    assert Node("_contrib_quantize_v2", out_type="auto", min_calib_range=-0.1,
                max_calib_range=1.0).infer_type([F32])[1][0] == I8
    assert Node("_contrib_quantize_v2", out_type="auto").infer_type([F32])[1][0] == I8
    # calibration ranges arrive as std::to_string(float) text, "None" is absent
    n = Node("_contrib_requantize", min_calib_range="-134.348999", max_calib_range="523.429993")
    assert n.infer_type([None, None, None])[0] == [I32, F32, F32]
    Node("_contrib_requantize", min_calib_range="None", max_calib_range="None")
    # bool spellings
    for v in ["True", "true", "1", True]:
        assert Node("_contrib_quantized_fully_connected", num_hidden=4, no_bias=v).num_inputs == 6
    for v in ["False", "false", "0", False]:
        assert Node("_contrib_quantized_fully_connected", num_hidden=4, no_bias=v).num_inputs == 9
    # tuple spellings
    for k in ["(3, 3)", "[3,3]", "(3,3)"]:
        n = Node("_contrib_quantized_conv", kernel=k, num_filter=8, no_bias=True)
        assert n.infer_shape([(1, 4, 8, 8)] + [None] * 5)[1][0] == (1, 8, 6, 6)
    # errors
    with pytest.raises(MXNetError, match="Invalid Parameter format for out_type"):
        Node("_contrib_quantize_v2", out_type="int4")
    with pytest.raises(MXNetError, match="Cannot find argument 'foo'"):
        Node("_contrib_dequantize", foo=1)
    with pytest.raises(MXNetError, match="Required parameter num_hidden"):
        Node("_contrib_quantized_fully_connected")
    with pytest.raises(MXNetError, match="greater equal to 1"):
        Node("_contrib_quantized_fully_connected", num_hidden=0)
    with pytest.raises(MXNetError, match="float32"):
        Node("_contrib_dequantize", out_type="float16")
    with pytest.raises(MXNetError, match="in operator _contrib_quantize_v2"):
        Node("_contrib_quantize_v2", min_calib_range="abc")
    Node("_contrib_quantize_v2", __profiler_scope__="x")  # hidden keys are accepted


def test_shape_inference():
    n = Node("_contrib_quantize_v2")
    assert n.infer_shape([(2, 3, 4)]) == ([(2, 3, 4)], [(2, 3, 4), (1,), (1,)])
    # the batch dimension flows back from a known output (quantize_v2-inl.h:141-144)
    assert n.infer_shape([(-1, 3)], [(2, 3), None, None])[0] == [(2, 3)]
    with pytest.raises(MXNetError, match="Shape inconsistent"):
        n.infer_shape([(2, 3)], [(2, 4), None, None])
    n = Node("_contrib_requantize")
    assert n.infer_shape([(5, 6), None, None]) == ([(5, 6), (1,), (1,)], [(5, 6), (1,), (1,)])
    with pytest.raises(MXNetError, match="Shape inconsistent"):
        n.infer_shape([(5, 6), (2,), None])
    n = Node("_contrib_dequantize")
    assert n.infer_shape([(7,), None, None]) == ([(7,), (1,), (1,)], [(7,)])
    # quantized FC: flatten semantics (quantized_fully_connected.cc:54-78)
    n = Node("_contrib_quantized_fully_connected", num_hidden=100)
    ins, outs = n.infer_shape([(32, 111, 2, 2)] + [None] * 8)
    assert ins[1] == (100, 444) and ins[2] == (100,) and ins[3:] == [(1,)] * 6
    assert outs == [(32, 100), (1,), (1,)]
    n = Node("_contrib_quantized_fully_connected", num_hidden=100, flatten=False, no_bias=True)
    ins, outs = n.infer_shape([(32, 512, 2)] + [None] * 5)
    assert ins[1] == (100, 2) and outs[0] == (32, 512, 100)
    with pytest.raises(MXNetError, match="Shape inconsistent"):
        Node("_contrib_quantized_fully_connected", num_hidden=8, no_bias=True).infer_shape(
            [(4, 16), (8, 32)] + [None] * 4)
    # quantized conv (quantized_conv.cc:30-131): OH = (H + 2p - dilated_k) / s + 1
    n = Node("_contrib_quantized_conv", kernel=(3, 3), num_filter=128, pad=(1, 1))
    ins, outs = n.infer_shape([(3, 4, 28, 28)] + [None] * 8)
    assert ins[1] == (128, 4, 3, 3) and ins[2] == (128,) and outs[0] == (3, 128, 28, 28)
    n = Node("_contrib_quantized_conv", kernel=(1, 1), num_filter=512, stride=(2, 2),
             no_bias=True)
    assert n.infer_shape([(64, 256, 56, 56)] + [None] * 5)[1][0] == (64, 512, 28, 28)
    n = Node("_contrib_quantized_conv", kernel=(3, 3), num_filter=8, dilate=(2, 2), pad=(2, 2),
             stride=(2, 2), no_bias=True)
    assert n.infer_shape([(1, 16, 12, 13)] + [None] * 5)[1][0] == (1, 8, 6, 7)
    with pytest.raises(MXNetError, match="num_group"):
        Node("_contrib_quantized_conv", kernel=(3, 3), num_filter=8, num_group=2,
             no_bias=True).infer_shape([(1, 16, 12, 13)] + [None] * 5)
    with pytest.raises(MXNetError, match="NCHW"):
        Node("_contrib_quantized_conv", kernel=(3, 3), num_filter=8, layout="NHWC",
             no_bias=True).infer_shape([(1, 12, 13, 16)] + [None] * 5)
    n = Node("_contrib_quantized_act", act_type="relu")
    assert n.infer_shape([(4, 5), None, None])[1] == [(4, 5), (1,), (1,)]


def test_type_inference():
    n = Node("_contrib_quantized_fully_connected", num_hidden=4)
    ins, outs = n.infer_type([None] * 9)
    assert ins == [I8, I8, I8] + [F32] * 6 and outs == [I32, F32, F32]
    with pytest.raises(MXNetError, match="Type inconsistent"):
        n.infer_type([U8] + [None] * 8)           # gpu operator: int8 data only
    n = Node("_contrib_quantized_conv", kernel=(1, 1), num_filter=4, no_bias=True)
    assert n.infer_type([None] * 6) == ([I8, I8] + [F32] * 4, [I32, F32, F32])
    n = Node("_contrib_dequantize")
    assert n.infer_type([U8, None, None]) == ([U8, F32, F32], [F32])
    with pytest.raises(MXNetError, match="either uint8 or int8"):
        n.infer_type([F32, None, None])
    with pytest.raises(MXNetError, match="Type inconsistent"):
        Node("_contrib_requantize").infer_type([F32, None, None])
    with pytest.raises(MXNetError, match="relu"):
        Node("_contrib_quantized_act", act_type="tanh").infer_type([I8, None, None])
    assert Node("_contrib_quantize_v2").infer_type([I8])[1][0] == I8   # pass-through input


def test_pooling_and_flatten_inference():
    """quantized_pooling.cc:32-157, quantized_flatten-inl.h:96-131; the shapes are those
    of the reference's test (test_quantization.py:641-658)."""
    for n in ["_contrib_quantized_pooling", "_contrib_quantized_flatten"]:
        assert op.has_attr(n, "FCompute<gpu>") and op.has_attr(n, "FInferShape")
    assert op.has_attr("_npx_quantized_pooling", "FInferType")
    assert op.has_attr("_contrib_quantized_pooling", "FNeedRequantize")
    assert op.has_attr("_contrib_quantized_flatten", "FInplaceOption")
    n = Node("_contrib_quantized_pooling", kernel=(3, 3), pool_type="max", stride=(2, 2))
    assert n.list_inputs() == ["data", "min_data", "max_data"]
    assert n.list_outputs() == ["output", "min_output", "max_output"]
    ins, outs = n.infer_shape([(3, 4, 56, 56), None, None])
    assert ins == [(3, 4, 56, 56), (1,), (1,)] and outs == [(3, 4, 27, 27), (1,), (1,)]
    n = Node("_contrib_quantized_pooling", kernel=(3, 3), pool_type="max", stride=(2, 2),
             pooling_convention="full")
    assert n.infer_shape([(3, 4, 56, 56), None, None])[1][0] == (3, 4, 28, 28)
    n = Node("_contrib_quantized_pooling", kernel=(3, 3), pool_type="max", stride=(2, 2),
             global_pool=True)
    assert n.infer_shape([(3, 4, 56, 56), None, None])[1][0] == (3, 4, 1, 1)
    n = Node("_contrib_quantized_pooling", kernel=(7, 7), pool_type="avg")
    assert n.infer_shape([(3, 512, 7, 7), None, None])[1][0] == (3, 512, 1, 1)
    n = Node("_contrib_quantized_pooling", kernel=(3, 3), pool_type="max", stride=(2, 2),
             pad=(1, 1))
    assert n.infer_shape([(64, 64, 112, 112), None, None])[1][0] == (64, 64, 56, 56)
    # output type follows the data type
    assert n.infer_type([I8, None, None]) == ([I8, F32, F32], [I8, F32, F32])
    assert n.infer_type([U8, None, None])[1][0] == U8
    with pytest.raises(MXNetError, match="exceeds input"):
        Node("_contrib_quantized_pooling", kernel=(9, 9)).infer_shape([(1, 1, 7, 7), None, None])
    with pytest.raises(MXNetError, match="4D"):
        Node("_contrib_quantized_pooling", kernel=(3, 3)).infer_shape(
            [(1, 1, 3, 7, 7), None, None])
    with pytest.raises(MXNetError, match="max/avg"):
        Node("_contrib_quantized_pooling", kernel=(3, 3), pool_type="sum").infer_type(
            [I8, None, None])
    with pytest.raises(MXNetError, match="pool_type"):
        Node("_contrib_quantized_pooling", kernel=(3, 3), pool_type="median")
    n = Node("_contrib_quantized_flatten")
    assert n.infer_shape([(2, 3, 4, 5), None, None]) == ([(2, 3, 4, 5), (1,), (1,)],
                                                         [(2, 60), (1,), (1,)])
    assert n.infer_type([U8, None, None]) == ([U8, F32, F32], [U8, F32, F32])


def test_elemwise_add_and_concat_inference():
    """quantized_elemwise_add.cc:30-122, quantized_concat.cc:31-141."""
    for n in ["_contrib_quantized_elemwise_add", "_contrib_quantized_concat"]:
        assert op.has_attr(n, "FCompute<gpu>") and op.has_attr(n, "FInferShape")
    assert op.has_attr("_npx_quantized_elemwise_add", "FInferType")
    assert op.has_attr("_contrib_quantized_elemwise_add", "FNeedRequantize")
    assert not op.has_attr("_contrib_quantized_concat", "FNeedRequantize")
    assert op.has_attr("elemwise_add", "FQuantizedOp") and op.has_attr("Concat", "FQuantizedOp")
    n = Node("_contrib_quantized_elemwise_add")
    assert n.list_inputs() == ["lhs", "rhs", "lhs_min", "lhs_max", "rhs_min", "rhs_max"]
    assert n.list_outputs() == ["output", "min_output", "max_output"]
    ins, outs = n.infer_shape([(3, 4, 5), (3, 4, 5), None, None, None, None])
    assert ins == [(3, 4, 5), (3, 4, 5)] + [(1,)] * 4 and outs == [(3, 4, 5), (1,), (1,)]
    with pytest.raises(MXNetError):
        n.infer_shape([(3, 4, 5), (3, 4, 6), None, None, None, None])
    # int32 unless calibrated; then the operands' type, int8 when they differ
    assert n.infer_type([I8, U8, None, None, None, None])[1] == [I32, F32, F32]
    c = Node("_contrib_quantized_elemwise_add", min_calib_range=-1.0, max_calib_range=2.0)
    assert c.infer_type([I8, I8, None, None, None, None])[1][0] == I8
    assert c.infer_type([U8, U8, None, None, None, None])[1][0] == U8
    assert c.infer_type([I8, U8, None, None, None, None])[1][0] == I8
    half = Node("_contrib_quantized_elemwise_add", min_calib_range=-1.0)
    assert half.infer_type([I8, I8, None, None, None, None])[1][0] == I32
    with pytest.raises(MXNetError):
        Node("_contrib_quantized_elemwise_add", out_type="int8")

    n = Node("_contrib_quantized_concat", num_args=3, dim=1)
    assert n.num_inputs == 9
    assert n.list_inputs() == ["arg0", "arg1", "arg2", "arg0_min", "arg0_max", "arg1_min",
                               "arg1_max", "arg2_min", "arg2_max"]
    ins, outs = n.infer_shape([(2, 3, 4), (2, 5, 4), (2, 1, 4)] + [None] * 6)
    assert ins[:3] == [(2, 3, 4), (2, 5, 4), (2, 1, 4)] and ins[3:] == [(1,)] * 6
    assert outs == [(2, 9, 4), (1,), (1,)]
    assert Node("_contrib_quantized_concat", num_args=2, dim=-1).infer_shape(
        [(2, 3), (2, 4)] + [None] * 4)[1][0] == (2, 7)
    assert Node("_contrib_quantized_concat", num_args=2, dim=0).infer_shape(
        [(2, 3), (5, 3)] + [None] * 4)[1][0] == (7, 3)
    with pytest.raises(MXNetError, match="Incompatible input shape"):
        n.infer_shape([(2, 3, 4), (2, 5, 5), (2, 1, 4)] + [None] * 6)
    with pytest.raises(MXNetError, match="exceeds the input dimension"):
        Node("_contrib_quantized_concat", num_args=2, dim=2).infer_shape(
            [(2, 3), (2, 4)] + [None] * 4)
    assert n.infer_type([U8, U8, U8] + [None] * 6)[1] == [U8, F32, F32]
    assert n.infer_type([U8, I8, U8] + [None] * 6)[1] == [I8, F32, F32]
    with pytest.raises(MXNetError, match="num_args"):
        Node("_contrib_quantized_concat", dim=1)


# src/operator/tensor/matrix_op.cc:154-196: the examples of the Reshape documentation, and
# the quantized_reshape cases of tests/python/quantization/test_quantization.py:1057-1073
# that use the legacy special values only
RESHAPE_EXAMPLES = [
    ((2, 3, 4), (4, 0, 2), False, (4, 3, 2)), ((2, 3, 4), (2, 0, 0), False, (2, 3, 4)),
    ((2, 3, 4), (6, 1, -1), False, (6, 1, 4)), ((2, 3, 4), (3, -1, 8), False, (3, 1, 8)),
    ((2, 3, 4), (-1,), False, (24,)), ((2, 3, 4), (-2,), False, (2, 3, 4)),
    ((2, 3, 4), (2, -2), False, (2, 3, 4)), ((2, 3, 4), (-2, 1, 1), False, (2, 3, 4, 1, 1)),
    ((2, 3, 4), (-3, 4), False, (6, 4)), ((2, 3, 4, 5), (-3, -3), False, (6, 20)),
    ((2, 3, 4), (0, -3), False, (2, 12)), ((2, 3, 4), (-3, -2), False, (6, 4)),
    ((2, 3, 4), (-4, 1, 2, -2), False, (1, 2, 3, 4)),
    ((2, 3, 4), (2, -4, -1, 3, -2), False, (2, 1, 3, 4)),
    ((10, 5, 4), (-1, 0), False, (40, 5)), ((10, 5, 4), (-1, 0), True, (50, 4)),
]


def test_tensor_op_registrations_and_inference():
    """quantized_elemwise_mul.cc:33-89,208-256, quantized_indexing_op.cc:30-190,
    quantized_reshape.cc:48-127, quantized_transpose.cc:31-115, quantize_asym.cc:36-157."""
    for n in ["_contrib_quantized_elemwise_mul", "_contrib_quantized_embedding",
              "_contrib_quantized_reshape", "_contrib_quantized_transpose"]:
        assert op.has_attr(n, "FCompute<gpu>") and op.has_attr(n, "FInferShape")
        assert op.has_attr(n, "FInferType")
    assert op.has_attr("_contrib_quantize_asym", "FStatefulCompute<gpu>")
    assert op.has_attr("_contrib_quantize_asym", "FNeedCalibrateInput")
    for alias in ["_npx_quantized_elemwise_mul", "_npx_quantized_embedding", "quantized_reshape",
                  "quantized_transpose"]:
        assert op.has_attr(alias, "FInferShape")
    assert op.has_attr("_contrib_quantized_elemwise_mul", "FNeedRequantize")
    for n in ["_contrib_quantized_embedding", "_contrib_quantized_reshape",
              "_contrib_quantized_transpose"]:
        assert not op.has_attr(n, "FNeedRequantize")
    for n in ["elemwise_mul", "Embedding", "Reshape", "transpose"]:
        assert op.has_attr(n, "FQuantizedOp")
    assert op.has_attr("Embedding", "FAvoidQuantizeInput")

    # elemwise_mul: three outputs, or the float product alone
    n = Node("_contrib_quantized_elemwise_mul")
    assert n.list_inputs() == ["lhs", "rhs", "lhs_min", "lhs_max", "rhs_min", "rhs_max"]
    assert n.num_outputs == 3
    ins, outs = n.infer_shape([(3, 4), (3, 4), None, None, None, None])
    assert ins == [(3, 4), (3, 4)] + [(1,)] * 4 and outs == [(3, 4), (1,), (1,)]
    with pytest.raises(MXNetError):
        n.infer_shape([(3, 4), (3, 5), None, None, None, None])
    with pytest.raises(MXNetError, match="broadcast"):
        n.infer_shape([(3, 4), (4,), None, None, None, None])
    assert n.infer_type([I8, I8, None, None, None, None])[1] == [I32, F32, F32]
    c = Node("_contrib_quantized_elemwise_mul", min_calib_range=-1.0, max_calib_range=2.0)
    assert c.infer_type([I8, I8, None, None, None, None])[1] == [I8, F32, F32]
    fo = Node("_contrib_quantized_elemwise_mul", enable_float_output=True)
    assert fo.num_outputs == 1
    assert fo.infer_shape([(3, 4), (3, 4), None, None, None, None])[1] == [(3, 4)]
    assert fo.infer_type([I8, I8, None, None, None, None])[1] == [F32]
    with pytest.raises(MXNetError):
        Node("_contrib_quantized_elemwise_mul", out_type="int8")

    # embedding
    e = Node("_contrib_quantized_embedding", input_dim=1000, output_dim=256)
    assert e.list_inputs() == ["data", "weight", "min_weight", "max_weight"]
    assert e.list_outputs() == ["output", "min_output", "max_output"]
    ins, outs = e.infer_shape([(32, 128), None, None, None])
    assert ins == [(32, 128), (1000, 256), (1,), (1,)]
    assert outs == [(32, 128, 256), (1,), (1,)]
    with pytest.raises(MXNetError):
        e.infer_shape([(32,), (999, 256), None, None])
    assert e.infer_type([F32, None, None, None]) == ([F32, I8, F32, F32], [I8, F32, F32])
    assert e.infer_type([I32, None, None, None])[1] == [I8, F32, F32]
    with pytest.raises(MXNetError, match="input_dim"):
        Node("_contrib_quantized_embedding", output_dim=4)
    with pytest.raises(MXNetError):
        Node("_contrib_quantized_embedding", input_dim=0, output_dim=4)

    # reshape: the special values
    for shape, newshape, reverse, expected in RESHAPE_EXAMPLES:
        r = Node("_contrib_quantized_reshape", shape=newshape, reverse=reverse)
        ins, outs = r.infer_shape([shape, None, None])
        assert outs == [expected, (1,), (1,)] and ins == [shape, (1,), (1,)]
    r = Node("_contrib_quantized_reshape", shape=(-1, 4))
    assert r.infer_type([U8, None, None]) == ([U8, F32, F32], [U8, F32, F32])
    with pytest.raises(MXNetError, match="Split dims"):
        Node("_contrib_quantized_reshape", shape=(-4, 5, -1, -2)).infer_shape(
            [(12, 3), None, None])

    # transpose
    t = Node("_contrib_quantized_transpose", axes=(2, 3, 0, 1))
    assert t.list_inputs() == ["data", "min_data", "max_data"]
    ins, outs = t.infer_shape([(5, 3, 6, 8), None, None])
    assert outs == [(6, 8, 5, 3), (1,), (1,)] and ins == [(5, 3, 6, 8), (1,), (1,)]
    assert Node("_contrib_quantized_transpose").infer_shape([(5, 3, 6), None, None])[1][0] == \
        (6, 3, 5)
    # the input's shape from the output's
    ins, _ = t.infer_shape([None, None, None], [(6, 8, 5, 3), None, None])
    assert ins[0] == (5, 3, 6, 8)
    assert t.infer_type([I8, None, None]) == ([I8, F32, F32], [I8, F32, F32])
    with pytest.raises(MXNetError):
        t.infer_shape([(5, 3, 6), None, None])

    # quantize_asym
    q = Node("_contrib_quantize_asym")
    assert q.list_inputs() == ["data"] and q.list_outputs() == ["output", "scale", "shift"]
    assert q.infer_shape([(4, 5, 6)])[1] == [(4, 5, 6), (1,), (1,)]
    assert q.infer_type([F32])[1] == [U8, F32, F32]
    with pytest.raises(MXNetError):
        q.infer_type([I8])


def test_quantized_batch_norm_registration_and_inference():
    """quantized_batch_norm.cc:34-122, quantized_batch_norm_relu.cc:33-121."""
    for n in ["_contrib_quantized_batch_norm", "_contrib_quantized_batch_norm_relu"]:
        assert op.has_attr(n, "FCompute<gpu>") and op.has_attr(n, "FNeedCalibrateOutput")
        assert op.has_attr(n, "FResourceRequest") and op.has_attr(n, "FMutateInputs")
        node = Node(n, min_calib_range=-1.0, max_calib_range=2.0)
        assert node.list_inputs() == ["data", "gamma", "beta", "moving_mean", "moving_var",
                                      "min_data", "max_data"]
        assert node.list_outputs() == ["output", "min_output", "max_output"]
        ins, outs = node.infer_shape([(8, 16, 5, 5)] + [None] * 6)
        assert ins == [(8, 16, 5, 5)] + [(16,)] * 4 + [(1,), (1,)]
        assert outs == [(8, 16, 5, 5), (1,), (1,)]
        assert node.infer_type([U8] + [None] * 6) == ([U8] + [F32] * 6, [I8, F32, F32])
        assert node.infer_type([I8] + [None] * 6)[1] == [I8, F32, F32]
        with pytest.raises(MXNetError, match="int8/uint8"):
            node.infer_type([F32] + [None] * 6)
    last = Node("_contrib_quantized_batch_norm", axis=-1)
    assert last.infer_shape([(8, 5, 5, 16)] + [None] * 6)[0][1] == (16,)
    with pytest.raises(MXNetError, match="Channel axis out of range"):
        Node("_contrib_quantized_batch_norm", axis=4).infer_shape([(8, 5, 5, 16)] + [None] * 6)
    with pytest.raises(MXNetError):
        Node("_contrib_quantized_batch_norm", epsilon=1.0)
    # the float BatchNorm keeps no FQuantizedOp here: the pass leaves it float, as the
    # reference does for the gpu context
    assert not op.has_attr("BatchNorm", "FQuantizedOp")


# (input shape, newshape, reverse, output shape): the examples of the reference's npx.reshape
# documentation (python/mxnet/_numpy_op_doc.py:607-624), the cases of its own test
# (tests/python/unittest/test_numpy_op.py:9316-9334), then inputs it must refuse
NPX_RESHAPE_EXAMPLES = [
    ((2, 3, 8), (-2, -2, 2, -1), False, (2, 3, 2, 4)),
    ((8, 3, 3, 3, 4, 4), (-6, 2, -1, -4), False, (2, 4, 3, 3, 3, 4, 4)),
    ((8, 3, 3, 3, 4, 4), (-5, -4), False, (24, 3, 3, 4, 4)),
    ((8, 1, 1, 1, 3), (-2, -3, -3, -3, -2), False, (8, 3)),
    ((8, 3, 3, 3, 3, 8), (-4, -5), True, (8, 3, 3, 3, 24)),
    ((8, 3, 2, 4, 8), (-4, -1, 2, -6), True, (8, 3, 2, 4, 4, 2)),
    ((2, 3, 5, 5), (-2, -1), False, (2, 75)),
    ((2, 3, 5, 5), (-2, -2, -1), False, (2, 3, 25)),
    ((5, 3, 4, 5), (-2, -1, -2), False, (5, 15, 4)),
    ((2, 3, 5, 4), (-1, -2, -2), False, (8, 3, 5)),
    ((2, 3, 5, 5), (-2, -2, -2, -2), False, (2, 3, 5, 5)),
    ((2, 1, 4, 5), (-2, -3, -2, -2), False, (2, 4, 5)),
    ((1, 1, 4, 1), (-3, -3, -2, -2), False, (4, 1)),
    ((1, 1, 1, 1), (-3, -3, -3, -3), False, ()),
    ((2, 4, 5, 3), (-1, 2, 2, 1), False, (30, 2, 2, 1)),
    ((2, 3, 5, 6), (-4,), False, (2, 3, 5, 6)),
    ((2, 3, 5, 6), (6, 1, -4), False, (6, 1, 5, 6)),
    ((2, 3, 5, 6), (-5, -5), False, (6, 30)),
    ((2, 3, 5, 6), (-5, -1), False, (6, 30)),
    ((64,), (-6, 16, 4), False, (16, 4)),
    ((64,), (-6, 16, -1), False, (16, 4)),
    ((64, 1, 2, 3), (-6, 16, -1, -4), False, (16, 4, 1, 2, 3)),
    ((8, 5, 4, 6), (-4, -1, 3, -6), True, (8, 5, 4, 2, 3)),
    ((2, 3, 8), (6, 8), False, (6, 8)),
    ((0, 3), (-1,), False, (0,)),
    ((0, 3), (-1, 0), False, None),
    ((2, 3, 8), (5, -1), False, None),
    ((2, 3, 8), (-2, -3, -4), False, None),
    ((2, 3, 8), (-6, 3, 2, -4), False, None),
    ((2, 3, 8), (-1, -1), False, None),
    ((2, 3, 8), (-7,), False, None),
]


def test_numpy_namespace_reshape_and_transpose_inference():
    """quantized_reshape.cc:91-100, quantized_transpose.cc:96-99."""
    for n in ["_npx_quantized_reshape", "_npx_quantized_transpose"]:
        assert op.has_attr(n, "FCompute<gpu>") and op.has_attr(n, "FQuantizable")
    assert op.has_attr("_npx_reshape", "FQuantizedOp") and op.has_attr("_npi_reshape", "FQuantizedOp")
    assert op.has_attr("_npi_transpose", "FQuantizedOp")
    for shape, newshape, reverse, want in NPX_RESHAPE_EXAMPLES:
        node = Node("_npx_quantized_reshape", newshape=newshape, reverse=reverse)
        if want is None:
            with pytest.raises(MXNetError):
                node.infer_shape([shape, None, None])
            continue
        ins, outs = node.infer_shape([shape, None, None])
        assert outs == [want, (1,), (1,)], (shape, newshape, reverse)
        assert ins == [shape, (1,), (1,)]
        # numpy agrees wherever the special values reduce to a plain reshape
        assert np.zeros(shape, np.int8).reshape(want).shape == want
    with pytest.raises(MXNetError):
        Node("_npx_quantized_reshape")
    with pytest.raises(MXNetError, match="order"):
        Node("_npx_quantized_reshape", newshape=(-1,), order="F").infer_shape([(2, 3), None, None])
    assert Node("_npx_quantized_reshape", newshape=(-1,)).infer_type([I8, None, None]) == \
        ([I8, F32, F32], [I8, F32, F32])

    t = Node("_npx_quantized_transpose")
    assert t.infer_shape([(2, 3, 4), None, None])[1] == [(4, 3, 2), (1,), (1,)]
    t = Node("_npx_quantized_transpose", axes=(-1, 0, -2))
    assert t.infer_shape([(2, 3, 4), None, None])[1] == [(4, 2, 3), (1,), (1,)]
    assert t.infer_type([U8, None, None])[1] == [U8, F32, F32]
    with pytest.raises(MXNetError, match="Repeated axis"):
        Node("_npx_quantized_transpose", axes=(0, -3, 1)).infer_shape([(2, 3, 4), None, None])
    with pytest.raises(MXNetError, match="exceeds the range"):
        Node("_npx_quantized_transpose", axes=(0, 1, 3)).infer_shape([(2, 3, 4), None, None])
    with pytest.raises(MXNetError, match="number of axes"):
        Node("_npx_quantized_transpose", axes=(0, 1)).infer_shape([(2, 3, 4), None, None])


def test_quantized_npi_add_registration_and_inference():
    """quantized_elemwise_add.cc:141-189, quantized_elemwise_add-inl.h:58-70."""
    n = "_contrib_quantized_npi_add"
    assert op.has_attr(n, "FCompute<gpu>") and op.has_attr(n, "FNeedRequantize")
    assert op.has_attr("_npx_quantized_npi_add", "FCompute<gpu>")
    assert op.has_attr("_npi_add", "FQuantizedOp")
    node = Node(n)
    assert node.list_inputs() == ["lhs", "rhs", "lhs_min", "lhs_max", "rhs_min", "rhs_max"]
    assert node.list_outputs() == ["output", "min_output", "max_output"]
    for a, b, want in [((3, 4, 5), (4, 1), (3, 4, 5)), ((1, 1), (7, 2), (7, 2)),
                       ((2, 0, 3), (1, 3), (2, 0, 3)), ((5,), (5,), (5,)), ((6, 1), (), (6, 1))]:
        ins, outs = node.infer_shape([a, b] + [None] * 4)
        assert outs == [want, (1,), (1,)] and ins[2:] == [(1,)] * 4
    with pytest.raises(MXNetError, match="could not be broadcast"):
        node.infer_shape([(2, 3), (2, 0, 3)] + [None] * 4)
    assert node.infer_type([I8, U8] + [None] * 4)[1] == [I32, F32, F32]
    cal = Node(n, min_calib_range=-1.0, max_calib_range=1.0)
    assert cal.infer_type([U8, U8] + [None] * 4)[1] == [U8, F32, F32]
    assert cal.infer_type([I8, U8] + [None] * 4)[1] == [I8, F32, F32]
