// Graph-level registrations of the float operators the quantization pass looks at: no
// compute functions, only what the pass asks the registry (argument and output names,
// output counts, FQuantizable, FQuantizedOp).  Each block cites the registration it
// restates in the reference.
#include <string>
#include <vector>

#include "mxq_params.h"
#include "mxq_shim.h"

namespace mxnet {
namespace op {

namespace {

std::vector<std::string> OneOutput(const NodeAttrs&) { return {"output"}; }
std::vector<std::string> DataOnly(const NodeAttrs&) { return {"data"}; }

// The common body of the FQuantizedOp functions: same attribute dict under the
// quantized operator, named "quantized_<name>" (e.g. quantized_conv.cc:242-251).
nnvm::ObjectPtr QuantizedTwin(const NodeAttrs& attrs, const char* quantized_op) {
  nnvm::ObjectPtr node = nnvm::Node::Create();
  node->attrs.op = nnvm::Op::Get(quantized_op);
  node->attrs.name = "quantized_" + attrs.name;
  node->attrs.dict = attrs.dict;
  if (node->op()->attr_parser) node->op()->attr_parser(&(node->attrs));
  return node;
}

// A float node that stays as it is: no operator on the returned node tells the pass so
// (quantized_activation.cc:128-133).
nnvm::ObjectPtr NotQuantized(const NodeAttrs& attrs) {
  nnvm::ObjectPtr node = nnvm::Node::Create();
  node->attrs.op = nullptr;
  node->attrs.name = attrs.name;
  node->attrs.dict = attrs.dict;
  return node;
}

}  // namespace

// src/operator/nn/convolution.cc:435-548, quantized_conv.cc:239-251
NNVM_REGISTER_OP(Convolution)
    .set_num_inputs([](const NodeAttrs& attrs) {
      return nnvm::get<ConvolutionParam>(attrs.parsed).no_bias ? 2U : 3U;
    })
    .set_num_outputs(1)
    .set_attr_parser(ConvolutionParamParser)
    .set_attr<nnvm::FListInputNames>("FListInputNames",
                                     [](const NodeAttrs& attrs) {
                                       if (nnvm::get<ConvolutionParam>(attrs.parsed).no_bias)
                                         return std::vector<std::string>{"data", "weight"};
                                       return std::vector<std::string>{"data", "weight", "bias"};
                                     })
    .set_attr<nnvm::FListOutputNames>("FListOutputNames", OneOutput)
    .set_attr<FQuantizable>("FQuantizable",
                            [](const NodeAttrs&) { return QuantizeType::kMust; })
    .set_attr<FQuantizedOp>("FQuantizedOp", [](const NodeAttrs& attrs) {
      return QuantizedTwin(attrs, "_contrib_quantized_conv");
    });

// src/operator/nn/fully_connected.cc:255-326, quantized_fully_connected.cc:384-396
NNVM_REGISTER_OP(FullyConnected)
    .set_num_inputs([](const NodeAttrs& attrs) {
      return nnvm::get<FullyConnectedParam>(attrs.parsed).no_bias ? 2U : 3U;
    })
    .set_num_outputs(1)
    .set_attr_parser(ParamParser<FullyConnectedParam>)
    .set_attr<nnvm::FListInputNames>("FListInputNames",
                                     [](const NodeAttrs& attrs) {
                                       if (nnvm::get<FullyConnectedParam>(attrs.parsed).no_bias)
                                         return std::vector<std::string>{"data", "weight"};
                                       return std::vector<std::string>{"data", "weight", "bias"};
                                     })
    .set_attr<nnvm::FListOutputNames>("FListOutputNames", OneOutput)
    .set_attr<FQuantizable>("FQuantizable",
                            [](const NodeAttrs&) { return QuantizeType::kMust; })
    .set_attr<FQuantizedOp>("FQuantizedOp", [](const NodeAttrs& attrs) {
      return QuantizedTwin(attrs, "_contrib_quantized_fully_connected");
    });

// src/operator/nn/activation.cc:157-193, quantized_activation.cc:122-140: relu only
NNVM_REGISTER_OP(Activation)
    .set_num_inputs(1)
    .set_num_outputs(1)
    .set_attr_parser(ParamParser<ActivationParam>)
    .set_attr<nnvm::FListInputNames>("FListInputNames", DataOnly)
    .set_attr<nnvm::FListOutputNames>("FListOutputNames", OneOutput)
    .set_attr<FQuantizedOp>("FQuantizedOp", [](const NodeAttrs& attrs) {
      const ActivationParam& param = nnvm::get<ActivationParam>(attrs.parsed);
      if (param.act_type == activation::kReLU) return QuantizedTwin(attrs, "_contrib_quantized_act");
      return NotQuantized(attrs);
    });

// src/operator/nn/pooling.cc:358-446, quantized_pooling.cc:218-236: max and avg only.
// (For sum / lp pooling the reference hands back a node that still carries the float
// Pooling operator; here such a node is simply left alone.)
NNVM_REGISTER_OP(Pooling)
    .set_num_inputs(1)
    .set_num_outputs(1)
    .set_attr_parser(PoolingParamParser)
    .set_attr<nnvm::FListInputNames>("FListInputNames", DataOnly)
    .set_attr<nnvm::FListOutputNames>("FListOutputNames", OneOutput)
    .set_attr<FQuantizedOp>("FQuantizedOp", [](const NodeAttrs& attrs) {
      PoolingParam param;
      param.Init(attrs.dict);
      if (param.pool_type == pool_enum::kMaxPooling || param.pool_type == pool_enum::kAvgPooling)
        return QuantizedTwin(attrs, "_contrib_quantized_pooling");
      return NotQuantized(attrs);
    });

// src/operator/tensor/matrix_op.cc:256-290 (no argument or output names registered),
// quantized_flatten.cc:65-74
NNVM_REGISTER_OP(Flatten)
    .add_alias("flatten")
    .set_num_inputs(1)
    .set_num_outputs(1)
    .set_attr<FQuantizedOp>("FQuantizedOp", [](const NodeAttrs& attrs) {
      return QuantizedTwin(attrs, "_contrib_quantized_flatten");
    });

// Float operators that are never quantized here but whose output names the pass spells
// into node and calibration names.
// src/operator/nn/batch_norm.cc:571-640
NNVM_REGISTER_OP(BatchNorm)
    .set_num_inputs(5)
    .set_num_outputs(3)
    .set_attr<nnvm::FListInputNames>("FListInputNames",
                                     [](const NodeAttrs&) {
                                       return std::vector<std::string>{"data", "gamma", "beta",
                                                                       "moving_mean",
                                                                       "moving_var"};
                                     })
    .set_attr<nnvm::FListOutputNames>("FListOutputNames",
                                      [](const NodeAttrs&) {
                                        return std::vector<std::string>{"output", "mean", "var"};
                                      })
    .set_attr<nnvm::FNumVisibleOutputs>("FNumVisibleOutputs",
                                        [](const NodeAttrs&) { return 1U; });

// src/operator/nn/softmax.cc:108-160
NNVM_REGISTER_OP(softmax)
    .set_num_inputs(1)
    .set_num_outputs(1)
    .set_attr<nnvm::FListInputNames>("FListInputNames", DataOnly)
    .set_attr<nnvm::FListOutputNames>("FListOutputNames", OneOutput);

// src/operator/softmax_output.cc:166-272
NNVM_REGISTER_OP(SoftmaxOutput)
    .add_alias("Softmax")
    .set_num_inputs(2)
    .set_num_outputs(1)
    .set_attr<nnvm::FListInputNames>("FListInputNames",
                                     [](const NodeAttrs&) {
                                       return std::vector<std::string>{"data", "label"};
                                     })
    .set_attr<nnvm::FListOutputNames>("FListOutputNames", OneOutput);

// the operator MakeZeroGradNodes (src/operator/operator_common.h:430-444) names as the
// gradient of an inference-only operator
NNVM_REGISTER_OP(zeros_like)
    .set_num_inputs(1)
    .set_num_outputs(1)
    .set_attr<nnvm::FListInputNames>("FListInputNames", DataOnly);

// src/operator/nn/dropout.cc:64-110
NNVM_REGISTER_OP(Dropout)
    .set_num_inputs(1)
    .set_num_outputs(2)
    .set_attr<nnvm::FListInputNames>("FListInputNames", DataOnly)
    .set_attr<nnvm::FListOutputNames>("FListOutputNames",
                                      [](const NodeAttrs&) {
                                        return std::vector<std::string>{"output", "mask"};
                                      })
    .set_attr<nnvm::FNumVisibleOutputs>("FNumVisibleOutputs",
                                        [](const NodeAttrs&) { return 1U; });

// src/operator/tensor/elemwise_binary_op_basic.cc:82-110, quantized_elemwise_add.cc:124-133
NNVM_REGISTER_OP(elemwise_add)
    .add_alias("_add")
    .add_alias("_plus")
    .add_alias("_Plus")
    .set_num_inputs(2)
    .set_num_outputs(1)
    .set_attr<nnvm::FListInputNames>("FListInputNames",
                                     [](const NodeAttrs&) {
                                       return std::vector<std::string>{"lhs", "rhs"};
                                     })
    .set_attr<nnvm::FListOutputNames>("FListOutputNames", OneOutput)
    .set_attr<FQuantizedOp>("FQuantizedOp", [](const NodeAttrs& attrs) {
      return QuantizedTwin(attrs, "_contrib_quantized_elemwise_add");
    });

// src/operator/nn/concat.cc:325-411, quantized_concat.cc:143-152
NNVM_REGISTER_OP(Concat)
    .add_alias("concat")
    .set_num_inputs([](const NodeAttrs& attrs) {
      return static_cast<uint32_t>(nnvm::get<ConcatParam>(attrs.parsed).num_args);
    })
    .set_num_outputs(1)
    .set_attr_parser(ParamParser<ConcatParam>)
    .set_attr<nnvm::FListInputNames>("FListInputNames",
                                     [](const NodeAttrs& attrs) {
                                       const ConcatParam& params =
                                           nnvm::get<ConcatParam>(attrs.parsed);
                                       std::vector<std::string> ret;
                                       for (int i = 0; i < params.num_args; ++i)
                                         ret.push_back("arg" + std::to_string(i));
                                       return ret;
                                     })
    .set_attr<nnvm::FListOutputNames>("FListOutputNames", OneOutput)
    .set_attr<std::string>("key_var_num_args", "num_args")
    .set_attr<FQuantizedOp>("FQuantizedOp", [](const NodeAttrs& attrs) {
      return QuantizedTwin(attrs, "_contrib_quantized_concat");
    });

// src/operator/tensor/elemwise_binary_op_basic.cc:236-263, quantized_elemwise_mul.cc:247-256.
// Like the three operators after it, it registers no output names: its output is spelled
// "<name>_0" in calibration keys (common::GetOutputName, src/common/utils.h), and so is the
// quantized twin's, which is how the two meet in the calibration table.
NNVM_REGISTER_OP(elemwise_mul)
    .add_alias("_mul")
    .add_alias("_Mul")
    .set_num_inputs(2)
    .set_num_outputs(1)
    .set_attr<nnvm::FListInputNames>("FListInputNames",
                                     [](const NodeAttrs&) {
                                       return std::vector<std::string>{"lhs", "rhs"};
                                     })
    .set_attr<FQuantizedOp>("FQuantizedOp", [](const NodeAttrs& attrs) {
      return QuantizedTwin(attrs, "_contrib_quantized_elemwise_mul");
    });

// src/operator/tensor/indexing_op.cc:565-650, quantized_indexing_op.cc:162-190: float32
// tables only; the indices (input 0) are never quantized
NNVM_REGISTER_OP(Embedding)
    .set_num_inputs(2)
    .set_num_outputs(1)
    .set_attr_parser(ParamParser<EmbeddingParam>)
    .set_attr<nnvm::FListInputNames>("FListInputNames",
                                     [](const NodeAttrs&) {
                                       return std::vector<std::string>{"data", "weight"};
                                     })
    .set_attr<FQuantizable>("FQuantizable",
                            [](const NodeAttrs&) { return QuantizeType::kSupport; })
    .set_attr<FQuantizedOp>("FQuantizedOp",
                            [](const NodeAttrs& attrs) {
                              EmbeddingParam param;
                              param.Init(attrs.dict);
                              if (param.dtype == mshadow::kFloat32)
                                return QuantizedTwin(attrs, "_contrib_quantized_embedding");
                              nnvm::ObjectPtr node = nnvm::Node::Create();
                              node->attrs.op = nnvm::Op::Get("Embedding");
                              node->attrs.name = attrs.name;
                              node->attrs.dict = attrs.dict;
                              if (node->op()->attr_parser) node->op()->attr_parser(&(node->attrs));
                              return node;
                            })
    .set_attr<FAvoidQuantizeInput>("FAvoidQuantizeInput",
                                   [](const NodeAttrs&, const size_t index, const std::string) {
                                     return index == 0;
                                   });

// src/operator/tensor/matrix_op.cc:110-190, quantized_reshape.cc:119-127
NNVM_REGISTER_OP(Reshape)
    .add_alias("reshape")
    .set_num_inputs(1)
    .set_num_outputs(1)
    .set_attr_parser(ParamParser<ReshapeParam>)
    .set_attr<FQuantizedOp>("FQuantizedOp", [](const NodeAttrs& attrs) {
      return QuantizedTwin(attrs, "_contrib_quantized_reshape");
    });

// src/operator/tensor/matrix_op.cc:292-350, quantized_transpose.cc:106-115
NNVM_REGISTER_OP(transpose)
    .set_num_inputs(1)
    .set_num_outputs(1)
    .set_attr_parser(ParamParser<TransposeParam>)
    .set_attr<FQuantizedOp>("FQuantizedOp", [](const NodeAttrs& attrs) {
      return QuantizedTwin(attrs, "_contrib_quantized_transpose");
    });

// src/operator/numpy/np_elemwise_broadcast_op_add.cc, quantized_elemwise_add.cc:180-189
NNVM_REGISTER_OP(_npi_add)
    .set_num_inputs(2)
    .set_num_outputs(1)
    .set_attr<FQuantizedOp>("FQuantizedOp", [](const NodeAttrs& attrs) {
      return QuantizedTwin(attrs, "_contrib_quantized_npi_add");
    });

// src/operator/numpy/np_matrix_op.cc:353-375, quantized_reshape.cc:125-126
NNVM_REGISTER_OP(_npx_reshape)
    .add_alias("_npi_reshape")
    .set_num_inputs(1)
    .set_num_outputs(1)
    .set_attr_parser(ParamParser<NumpyXReshapeParam>)
    .set_attr<FQuantizedOp>("FQuantizedOp", [](const NodeAttrs& attrs) {
      return QuantizedTwin(attrs, "_npx_quantized_reshape");
    });

// src/operator/numpy/np_matrix_op.cc:80-110, quantized_transpose.cc:118-127
NNVM_REGISTER_OP(_npi_transpose)
    .set_num_inputs(1)
    .set_num_outputs(1)
    .set_attr_parser(ParamParser<NumpyTransposeParam>)
    .set_attr<FQuantizedOp>("FQuantizedOp", [](const NodeAttrs& attrs) {
      return QuantizedTwin(attrs, "_npx_quantized_transpose");
    });

}  // namespace op
}  // namespace mxnet
