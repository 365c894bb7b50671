// Host side of the INT8 operators for the gpu device: attribute parsing, shape /
// type inference and the FCompute<gpu> / FStatefulCompute<gpu> functions, attached
// to the NNVM registry under the reference's operator names.  Every compute
// function only unpacks TBlobs, attributes, the stream and the temp space and calls
// the C ABI of libmxq_hip.so (include/mxq.h); no kernel is launched from here.
//
// Reference registrations this file mirrors (names, aliases, argument order,
// attributes, resource requests):
//   _contrib_quantize_v2                 quantize_v2.cc:68-138, quantize_v2.cu:29-30
//   _contrib_quantize                    quantize.cc:67-124, quantize.cu
//   _contrib_requantize                  requantize.cc:71-124, requantize.cu:29
//   _contrib_dequantize                  dequantize.cc:65-110, dequantize.cu:29-30
//   _contrib_quantized_fully_connected   quantized_fully_connected.cc:317-382, .cu:141-143
//   _contrib_quantized_conv              quantized_conv.cc:176-237, .cu:293-294
//   _contrib_quantized_act               quantized_activation.cc:84-120
//   _contrib_quantized_pooling           quantized_pooling.cc:159-209, quantized_pooling.cu:126-127
//   _contrib_quantized_flatten           quantized_flatten.cc:30-63
// (all under src/operator/quantization/).  Inside MXNet only the "<gpu>" attributes
// of this file would be compiled (the CPU .cc files already register the rest).
#include <algorithm>
#include <cmath>
#include <string>
#include <vector>

#include "../../../include/mxq.h"
#include "mxq_params.h"
#include "mxq_shim.h"

namespace mxnet {
namespace op {

using mshadow::gpu;

namespace {

// Non-zero return code of the launcher -> the exception MXNet's CHECK would raise.
inline void MXQ_CALL(int rc) {
  if (rc != 0) throw dmlc::Error(std::string("libmxq_hip: ") + mxq_last_error());
}

inline void* raw_stream(const OpContext& ctx) {
  mshadow::Stream<gpu>* s = ctx.get_stream<gpu>();
  return s ? s->stream_ : nullptr;
}

// quantization_utils.h:201-220
template <typename Param>
int GetQuantizeOutputType(const Param& param) {
  if (param.out_type == kAuto) {
    if (param.min_calib_range.has_value() && param.max_calib_range.has_value() &&
        param.min_calib_range.value() >= 0.0)
      return mshadow::kUint8;
    return mshadow::kInt8;
  }
  if (param.out_type == kInt8) return mshadow::kInt8;
  if (param.out_type == kUint8) return mshadow::kUint8;
  LOG_FATAL << "Unsupported out_type in params: " << param.out_type;
  return mshadow::kInt8;
}

const TShape kScalarShape{1};

}  // namespace

// ---- shape / type inference ---------------------------------------------------------

// quantize_v2-inl.h:129-147: 1 input, outputs (data-shaped, (1,), (1,)); the batch
// dimension flows back from the output to the input.
static bool QuantizeV2Shape(const NodeAttrs&, ShapeVector* in, ShapeVector* out) {
  CHECK_EQ(in->size(), 1U);
  CHECK_EQ(out->size(), 3U);
  TShape d = (*in)[0];
  SHAPE_ASSIGN_CHECK(*out, 0, (*in)[0]);
  SHAPE_ASSIGN_CHECK(*out, 1, kScalarShape);
  SHAPE_ASSIGN_CHECK(*out, 2, kScalarShape);
  if ((*out)[0].ndim() > 0 && d.ndim() > 0) {
    d[0] = (*out)[0][0];
    SHAPE_ASSIGN_CHECK(*in, 0, d);
  }
  return !shape_is_none((*out)[0]);
}

// quantize_v2-inl.h:149-179 (the non-oneDNN branch: fp32, uint8 or int8 input)
static bool QuantizeV2Type(const NodeAttrs& attrs, std::vector<int>* in, std::vector<int>* out) {
  CHECK_EQ(in->size(), 1U);
  CHECK_EQ(out->size(), 3U);
  const auto& param = nnvm::get<QuantizeV2Param>(attrs.parsed);
  const int t = (*in)[0];
  CHECK(t == mshadow::kFloat32 || t == mshadow::kUint8 || t == mshadow::kInt8 || t == -1)
      << "quantize_v2 only supports float32, uint8 and int8 input, got " << type_string(t);
  TYPE_ASSIGN_CHECK(*out, 0, GetQuantizeOutputType(param));
  TYPE_ASSIGN_CHECK(*out, 1, mshadow::kFloat32);
  TYPE_ASSIGN_CHECK(*out, 2, mshadow::kFloat32);
  return t != -1;
}

// quantize-inl.h:133-154, shared by _contrib_quantize and _contrib_requantize
static bool QuantizeShape(const NodeAttrs&, ShapeVector* in, ShapeVector* out) {
  CHECK_EQ(in->size(), 3U);
  CHECK_EQ(out->size(), 3U);
  TShape d = (*in)[0];
  SHAPE_ASSIGN_CHECK(*in, 1, kScalarShape);
  SHAPE_ASSIGN_CHECK(*in, 2, kScalarShape);
  SHAPE_ASSIGN_CHECK(*out, 0, (*in)[0]);
  SHAPE_ASSIGN_CHECK(*out, 1, kScalarShape);
  SHAPE_ASSIGN_CHECK(*out, 2, kScalarShape);
  if ((*out)[0].ndim() > 0 && d.ndim() > 0) {
    d[0] = (*out)[0][0];
    SHAPE_ASSIGN_CHECK(*in, 0, d);
  }
  return shape_is_known((*out)[0]);
}

// quantize-inl.h:156-176
static bool QuantizeType(const NodeAttrs& attrs, std::vector<int>* in, std::vector<int>* out) {
  CHECK_EQ(in->size(), 3U);
  CHECK_EQ(out->size(), 3U);
  const auto& param = nnvm::get<QuantizeParam>(attrs.parsed);
  TYPE_ASSIGN_CHECK(*in, 0, mshadow::kFloat32);
  TYPE_ASSIGN_CHECK(*in, 1, mshadow::kFloat32);
  TYPE_ASSIGN_CHECK(*in, 2, mshadow::kFloat32);
  CHECK(param.out_type == mshadow::kInt8 || param.out_type == mshadow::kUint8)
      << "quantize op only supports int8 and uint8 as output type";
  TYPE_ASSIGN_CHECK(*out, 0, param.out_type);
  TYPE_ASSIGN_CHECK(*out, 1, mshadow::kFloat32);
  TYPE_ASSIGN_CHECK(*out, 2, mshadow::kFloat32);
  return (*in)[0] != -1;
}

// requantize-inl.h:67-87
static bool RequantizeType(const NodeAttrs& attrs, std::vector<int>* in, std::vector<int>* out) {
  CHECK_EQ(in->size(), 3U);
  CHECK_EQ(out->size(), 3U);
  const auto& param = nnvm::get<RequantizeParam>(attrs.parsed);
  TYPE_ASSIGN_CHECK(*in, 0, mshadow::kInt32);
  TYPE_ASSIGN_CHECK(*in, 1, mshadow::kFloat32);
  TYPE_ASSIGN_CHECK(*in, 2, mshadow::kFloat32);
  TYPE_ASSIGN_CHECK(*out, 0, GetQuantizeOutputType(param));
  TYPE_ASSIGN_CHECK(*out, 1, mshadow::kFloat32);
  TYPE_ASSIGN_CHECK(*out, 2, mshadow::kFloat32);
  return (*in)[0] != -1;
}

// dequantize-inl.h:77-96
static bool DequantizeShape(const NodeAttrs&, ShapeVector* in, ShapeVector* out) {
  CHECK_EQ(in->size(), 3U);
  CHECK_EQ(out->size(), 1U);
  TShape d = (*in)[0];
  SHAPE_ASSIGN_CHECK(*in, 1, kScalarShape);
  SHAPE_ASSIGN_CHECK(*in, 2, kScalarShape);
  SHAPE_ASSIGN_CHECK(*out, 0, (*in)[0]);
  if ((*out)[0].ndim() > 0 && d.ndim() > 0) {
    d[0] = (*out)[0][0];
    SHAPE_ASSIGN_CHECK(*in, 0, d);
  }
  return shape_is_known((*out)[0]);
}

// dequantize-inl.h:98-109
static bool DequantizeType(const NodeAttrs&, std::vector<int>* in, std::vector<int>* out) {
  CHECK_EQ(in->size(), 3U);
  CHECK_EQ(out->size(), 1U);
  CHECK((*in)[0] == mshadow::kUint8 || (*in)[0] == mshadow::kInt8)
      << "the input data type of dequantize op must be provided, either uint8 or int8";
  TYPE_ASSIGN_CHECK(*in, 1, mshadow::kFloat32);
  TYPE_ASSIGN_CHECK(*in, 2, mshadow::kFloat32);
  TYPE_ASSIGN_CHECK(*out, 0, mshadow::kFloat32);
  return (*in)[0] != -1;
}

// quantized_fully_connected.cc:40-93
static bool QuantizedFullyConnectedShape(const NodeAttrs& attrs, ShapeVector* in,
                                         ShapeVector* out) {
  const auto& param = nnvm::get<FullyConnectedParam>(attrs.parsed);
  const uint32_t num_inputs = param.no_bias ? 2 : 3;
  CHECK_EQ(in->size(), num_inputs * 3);
  CHECK_EQ(out->size(), 3U);
  TShape dshape = (*in)[0];
  if (!ndim_is_known(dshape)) return false;
  CHECK(dshape.ndim() >= 1) << "quantized_fully_connected needs at least 1-D data";
  const index_t num_input =
      param.flatten ? dshape.ProdShape(1, dshape.ndim()) : dshape[dshape.ndim() - 1];
  SHAPE_ASSIGN_CHECK(*in, 1, Shape2(param.num_hidden, num_input));
  if (!param.no_bias) SHAPE_ASSIGN_CHECK(*in, 2, Shape1(param.num_hidden));
  for (size_t i = num_inputs; i < 3 * num_inputs; ++i) SHAPE_ASSIGN_CHECK(*in, i, kScalarShape);
  if (param.flatten) {
    SHAPE_ASSIGN_CHECK(*out, 0, Shape2(dshape[0], param.num_hidden));
  } else {
    TShape result(dshape);
    result[dshape.ndim() - 1] = param.num_hidden;
    SHAPE_ASSIGN_CHECK(*out, 0, result);
  }
  SHAPE_ASSIGN_CHECK(*out, 1, kScalarShape);
  SHAPE_ASSIGN_CHECK(*out, 2, kScalarShape);
  if ((*out)[0].ndim() > 0) {
    dshape[0] = (*out)[0][0];
    SHAPE_ASSIGN_CHECK(*in, 0, dshape);
  }
  return true;
}

// quantized_fully_connected.cc:95-120 (non-oneDNN branch: int8 data only)
static bool QuantizedFullyConnectedType(const NodeAttrs& attrs, std::vector<int>* in,
                                        std::vector<int>* out) {
  const auto& param = nnvm::get<FullyConnectedParam>(attrs.parsed);
  const uint32_t num_inputs = param.no_bias ? 2 : 3;
  CHECK_EQ(in->size(), num_inputs * 3);
  CHECK_EQ(out->size(), 3U);
  for (size_t i = 0; i < num_inputs; ++i) TYPE_ASSIGN_CHECK(*in, i, mshadow::kInt8);
  for (size_t i = num_inputs; i < 3 * num_inputs; ++i) TYPE_ASSIGN_CHECK(*in, i, mshadow::kFloat32);
  TYPE_ASSIGN_CHECK(*out, 0, mshadow::kInt32);
  TYPE_ASSIGN_CHECK(*out, 1, mshadow::kFloat32);
  TYPE_ASSIGN_CHECK(*out, 2, mshadow::kFloat32);
  return true;
}

// quantized_conv.cc:30-131 (the non-oneDNN branch: 2-D, NCHW, dilation allowed here
// because the kernel implements it; channel multiple-of-4 rule of cuDNN dropped)
static bool QuantizedConvShape(const NodeAttrs& attrs, ShapeVector* in, ShapeVector* out) {
  const auto& param = nnvm::get<ConvolutionParam>(attrs.parsed);
  CHECK_EQ(param.num_group, 1U) << "quantized_conv only supports num_group=1 for now";
  CHECK_EQ(in->size(), param.no_bias ? 6U : 9U);
  CHECK_EQ(out->size(), 3U);
  if (param.layout.has_value())
    CHECK_EQ(param.layout.value(), mshadow::kNCHW) << "quantized_conv only supports NCHW for now";
  const TShape& dshape = (*in)[0];
  if (dshape.ndim() <= 0) return false;
  CHECK_EQ(param.kernel.ndim(), 2) << "quantized_conv only supports 2D convolution for now";
  CHECK_EQ(dshape.ndim(), 4);
  TShape wshape{static_cast<index_t>(param.num_filter), dshape[1], param.kernel[0],
                param.kernel[1]};
  SHAPE_ASSIGN_CHECK(*in, 1, wshape);
  TShape oshape{dshape[0], static_cast<index_t>(param.num_filter), 1, 1};
  oshape[2] = (dshape[2] + 2 * param.pad[0] - param.DilatedKernelSize(0)) / param.stride[0] + 1;
  oshape[3] = (dshape[3] + 2 * param.pad[1] - param.DilatedKernelSize(1)) / param.stride[1] + 1;
  SHAPE_ASSIGN_CHECK(*out, 0, oshape);
  SHAPE_ASSIGN_CHECK(*out, 1, kScalarShape);
  SHAPE_ASSIGN_CHECK(*out, 2, kScalarShape);
  const int start = param.no_bias ? 2 : 3, end = param.no_bias ? 6 : 9;
  for (int i = start; i < end; ++i) SHAPE_ASSIGN_CHECK(*in, i, kScalarShape);
  if (!param.no_bias) SHAPE_ASSIGN_CHECK(*in, 2, Shape1(param.num_filter));
  return true;
}

// quantized_conv.cc:133-156
static bool QuantizedConvType(const NodeAttrs& attrs, std::vector<int>* in, std::vector<int>* out) {
  const auto& param = nnvm::get<ConvolutionParam>(attrs.parsed);
  CHECK_EQ(in->size(), param.no_bias ? 6U : 9U);
  CHECK_EQ(out->size(), 3U);
  TYPE_ASSIGN_CHECK(*in, 0, mshadow::kInt8);
  TYPE_ASSIGN_CHECK(*in, 1, mshadow::kInt8);
  if (!param.no_bias) TYPE_ASSIGN_CHECK(*in, 2, mshadow::kInt8);
  const size_t start = param.no_bias ? 2 : 3, end = param.no_bias ? 6 : 9;
  for (size_t i = start; i < end; ++i) TYPE_ASSIGN_CHECK(*in, i, mshadow::kFloat32);
  TYPE_ASSIGN_CHECK(*out, 0, mshadow::kInt32);
  TYPE_ASSIGN_CHECK(*out, 1, mshadow::kFloat32);
  TYPE_ASSIGN_CHECK(*out, 2, mshadow::kFloat32);
  return true;
}

// quantized_activation.cc:30-64
static bool QuantizedActivationShape(const NodeAttrs&, ShapeVector* in, ShapeVector* out) {
  CHECK_EQ(in->size(), 3U);
  if (shape_is_none((*in)[0])) return false;
  SHAPE_ASSIGN_CHECK(*in, 1, kScalarShape);
  SHAPE_ASSIGN_CHECK(*in, 2, kScalarShape);
  out->clear();
  out->push_back((*in)[0]);
  out->push_back(kScalarShape);
  out->push_back(kScalarShape);
  return true;
}
static bool QuantizedActivationType(const NodeAttrs& attrs, std::vector<int>* in,
                                    std::vector<int>* out) {
  const auto& param = nnvm::get<ActivationParam>(attrs.parsed);
  CHECK_EQ(in->size(), 3U);
  CHECK_EQ(out->size(), 3U);
  CHECK(param.act_type == activation::kReLU)
      << "_contrib_quantized_act only supports act_type=relu for now";
  TYPE_ASSIGN_CHECK(*out, 0, mshadow::kInt8);
  TYPE_ASSIGN_CHECK(*in, 1, mshadow::kFloat32);
  TYPE_ASSIGN_CHECK(*in, 2, mshadow::kFloat32);
  TYPE_ASSIGN_CHECK(*out, 1, mshadow::kFloat32);
  TYPE_ASSIGN_CHECK(*out, 2, mshadow::kFloat32);
  return true;
}

// quantized_pooling.cc:32-133.  The reference's GPU build accepts 4-D NCHW with a 2-D
// kernel only (:53-58); so does this one.
static bool QuantizedPoolingShape(const NodeAttrs& attrs, ShapeVector* in, ShapeVector* out) {
  const auto& param = nnvm::get<PoolingParam>(attrs.parsed);
  CHECK_EQ(in->size(), 3U);
  if (!shape_is_known((*in)[0])) return false;
  const TShape& dshape = (*in)[0];
  const int data_ndims = dshape.ndim();
  const int kernel_ndims = param.kernel.ndim();
  CHECK_EQ(data_ndims, 4) << "quantized_pooling: Input data should be 4D in "
                          << "(batch, channel, y, x)";
  const int layout = param.GetLayout(data_ndims);
  CHECK_EQ(layout, static_cast<int>(mshadow::kNCHW))
      << "QuantizedPoolingOp only supports NCHW layout for now, saw " << layout;
  CHECK(param.global_pool || kernel_ndims == 2)
      << "QuantizedPoolingOp only supports 2D pooling for now";
  CHECK(!param.has_output_size) << "QuantizedPoolingOp does not support adaptive pooling";
  const int N = 0, C = 1, H = 2, W = 3;
  TShape oshape(data_ndims, -1);
  oshape[N] = dshape[N];
  oshape[C] = dshape[C];
  if (param.global_pool) {
    oshape[H] = 1;
    oshape[W] = 1;
  } else {
    for (int idx = 0; idx < 2; ++idx) {
      const int dim = H + idx;
      CHECK(param.kernel[idx] <= dshape[dim] + 2 * param.pad[idx])
          << "kernel size (" << param.kernel[idx] << ") exceeds input (" << dshape[dim]
          << " padded to " << (dshape[dim] + 2 * param.pad[idx]) << ")";
      const index_t span = dshape[dim] + 2 * param.pad[idx] - param.kernel[idx];
      if (param.pooling_convention == pool_enum::kValid) {
        oshape[dim] = 1 + span / param.stride[idx];
      } else {
        // the reference evaluates the ceiling in binary32 (:95-101); "same" takes this
        // branch as well (:108-120)
        oshape[dim] = 1 + static_cast<int>(std::ceil(static_cast<float>(span) /
                                                     static_cast<float>(param.stride[idx])));
      }
    }
  }
  SHAPE_ASSIGN_CHECK(*in, 1, kScalarShape);
  SHAPE_ASSIGN_CHECK(*in, 2, kScalarShape);
  out->clear();
  out->push_back(oshape);
  out->push_back(kScalarShape);
  out->push_back(kScalarShape);
  return true;
}

// quantized_pooling.cc:135-157: the output takes the input's type (int8 or uint8).
static bool QuantizedPoolingType(const NodeAttrs& attrs, std::vector<int>* in,
                                 std::vector<int>* out) {
  const auto& param = nnvm::get<PoolingParam>(attrs.parsed);
  CHECK_EQ(in->size(), 3U);
  CHECK_EQ(out->size(), 3U);
  if (param.pool_type == pool_enum::kMaxPooling || param.pool_type == pool_enum::kAvgPooling) {
    TYPE_ASSIGN_CHECK(*out, 0, (*in)[0]);
  } else {
    LOG_FATAL << "QuantizedPoolingOp only supports pool_type=max/avg for now";
  }
  TYPE_ASSIGN_CHECK(*in, 1, mshadow::kFloat32);
  TYPE_ASSIGN_CHECK(*in, 2, mshadow::kFloat32);
  TYPE_ASSIGN_CHECK(*out, 1, mshadow::kFloat32);
  TYPE_ASSIGN_CHECK(*out, 2, mshadow::kFloat32);
  return true;
}

// quantized_flatten-inl.h:96-131
static bool QuantizedFlattenShape(const NodeAttrs&, ShapeVector* in, ShapeVector* out) {
  CHECK_EQ(in->size(), 3U);
  CHECK_EQ(out->size(), 3U);
  const TShape& dshape = (*in)[0];
  if (!shape_is_known(dshape)) return false;
  index_t target_dim = 1;
  for (int i = 1; i < dshape.ndim(); ++i) target_dim *= dshape[i];
  SHAPE_ASSIGN_CHECK(*in, 1, kScalarShape);
  SHAPE_ASSIGN_CHECK(*in, 2, kScalarShape);
  SHAPE_ASSIGN_CHECK(*out, 0, TShape(std::vector<index_t>{dshape[0], target_dim}));
  SHAPE_ASSIGN_CHECK(*out, 1, kScalarShape);
  SHAPE_ASSIGN_CHECK(*out, 2, kScalarShape);
  return true;
}
static bool QuantizedFlattenType(const NodeAttrs&, std::vector<int>* in, std::vector<int>* out) {
  CHECK_EQ(in->size(), 3U);
  CHECK_EQ(out->size(), 3U);
  TYPE_ASSIGN_CHECK(*in, 1, mshadow::kFloat32);
  TYPE_ASSIGN_CHECK(*in, 2, mshadow::kFloat32);
  TYPE_ASSIGN_CHECK(*out, 0, (*in)[0]);
  TYPE_ASSIGN_CHECK(*out, 1, mshadow::kFloat32);
  TYPE_ASSIGN_CHECK(*out, 2, mshadow::kFloat32);
  return (*in)[0] != -1;
}

// quantized_elemwise_add.cc:30-78
static bool ElemwiseAddShape(const NodeAttrs&, ShapeVector* in_shape, ShapeVector* out_shape) {
  // A, B, A_min, A_max, B_min, B_max -> C, C_min, C_max
  CHECK_EQ(in_shape->size(), 6U);
  CHECK_EQ(out_shape->size(), 3U);
  CHECK_EQ((*in_shape)[0], (*in_shape)[1]);
  for (int i = 2; i < 6; ++i) SHAPE_ASSIGN_CHECK(*in_shape, i, kScalarShape);
  SHAPE_ASSIGN_CHECK(*out_shape, 0, (*in_shape)[0]);
  SHAPE_ASSIGN_CHECK(*out_shape, 1, kScalarShape);
  SHAPE_ASSIGN_CHECK(*out_shape, 2, kScalarShape);
  return true;
}
static bool ElemwiseAddType(const NodeAttrs& attrs, std::vector<int>* in_type,
                            std::vector<int>* out_type) {
  CHECK_EQ(in_type->size(), 6U);
  CHECK_EQ(out_type->size(), 3U);
  for (int i = 0; i < 2; ++i) {
    if (in_type->at(i) == mshadow::kInt8) {
      TYPE_ASSIGN_CHECK(*in_type, i, mshadow::kInt8);
    } else {
      TYPE_ASSIGN_CHECK(*in_type, i, mshadow::kUint8);
    }
  }
  int dtype = mshadow::kInt32;
  const auto& params = nnvm::get<QuantizeElemwiseAddParam>(attrs.parsed);
  if (params.max_calib_range.has_value() && params.min_calib_range.has_value())
    dtype = (in_type->at(0) == in_type->at(1)) ? in_type->at(0) : mshadow::kInt8;
  TYPE_ASSIGN_CHECK(*out_type, 0, dtype);
  TYPE_ASSIGN_CHECK(*out_type, 1, mshadow::kFloat32);
  TYPE_ASSIGN_CHECK(*out_type, 2, mshadow::kFloat32);
  return true;
}

// quantized_concat.cc:31-103
static bool QuantizedConcatShape(const NodeAttrs& attrs, ShapeVector* in_shape,
                                 ShapeVector* out_shape) {
  const ConcatParam& param_ = nnvm::get<ConcatParam>(attrs.parsed);
  CHECK_EQ(in_shape->size(), static_cast<size_t>(param_.num_args * 3));
  CHECK_EQ(out_shape->size(), 3U);
  TShape dshape;
  index_t size = 0;
  bool has_unknown_dim_size = false;
  int axis = -1;
  const int param_dim = param_.dim.has_value() ? param_.dim.value() : 0;
  for (int i = 0; i < param_.num_args; ++i) {
    TShape tmp = (*in_shape)[i];
    if (tmp.ndim() > 0) {
      axis = CheckAxis(param_dim, tmp.ndim());
      has_unknown_dim_size = !dim_size_is_known(tmp, axis) || has_unknown_dim_size;
      size += tmp[axis];
      tmp[axis] = -1;
      shape_assign(&dshape, tmp);
    }
  }
  TShape tmp = (*out_shape)[0];
  if (tmp.ndim() > 0) {
    axis = CheckAxis(param_dim, tmp.ndim());
    tmp[axis] = -1;
    shape_assign(&dshape, tmp);
  }
  if (!ndim_is_known(dshape)) return false;
  for (int i = 0; i < param_.num_args; ++i) {
    CHECK(shape_assign(&(*in_shape)[i], dshape))
        << "Incompatible input shape: expected " << dshape << ", got " << (*in_shape)[i];
  }
  if (!has_unknown_dim_size) dshape[axis] = size;
  CHECK(shape_assign(&(*out_shape)[0], dshape))
      << "Incompatible output shape: expected " << dshape << ", got " << (*out_shape)[0];
  for (int i = param_.num_args; i < param_.num_args * 3; ++i)
    SHAPE_ASSIGN_CHECK(*in_shape, i, kScalarShape);
  SHAPE_ASSIGN_CHECK(*out_shape, 1, kScalarShape);
  SHAPE_ASSIGN_CHECK(*out_shape, 2, kScalarShape);
  return shape_is_known(dshape);
}
static bool QuantizedConcatType(const NodeAttrs& attrs, std::vector<int>* in_type,
                                std::vector<int>* out_type) {
  const ConcatParam& param_ = nnvm::get<ConcatParam>(attrs.parsed);
  CHECK_EQ(in_type->size(), static_cast<size_t>(param_.num_args * 3));
  CHECK_EQ(out_type->size(), 3U);
  int dtype = mshadow::kUint8;
  for (int i = 0; i < param_.num_args; ++i) {
    if (in_type->at(i) == mshadow::kInt8) {
      dtype = mshadow::kInt8;
    } else {
      TYPE_ASSIGN_CHECK(*in_type, i, mshadow::kUint8);
    }
  }
  TYPE_ASSIGN_CHECK(*out_type, 0, dtype);
  TYPE_ASSIGN_CHECK(*out_type, 1, mshadow::kFloat32);
  TYPE_ASSIGN_CHECK(*out_type, 2, mshadow::kFloat32);
  return true;
}

static bool DefaultStorageType(const NodeAttrs&, const int, DispatchMode* dispatch_mode,
                               std::vector<int>* in, std::vector<int>* out) {
  *dispatch_mode = DispatchMode::kFCompute;
  for (int& v : *in) v = kDefaultStorage;
  for (int& v : *out) v = kDefaultStorage;
  return true;
}

// ---- compute: gpu ------------------------------------------------------------------

// QuantizeV2Operator<gpu>::Forward, quantize_v2-inl.h:186-308
class QuantizeV2OperatorGPU {
 public:
  explicit QuantizeV2OperatorGPU(const NodeAttrs& attrs) : attrs_(attrs) {}
  void Forward(const OpContext& ctx, const std::vector<TBlob>& inputs,
               const std::vector<OpReqType>&, const std::vector<TBlob>& outputs) {
    const auto& param = nnvm::get<QuantizeV2Param>(attrs_.parsed);
    const int out_type = GetQuantizeOutputType(param);
    const bool calibrated = param.min_calib_range.has_value() && param.max_calib_range.has_value();
    const float lo = calibrated ? param.min_calib_range.value() : 0.f;
    const float hi = calibrated ? param.max_calib_range.value() : 0.f;
    void* stream = raw_stream(ctx);
    const int in_type = inputs[0].type_flag_;
    if (in_type == mshadow::kUint8 || in_type == mshadow::kInt8) {
      MXQ_CALL(mxq_quantize_v2_passthrough(stream, inputs[0].dptr_, outputs[0].dptr_,
                                           outputs[1].dptr<float>(), outputs[2].dptr<float>(),
                                           inputs[0].Size(), in_type, calibrated, lo, hi));
      return;
    }
    CHECK(in_type == mshadow::kFloat32) << "quantize_v2 expects float32 data";
    void* ws = nullptr;
    size_t ws_bytes = 0;
    if (!calibrated) {
      CHECK(!ctx.requested.empty()) << "uncalibrated quantize_v2 needs its temp space resource";
      ws_bytes = mxq_quantize_v2_workspace(inputs[0].Size());
      ws = ctx.requested[0].get_space(ws_bytes);
    }
    MXQ_CALL(mxq_quantize_v2(stream, inputs[0].dptr<float>(), outputs[0].dptr_,
                             outputs[1].dptr<float>(), outputs[2].dptr<float>(), inputs[0].Size(),
                             out_type, calibrated, lo, hi, ws, ws_bytes));
  }

 private:
  NodeAttrs attrs_;
};

static OpStatePtr CreateQuantizeV2State(const NodeAttrs& attrs, Context ctx, const ShapeVector&,
                                        const std::vector<int>&) {
  CHECK(ctx.dev_type == Context::kGPU) << "this build only provides the gpu operator";
  return OpStatePtr::Create<QuantizeV2OperatorGPU>(attrs);
}

static void QuantizeV2ForwardGPU(const OpStatePtr& state, const OpContext& ctx,
                                 const std::vector<TBlob>& inputs,
                                 const std::vector<OpReqType>& req,
                                 const std::vector<TBlob>& outputs) {
  state.get_state<QuantizeV2OperatorGPU>().Forward(ctx, inputs, req, outputs);
}

// QuantizeCompute<gpu>, quantize-inl.h:90-131
static void QuantizeComputeGPU(const NodeAttrs& attrs, const OpContext& ctx,
                               const std::vector<TBlob>& inputs, const std::vector<OpReqType>&,
                               const std::vector<TBlob>& outputs) {
  const auto& param = nnvm::get<QuantizeParam>(attrs.parsed);
  MXQ_CALL(mxq_quantize(raw_stream(ctx), inputs[0].dptr<float>(), inputs[1].dptr<float>(),
                        inputs[2].dptr<float>(), outputs[0].dptr_, outputs[1].dptr<float>(),
                        outputs[2].dptr<float>(), inputs[0].Size(), param.out_type));
}

// RequantizeForward<gpu>, requantize-inl.h:127-240
static void RequantizeForwardGPU(const NodeAttrs& attrs, const OpContext& ctx,
                                 const std::vector<TBlob>& inputs, const std::vector<OpReqType>&,
                                 const std::vector<TBlob>& outputs) {
  const auto& param = nnvm::get<RequantizeParam>(attrs.parsed);
  const int out_type = GetQuantizeOutputType(param);
  if (out_type == mshadow::kUint8)
    LOG_FATAL << "currently, uint8 requantization is only supported by CPU, "
                 "please switch to the context of CPU or int8 data type for GPU.";
  const bool calibrated = param.min_calib_range.has_value() && param.max_calib_range.has_value();
  void* ws = nullptr;
  size_t ws_bytes = 0;
  if (!calibrated) {
    CHECK(!ctx.requested.empty()) << "uncalibrated requantize needs its temp space resource";
    ws_bytes = mxq_requantize_workspace(inputs[0].Size());
    ws = ctx.requested[0].get_space(ws_bytes);
  }
  MXQ_CALL(mxq_requantize(raw_stream(ctx), inputs[0].dptr<int32_t>(), inputs[1].dptr<float>(),
                          inputs[2].dptr<float>(), outputs[0].dptr<int8_t>(),
                          outputs[1].dptr<float>(), outputs[2].dptr<float>(), inputs[0].Size(),
                          calibrated, calibrated ? param.min_calib_range.value() : 0.f,
                          calibrated ? param.max_calib_range.value() : 0.f, ws, ws_bytes));
}

// DequantizeOperator<gpu>::Forward, dequantize-inl.h:112-148
class DequantizeOperatorGPU {
 public:
  explicit DequantizeOperatorGPU(const NodeAttrs& attrs) : attrs_(attrs) {}
  void Forward(const OpContext& ctx, const std::vector<TBlob>& inputs,
               const std::vector<OpReqType>&, const std::vector<TBlob>& outputs) {
    const int t = inputs[0].type_flag_;
    if (t != mshadow::kUint8 && t != mshadow::kInt8)
      LOG_FATAL << "dequantize op only supports input type int8 or uint8";
    MXQ_CALL(mxq_dequantize(raw_stream(ctx), inputs[0].dptr_, t, inputs[1].dptr<float>(),
                            inputs[2].dptr<float>(), outputs[0].dptr<float>(),
                            outputs[0].Size()));
  }

 private:
  NodeAttrs attrs_;
};

static OpStatePtr CreateDequantizeState(const NodeAttrs& attrs, Context ctx, const ShapeVector&,
                                        const std::vector<int>&) {
  CHECK(ctx.dev_type == Context::kGPU) << "this build only provides the gpu operator";
  return OpStatePtr::Create<DequantizeOperatorGPU>(attrs);
}

static void DequantizeForwardGPU(const OpStatePtr& state, const OpContext& ctx,
                                 const std::vector<TBlob>& inputs,
                                 const std::vector<OpReqType>& req,
                                 const std::vector<TBlob>& outputs) {
  state.get_state<DequantizeOperatorGPU>().Forward(ctx, inputs, req, outputs);
}

// QuantizedFullyConnectedForwardGPU, quantized_fully_connected.cu:58-138
static void QuantizedFullyConnectedForwardGPU(const NodeAttrs& attrs, const OpContext& ctx,
                                              const std::vector<TBlob>& inputs,
                                              const std::vector<OpReqType>&,
                                              const std::vector<TBlob>& outputs) {
  const auto& param = nnvm::get<FullyConnectedParam>(attrs.parsed);
  const size_t num_inputs = param.no_bias ? 2 : 3;
  CHECK_EQ(inputs.size(), num_inputs * 3);
  CHECK_EQ(outputs.size(), 3U);
  const TShape& dshape = inputs[0].shape_;
  const TShape& wshape = inputs[1].shape_;
  index_t m, k;
  if (param.flatten || dshape.ndim() == 2) {
    m = dshape[0];
    k = dshape.ProdShape(1, dshape.ndim());
  } else {
    // flatten=false: every leading dimension is a row (the oneDNN operator's rule)
    k = dshape[dshape.ndim() - 1];
    m = dshape.ProdShape(0, dshape.ndim() - 1);
  }
  const index_t n = wshape[0];
  CHECK_EQ(wshape[1], k);
  const int8_t* bias = param.no_bias ? nullptr : inputs[2].dptr<int8_t>();
  // the operator's temp space (quantized_fully_connected.cc:369-372) carries the split-K
  // partial sums of shapes with few output tiles and a long reduction
  const size_t ws_bytes = mxq_quantized_fc_workspace(static_cast<int>(m), static_cast<int>(n),
                                                     static_cast<int>(k), 0);
  void* ws = nullptr;
  if (ws_bytes != 0 && !ctx.requested.empty()) ws = ctx.requested[0].get_space(ws_bytes);
  MXQ_CALL(mxq_quantized_fc(
      raw_stream(ctx), inputs[0].dptr<int8_t>(), inputs[1].dptr<int8_t>(), bias,
      static_cast<int>(m), static_cast<int>(n), static_cast<int>(k),
      inputs[num_inputs].dptr<float>(), inputs[num_inputs + 1].dptr<float>(),
      inputs[num_inputs + 2].dptr<float>(), inputs[num_inputs + 3].dptr<float>(),
      param.no_bias ? nullptr : inputs[7].dptr<float>(),
      param.no_bias ? nullptr : inputs[8].dptr<float>(), outputs[0].dptr<int32_t>(),
      outputs[1].dptr<float>(), outputs[2].dptr<float>(), nullptr, nullptr, nullptr, 0, 0.f, 0.f,
      ws, ws != nullptr ? ws_bytes : 0));
}

// Temp space of the convolution: what mxq_quantized_conv_nchw wants for the geometry.  The
// reference asks for NHWC copies of data, weight and output plus cuDNN's workspace
// (quantized_conv.cu:121-160); here an unpadded 1x1 layer over 16 | C channels runs on the
// NCHW tensors as they are and needs none, every other geometry
// the two operand copies (channels zero-padded to a multiple of 16 on the way) and, for
// few tiles under a long reduction, the split-K partial sums.
static size_t QuantizedConvTempBytes(const ConvolutionParam& param, const TShape& d,
                                     const TShape& w, bool operands_aligned16) {
  return mxq_quantized_conv_nchw_workspace(
      static_cast<int>(d[0]), static_cast<int>(d[1]), static_cast<int>(d[2]),
      static_cast<int>(d[3]), static_cast<int>(w[0]), static_cast<int>(w[2]),
      static_cast<int>(w[3]), static_cast<int>(param.stride[0]),
      static_cast<int>(param.stride[1]), static_cast<int>(param.pad[0]),
      static_cast<int>(param.pad[1]), static_cast<int>(param.dilate[0]),
      static_cast<int>(param.dilate[1]), operands_aligned16 ? 1 : 0);
}

// QuantizedConvForwardGPU, quantized_conv.cu:268-291
static void QuantizedConvForwardGPU(const NodeAttrs& attrs, const OpContext& ctx,
                                    const std::vector<TBlob>& inputs,
                                    const std::vector<OpReqType>&,
                                    const std::vector<TBlob>& outputs) {
  const auto& param = nnvm::get<ConvolutionParam>(attrs.parsed);
  CHECK_EQ(param.kernel.ndim(), 2) << "QuantizedConvForward<gpu> only supports 2D convolution";
  CHECK_EQ(inputs.size(), param.no_bias ? 6U : 9U);
  CHECK_EQ(outputs.size(), 3U);
  const TShape& d = inputs[0].shape_;
  const TShape& w = inputs[1].shape_;
  const int N = d[0], C = d[1], H = d[2], W = d[3], O = w[0], KH = w[2], KW = w[3];
  auto on16 = [](const void* q) { return (reinterpret_cast<uintptr_t>(q) & 15u) == 0; };
  const size_t ws_bytes =
      QuantizedConvTempBytes(param, d, w, on16(inputs[0].dptr_) && on16(inputs[1].dptr_));
  char* ws = nullptr;
  if (ws_bytes != 0) {
    CHECK(!ctx.requested.empty()) << "quantized_conv needs its temp space resource";
    ws = ctx.requested[0].get_space(ws_bytes);
  }
  const size_t ni = param.no_bias ? 2 : 3;
  MXQ_CALL(mxq_quantized_conv_nchw(
      raw_stream(ctx), inputs[0].dptr<int8_t>(), inputs[1].dptr<int8_t>(),
      param.no_bias ? nullptr : inputs[2].dptr<int8_t>(), N, C, H, W, O, KH, KW,
      static_cast<int>(param.stride[0]), static_cast<int>(param.stride[1]),
      static_cast<int>(param.pad[0]), static_cast<int>(param.pad[1]),
      static_cast<int>(param.dilate[0]), static_cast<int>(param.dilate[1]),
      inputs[ni].dptr<float>(), inputs[ni + 1].dptr<float>(), inputs[ni + 2].dptr<float>(),
      inputs[ni + 3].dptr<float>(), param.no_bias ? nullptr : inputs[7].dptr<float>(),
      param.no_bias ? nullptr : inputs[8].dptr<float>(), outputs[0].dptr<int32_t>(),
      outputs[1].dptr<float>(), outputs[2].dptr<float>(), ws, ws_bytes));
}

// _contrib_quantized_act: int8 relu, ranges pass through (dnnl_quantized_act.cc:33-45)
static void QuantizedActivationForwardGPU(const NodeAttrs& attrs, const OpContext& ctx,
                                          const std::vector<TBlob>& inputs,
                                          const std::vector<OpReqType>&,
                                          const std::vector<TBlob>& outputs) {
  const auto& param = nnvm::get<ActivationParam>(attrs.parsed);
  CHECK(param.act_type == activation::kReLU)
      << "_contrib_quantized_act only supports act_type=relu for now";
  MXQ_CALL(mxq_quantized_relu(raw_stream(ctx), inputs[0].dptr<int8_t>(), inputs[1].dptr<float>(),
                              inputs[2].dptr<float>(), outputs[0].dptr<int8_t>(),
                              outputs[1].dptr<float>(), outputs[2].dptr<float>(),
                              inputs[0].Size()));
}

// Temp-space bytes the harness (or a framework without lazy resources) must provide.
// _contrib_quantized_pooling (quantized_pooling.cu:101-124)
static void QuantizedPoolingForwardGPU(const NodeAttrs& attrs, const OpContext& ctx,
                                       const std::vector<TBlob>& inputs,
                                       const std::vector<OpReqType>&,
                                       const std::vector<TBlob>& outputs) {
  const auto& param = nnvm::get<PoolingParam>(attrs.parsed);
  CHECK_EQ(inputs.size(), 3U);
  CHECK_EQ(outputs.size(), 3U);
  CHECK(param.global_pool || param.kernel.ndim() == 2)
      << "QuantizedPoolingForward<gpu> only supports 2D convolution for now";
  CHECK(param.pool_type == pool_enum::kMaxPooling || param.pool_type == pool_enum::kAvgPooling)
      << "QuantizedCuDNNPoolingOp only supports pool_type=max/avg";
  const TShape& d = inputs[0].shape_;
  const TShape& o = outputs[0].shape_;
  CHECK_EQ(d.ndim(), 4);
  CHECK_EQ(o.ndim(), 4);
  CHECK(inputs[0].type_flag_ == mshadow::kInt8 || inputs[0].type_flag_ == mshadow::kUint8)
      << "quantized_pooling takes int8 or uint8 data";
  CHECK_EQ(outputs[0].type_flag_, inputs[0].type_flag_);
  const bool g = param.global_pool;
  const int kh = g ? static_cast<int>(d[2]) : static_cast<int>(param.kernel[0]);
  const int kw = g ? static_cast<int>(d[3]) : static_cast<int>(param.kernel[1]);
  const int sh = g ? 1 : static_cast<int>(param.stride[0]);
  const int sw = g ? 1 : static_cast<int>(param.stride[1]);
  const int ph = g ? 0 : static_cast<int>(param.pad[0]);
  const int pw = g ? 0 : static_cast<int>(param.pad[1]);
  const bool include_pad = !param.count_include_pad.has_value() || param.count_include_pad.value();
  MXQ_CALL(mxq_quantized_pooling_nchw(
      raw_stream(ctx), inputs[0].dptr_, inputs[0].type_flag_, static_cast<int>(d[0]),
      static_cast<int>(d[1]), static_cast<int>(d[2]), static_cast<int>(d[3]), kh, kw, sh, sw, ph,
      pw, static_cast<int>(o[2]), static_cast<int>(o[3]),
      param.pool_type == pool_enum::kAvgPooling ? MXQ_POOL_AVG : MXQ_POOL_MAX, include_pad,
      inputs[1].dptr<float>(), inputs[2].dptr<float>(), outputs[0].dptr_,
      outputs[1].dptr<float>(), outputs[2].dptr<float>()));
}

// _contrib_quantized_flatten (quantized_flatten-inl.h:55-94): nothing to do when the
// engine runs it in place.
static void QuantizedFlattenComputeGPU(const NodeAttrs&, const OpContext& ctx,
                                       const std::vector<TBlob>& inputs,
                                       const std::vector<OpReqType>& req,
                                       const std::vector<TBlob>& outputs) {
  CHECK_EQ(inputs.size(), 3U);
  CHECK_EQ(outputs.size(), 3U);
  CHECK_EQ(req.size(), 3U);
  if (req[0] == kWriteInplace && req[1] == kWriteInplace && req[2] == kWriteInplace) return;
  CHECK(inputs[0].type_flag_ == mshadow::kInt8 || inputs[0].type_flag_ == mshadow::kUint8)
      << "quantized_flatten op only supports int8 and uint8 as input and output type";
  MXQ_CALL(mxq_quantized_flatten(raw_stream(ctx), inputs[0].dptr_, inputs[1].dptr<float>(),
                                 inputs[2].dptr<float>(), outputs[0].dptr_,
                                 outputs[1].dptr<float>(), outputs[2].dptr<float>(),
                                 outputs[0].Size()));
}

// _contrib_quantized_elemwise_add (dnnl_quantized_elemwise_add.cc:134-257; operands of
// one shape, the only form the operator's shape function admits)
static void QuantizedElemwiseAddForwardGPU(const NodeAttrs& attrs, const OpContext& ctx,
                                           const std::vector<TBlob>& inputs,
                                           const std::vector<OpReqType>&,
                                           const std::vector<TBlob>& outputs) {
  const auto& params = nnvm::get<QuantizeElemwiseAddParam>(attrs.parsed);
  CHECK_EQ(inputs.size(), 6U) << "should be A, B, A_min, A_max, B_min, B_max";
  CHECK_EQ(outputs.size(), 3U) << "should be C, C_min, C_max";
  CHECK_EQ(inputs[0].Size(), inputs[1].Size());
  const bool calibrated = params.max_calib_range.has_value() && params.min_calib_range.has_value();
  MXQ_CALL(mxq_quantized_elemwise_add(
      raw_stream(ctx), inputs[0].dptr_, inputs[0].type_flag_, inputs[1].dptr_,
      inputs[1].type_flag_, inputs[2].dptr<float>(), inputs[3].dptr<float>(),
      inputs[4].dptr<float>(), inputs[5].dptr<float>(), outputs[0].dptr_, outputs[0].type_flag_,
      outputs[1].dptr<float>(), outputs[2].dptr<float>(), outputs[0].Size(), calibrated ? 1 : 0,
      calibrated ? params.min_calib_range.value() : 0.f,
      calibrated ? params.max_calib_range.value() : 0.f));
}

// quantized_elemwise_add-inl.h:58-70 over elemwise_binary_broadcast_op.h:41-78
static bool QuantizedBinaryBroadcastShape(const NodeAttrs&, ShapeVector* in_attrs,
                                          ShapeVector* out_attrs) {
  CHECK_EQ(in_attrs->size(), 6U);
  CHECK_EQ(out_attrs->size(), 3U);
  for (int i = 2; i < 6; ++i) SHAPE_ASSIGN_CHECK(*in_attrs, i, TShape{1});
  SHAPE_ASSIGN_CHECK(*out_attrs, 1, TShape{1});
  SHAPE_ASSIGN_CHECK(*out_attrs, 2, TShape{1});
  const TShape& lhs = (*in_attrs)[0];
  const TShape& rhs = (*in_attrs)[1];
  if (!ndim_is_known(lhs) || !ndim_is_known(rhs)) return false;
  if (lhs == rhs) {
    SHAPE_ASSIGN_CHECK(*out_attrs, 0, lhs);
    return shape_is_known(lhs);
  }
  TShape out(std::max(lhs.ndim(), rhs.ndim()), -1);
  const int bl = out.ndim() - lhs.ndim();
  const int br = out.ndim() - rhs.ndim();
  for (int i = 0; i < out.ndim(); ++i) {
    index_t l = 1, r = 1;
    if (i >= bl) l = lhs[i - bl];
    if (i >= br) r = rhs[i - br];
    if (l < 0 || r < 0) continue;
    if (l != r) {
      CHECK(l == 1 || r == 1) << "operands could not be broadcast together with shapes " << lhs
                              << " " << rhs;
      out[i] = (l == 1 ? r : l);
    } else {
      out[i] = l;
    }
  }
  SHAPE_ASSIGN_CHECK(*out_attrs, 0, out);
  return shape_is_known(lhs) && shape_is_known(rhs) && shape_is_known(out);
}

// _contrib_quantized_npi_add (dnnl_quantized_elemwise_add.cc:134-257): operands of one shape
// take the sum above, others the broadcasting form
static void QuantizedNpiAddForwardGPU(const NodeAttrs& attrs, const OpContext& ctx,
                                      const std::vector<TBlob>& inputs,
                                      const std::vector<OpReqType>&,
                                      const std::vector<TBlob>& outputs) {
  const auto& params = nnvm::get<QuantizeElemwiseAddParam>(attrs.parsed);
  CHECK_EQ(inputs.size(), 6U) << "should be A, B, A_min, A_max, B_min, B_max";
  CHECK_EQ(outputs.size(), 3U) << "should be C, C_min, C_max";
  const bool calibrated = params.max_calib_range.has_value() && params.min_calib_range.has_value();
  std::vector<int64_t> ls, rs;
  for (int i = 0; i < inputs[0].shape_.ndim(); ++i) ls.push_back(inputs[0].shape_[i]);
  for (int i = 0; i < inputs[1].shape_.ndim(); ++i) rs.push_back(inputs[1].shape_[i]);
  MXQ_CALL(mxq_quantized_broadcast_add(
      raw_stream(ctx), inputs[0].dptr_, inputs[0].type_flag_, static_cast<int>(ls.size()),
      ls.data(), inputs[1].dptr_, inputs[1].type_flag_, static_cast<int>(rs.size()), rs.data(),
      inputs[2].dptr<float>(), inputs[3].dptr<float>(), inputs[4].dptr<float>(),
      inputs[5].dptr<float>(), outputs[0].dptr_, outputs[0].type_flag_, outputs[1].dptr<float>(),
      outputs[2].dptr<float>(), calibrated ? 1 : 0,
      calibrated ? params.min_calib_range.value() : 0.f,
      calibrated ? params.max_calib_range.value() : 0.f));
}

// _contrib_quantized_concat (dnnl_quantized_concat.cc:41-115)
static void QuantizedConcatForwardGPU(const NodeAttrs& attrs, const OpContext& ctx,
                                      const std::vector<TBlob>& inputs,
                                      const std::vector<OpReqType>&,
                                      const std::vector<TBlob>& outputs) {
  const ConcatParam& param_ = nnvm::get<ConcatParam>(attrs.parsed);
  const int n = param_.num_args;
  CHECK_EQ(inputs.size(), static_cast<size_t>(n * 3));
  CHECK_EQ(outputs.size(), 3U);
  const TShape& oshape = outputs[0].shape_;
  const int axis = CheckAxis(param_.dim.has_value() ? param_.dim.value() : 0, oshape.ndim());
  int64_t outer = 1, inner = 1;
  for (int i = 0; i < axis; ++i) outer *= oshape[i];
  for (int i = axis + 1; i < oshape.ndim(); ++i) inner *= oshape[i];
  std::vector<const void*> data(n);
  std::vector<int> types(n);
  std::vector<const float*> mins(n), maxs(n);
  std::vector<int64_t> extents(n);
  int64_t total = 0;
  for (int i = 0; i < n; ++i) {
    CHECK_EQ(inputs[i].shape_.ndim(), oshape.ndim());
    data[i] = inputs[i].dptr_;
    types[i] = inputs[i].type_flag_;
    mins[i] = inputs[n + 2 * i].dptr<float>();
    maxs[i] = inputs[n + 2 * i + 1].dptr<float>();
    extents[i] = inputs[i].shape_[axis];
    total += extents[i];
  }
  CHECK_EQ(total, oshape[axis]);
  MXQ_CALL(mxq_quantized_concat(raw_stream(ctx), n, data.data(), types.data(), mins.data(),
                                maxs.data(), extents.data(), outer, inner, outputs[0].dptr_,
                                outputs[0].type_flag_, outputs[1].dptr<float>(),
                                outputs[2].dptr<float>()));
}

size_t MXQTensorOpsTempSpaceBytes(const NodeAttrs& attrs, const ShapeVector& in);

size_t MXQTempSpaceBytes(const NodeAttrs& attrs, const ShapeVector& in, const ShapeVector& out) {
  const std::string& name = attrs.op->name;
  if (name == "_contrib_quantize_asym" || name == "_contrib_quantized_batch_norm" ||
      name == "_contrib_quantized_batch_norm_relu")
    return MXQTensorOpsTempSpaceBytes(attrs, in);
  if (name == "_contrib_quantize_v2") return mxq_quantize_v2_workspace(in[0].Size());
  if (name == "_contrib_requantize") return mxq_requantize_workspace(in[0].Size());
  if (name == "_contrib_quantized_conv")
    return QuantizedConvTempBytes(nnvm::get<ConvolutionParam>(attrs.parsed), in[0], in[1], false);
  if (name == "_contrib_quantized_fully_connected") {
    // rows x reduction as QuantizedFullyConnectedForwardGPU reads them off the shapes
    const auto& param = nnvm::get<FullyConnectedParam>(attrs.parsed);
    const TShape& d = in[0];
    if (d.ndim() < 1 || in[1].ndim() != 2) return 0;
    index_t m, k;
    if (param.flatten || d.ndim() == 2) {
      m = d[0];
      k = d.ProdShape(1, d.ndim());
    } else {
      k = d[d.ndim() - 1];
      m = d.ProdShape(0, d.ndim() - 1);
    }
    return mxq_quantized_fc_workspace(static_cast<int>(m), static_cast<int>(in[1][0]),
                                      static_cast<int>(k), 0);
  }
  return 0;
}

// ---- registration ---------------------------------------------------------------------

static std::vector<std::string> QuantizedFcConvInputNames(bool no_bias) {
  if (no_bias) return {"data", "weight", "min_data", "max_data", "min_weight", "max_weight"};
  return {"data",       "weight",     "bias",     "min_data", "max_data",
          "min_weight", "max_weight", "min_bias", "max_bias"};
}

template <typename Param>
static std::vector<ResourceRequest> TempSpaceUnlessCalibrated(const NodeAttrs& attrs) {
  const auto& param = nnvm::get<Param>(attrs.parsed);
  if (param.min_calib_range.has_value() && param.max_calib_range.has_value())
    return std::vector<ResourceRequest>();
  return std::vector<ResourceRequest>(1, ResourceRequest::kTempSpace);
}

NNVM_REGISTER_OP(_contrib_quantize_v2)
    .add_alias("_npx_contrib_quantize_v2")
    .describe("Quantize a input tensor from float to `out_type`, with user-specified "
              "`min_calib_range` and `max_calib_range` or the input range collected at runtime.")
    .set_attr_parser(ParamParser<QuantizeV2Param>)
    .set_num_inputs(1)
    .set_num_outputs(3)
    .set_attr<nnvm::FListInputNames>("FListInputNames",
                                     [](const NodeAttrs&) {
                                       return std::vector<std::string>{"data"};
                                     })
    .set_attr<mxnet::FInferShape>("FInferShape", QuantizeV2Shape)
    .set_attr<nnvm::FInferType>("FInferType", QuantizeV2Type)
    .set_attr<FInferStorageType>("FInferStorageType", DefaultStorageType)
    .set_attr<FCreateOpState>("FCreateOpState", CreateQuantizeV2State)
    .set_attr<FStatefulCompute>("FStatefulCompute<gpu>", QuantizeV2ForwardGPU)
    .set_attr<nnvm::FInplaceOption>("FInplaceOption",
                                    [](const NodeAttrs&) {
                                      return std::vector<std::pair<int, int>>{{0, 0}};
                                    })
    .set_attr<nnvm::FInplaceIdentity>("FInplaceIdentity",
                                      [](const NodeAttrs&) { return std::vector<bool>{true}; })
    .set_attr<FNeedCalibrateInput>("FNeedCalibrateInput",
                                   [](const NodeAttrs&) { return std::vector<int>{0}; })
    .set_attr<FResourceRequest>("FResourceRequest", TempSpaceUnlessCalibrated<QuantizeV2Param>)
    .set_attr<nnvm::FGradient>("FGradient", MakeZeroGradNodes)
    .add_argument("data", "NDArray-or-Symbol", "A ndarray/symbol of type `float32`")
    .add_arguments(QuantizeV2Param::__FIELDS__());

NNVM_REGISTER_OP(_contrib_quantize)
    .add_alias("_npx_contrib_quantize")
    .describe("Quantize a input tensor from float to `out_type`, with user-specified "
              "`min_range` and `max_range`.")
    .set_attr_parser(ParamParser<QuantizeParam>)
    .set_num_inputs(3)
    .set_num_outputs(3)
    .set_attr<nnvm::FListInputNames>("FListInputNames",
                                     [](const NodeAttrs&) {
                                       return std::vector<std::string>{"data", "min_range",
                                                                       "max_range"};
                                     })
    .set_attr<mxnet::FInferShape>("FInferShape", QuantizeShape)
    .set_attr<nnvm::FInferType>("FInferType", QuantizeType)
    .set_attr<FInferStorageType>("FInferStorageType", DefaultStorageType)
    .set_attr<FCompute>("FCompute<gpu>", QuantizeComputeGPU)
    .add_argument("data", "NDArray-or-Symbol", "A ndarray/symbol of type `float32`")
    .add_argument("min_range", "NDArray-or-Symbol",
                  "The minimum scalar value possibly produced for the input")
    .add_argument("max_range", "NDArray-or-Symbol",
                  "The maximum scalar value possibly produced for the input")
    .add_arguments(QuantizeParam::__FIELDS__());

NNVM_REGISTER_OP(_contrib_requantize)
    .add_alias("_npx_requantize")
    .describe("Given data that is quantized in int32 and the corresponding thresholds, "
              "requantize the data into int8 using min and max thresholds either calculated at "
              "runtime or from calibration.")
    .set_attr_parser(ParamParser<RequantizeParam>)
    .set_num_inputs(3)
    .set_num_outputs(3)
    .set_attr<nnvm::FListInputNames>("FListInputNames",
                                     [](const NodeAttrs&) {
                                       return std::vector<std::string>{"data", "min_range",
                                                                       "max_range"};
                                     })
    .set_attr<mxnet::FInferShape>("FInferShape", QuantizeShape)
    .set_attr<nnvm::FInferType>("FInferType", RequantizeType)
    .set_attr<FInferStorageType>("FInferStorageType", DefaultStorageType)
    .set_attr<FCompute>("FCompute<gpu>", RequantizeForwardGPU)
    .set_attr<FNeedCalibrateInput>("FNeedCalibrateInput",
                                   [](const NodeAttrs&) { return std::vector<int>{0}; })
    .set_attr<FResourceRequest>("FResourceRequest", TempSpaceUnlessCalibrated<RequantizeParam>)
    .set_attr<nnvm::FGradient>("FGradient", MakeZeroGradNodes)
    .add_argument("data", "NDArray-or-Symbol", "A ndarray/symbol of type `int32`")
    .add_argument("min_range", "NDArray-or-Symbol",
                  "The original minimum scalar value in the form of float32 used for quantizing "
                  "data into int32.")
    .add_argument("max_range", "NDArray-or-Symbol",
                  "The original maximum scalar value in the form of float32 used for quantizing "
                  "data into int32.")
    .add_arguments(RequantizeParam::__FIELDS__());

NNVM_REGISTER_OP(_contrib_dequantize)
    .describe("Dequantize the input tensor into a float tensor. min_range and max_range are "
              "scalar floats that specify the range for the output data.")
    .set_attr_parser(ParamParser<DequantizeParam>)
    .set_num_inputs(3)
    .set_num_outputs(1)
    .set_attr<nnvm::FListInputNames>("FListInputNames",
                                     [](const NodeAttrs&) {
                                       return std::vector<std::string>{"data", "min_range",
                                                                       "max_range"};
                                     })
    .set_attr<mxnet::FInferShape>("FInferShape", DequantizeShape)
    .set_attr<nnvm::FInferType>("FInferType", DequantizeType)
    .set_attr<FInferStorageType>("FInferStorageType", DefaultStorageType)
    .set_attr<FCreateOpState>("FCreateOpState", CreateDequantizeState)
    .set_attr<FStatefulCompute>("FStatefulCompute<gpu>", DequantizeForwardGPU)
    .set_attr<nnvm::FGradient>("FGradient", MakeZeroGradNodes)
    .add_argument("data", "NDArray-or-Symbol", "A ndarray/symbol of type `uint8`")
    .add_argument("min_range", "NDArray-or-Symbol",
                  "The minimum scalar value possibly produced for the input in float32")
    .add_argument("max_range", "NDArray-or-Symbol",
                  "The maximum scalar value possibly produced for the input in float32")
    .add_arguments(DequantizeParam::__FIELDS__());

NNVM_REGISTER_OP(_contrib_quantized_fully_connected)
    .add_alias("_npx_quantized_fully_connected")
    .describe("Fully Connected operator for input, weight and bias data type of int8, and "
              "accumulates in type int32 for the output.")
    .set_num_inputs([](const NodeAttrs& attrs) {
      return nnvm::get<FullyConnectedParam>(attrs.parsed).no_bias ? 6 : 9;
    })
    .set_num_outputs(3)
    .set_attr_parser(ParamParser<FullyConnectedParam>)
    .set_attr<nnvm::FListInputNames>(
        "FListInputNames",
        [](const NodeAttrs& attrs) {
          return QuantizedFcConvInputNames(nnvm::get<FullyConnectedParam>(attrs.parsed).no_bias);
        })
    .set_attr<nnvm::FListOutputNames>("FListOutputNames",
                                      [](const NodeAttrs&) {
                                        return std::vector<std::string>{"output", "min_output",
                                                                        "max_output"};
                                      })
    .set_attr<mxnet::FInferShape>("FInferShape", QuantizedFullyConnectedShape)
    .set_attr<nnvm::FInferType>("FInferType", QuantizedFullyConnectedType)
    .set_attr<FInferStorageType>("FInferStorageType", DefaultStorageType)
    .set_attr<FNeedRequantize>("FNeedRequantize", [](const NodeAttrs&) { return true; })
    .set_attr<FCompute>("FCompute<gpu>", QuantizedFullyConnectedForwardGPU)
    .set_attr<FResourceRequest>("FResourceRequest",
                                [](const NodeAttrs&) {
                                  return std::vector<ResourceRequest>{ResourceRequest::kTempSpace};
                                })
    .set_attr<nnvm::FGradient>("FGradient", MakeZeroGradNodes)
    .add_argument("data", "NDArray-or-Symbol", "Input data.")
    .add_argument("weight", "NDArray-or-Symbol", "weight.")
    .add_argument("bias", "NDArray-or-Symbol", "bias.")
    .add_argument("min_data", "NDArray-or-Symbol", "Minimum value of data.")
    .add_argument("max_data", "NDArray-or-Symbol", "Maximum value of data.")
    .add_argument("min_weight", "NDArray-or-Symbol", "Minimum value of weight.")
    .add_argument("max_weight", "NDArray-or-Symbol", "Maximum value of weight.")
    .add_argument("min_bias", "NDArray-or-Symbol", "Minimum value of bias.")
    .add_argument("max_bias", "NDArray-or-Symbol", "Maximum value of bias.")
    .add_arguments(FullyConnectedParam::__FIELDS__());

NNVM_REGISTER_OP(_contrib_quantized_conv)
    .add_alias("_npx_quantized_conv")
    .describe("Convolution operator for input, weight and bias data type of int8, and "
              "accumulates in type int32 for the output.")
    .set_num_inputs([](const NodeAttrs& attrs) {
      return nnvm::get<ConvolutionParam>(attrs.parsed).no_bias ? 6 : 9;
    })
    .set_num_outputs(3)
    .set_attr_parser(ConvolutionParamParser)
    .set_attr<nnvm::FListInputNames>(
        "FListInputNames",
        [](const NodeAttrs& attrs) {
          return QuantizedFcConvInputNames(nnvm::get<ConvolutionParam>(attrs.parsed).no_bias);
        })
    .set_attr<nnvm::FListOutputNames>("FListOutputNames",
                                      [](const NodeAttrs&) {
                                        return std::vector<std::string>{"output", "min_output",
                                                                        "max_output"};
                                      })
    .set_attr<mxnet::FInferShape>("FInferShape", QuantizedConvShape)
    .set_attr<nnvm::FInferType>("FInferType", QuantizedConvType)
    .set_attr<FInferStorageType>("FInferStorageType", DefaultStorageType)
    .set_attr<FResourceRequest>("FResourceRequest",
                                [](const NodeAttrs&) {
                                  return std::vector<ResourceRequest>(1,
                                                                      ResourceRequest::kTempSpace);
                                })
    .set_attr<FNeedRequantize>("FNeedRequantize", [](const NodeAttrs&) { return true; })
    .set_attr<FCompute>("FCompute<gpu>", QuantizedConvForwardGPU)
    .set_attr<nnvm::FGradient>("FGradient", MakeZeroGradNodes)
    .add_argument("data", "NDArray-or-Symbol", "Input data.")
    .add_argument("weight", "NDArray-or-Symbol", "weight.")
    .add_argument("bias", "NDArray-or-Symbol", "bias.")
    .add_argument("min_data", "NDArray-or-Symbol", "Minimum value of data.")
    .add_argument("max_data", "NDArray-or-Symbol", "Maximum value of data.")
    .add_argument("min_weight", "NDArray-or-Symbol", "Minimum value of weight.")
    .add_argument("max_weight", "NDArray-or-Symbol", "Maximum value of weight.")
    .add_argument("min_bias", "NDArray-or-Symbol", "Minimum value of bias.")
    .add_argument("max_bias", "NDArray-or-Symbol", "Maximum value of bias.")
    .add_arguments(ConvolutionParam::__FIELDS__());

NNVM_REGISTER_OP(_contrib_quantized_act)
    .add_alias("_npx_quantized_act")
    .describe("Activation operator for input and output data type of int8. Only `relu`.")
    .set_num_inputs(3)
    .set_num_outputs(3)
    .set_attr_parser(ParamParser<ActivationParam>)
    .set_attr<nnvm::FListInputNames>("FListInputNames",
                                     [](const NodeAttrs&) {
                                       return std::vector<std::string>{"data", "min_data",
                                                                       "max_data"};
                                     })
    .set_attr<nnvm::FListOutputNames>("FListOutputNames",
                                      [](const NodeAttrs&) {
                                        return std::vector<std::string>{"output", "min_output",
                                                                        "max_output"};
                                      })
    .set_attr<nnvm::FInferType>("FInferType", QuantizedActivationType)
    .set_attr<mxnet::FInferShape>("FInferShape", QuantizedActivationShape)
    .set_attr<FInferStorageType>("FInferStorageType", DefaultStorageType)
    .set_attr<FNeedRequantize>("FNeedRequantize", [](const NodeAttrs&) { return false; })
    .set_attr<FCompute>("FCompute<gpu>", QuantizedActivationForwardGPU)
    .add_argument("data", "NDArray-or-Symbol", "Input data.")
    .add_argument("min_data", "NDArray-or-Symbol", "Minimum value of data.")
    .add_argument("max_data", "NDArray-or-Symbol", "Maximum value of data.")
    .add_arguments(ActivationParam::__FIELDS__());

NNVM_REGISTER_OP(_contrib_quantized_pooling)
    .add_alias("_npx_quantized_pooling")
    .describe("Pooling operator for input and output data type of int8. Only `max` and `avg`.")
    .set_num_inputs(3)
    .set_num_outputs(3)
    .set_attr_parser(PoolingParamParser)
    .set_attr<nnvm::FListInputNames>("FListInputNames",
                                     [](const NodeAttrs&) {
                                       return std::vector<std::string>{"data", "min_data",
                                                                       "max_data"};
                                     })
    .set_attr<nnvm::FListOutputNames>("FListOutputNames",
                                      [](const NodeAttrs&) {
                                        return std::vector<std::string>{"output", "min_output",
                                                                        "max_output"};
                                      })
    .set_attr<mxnet::FInferShape>("FInferShape", QuantizedPoolingShape)
    .set_attr<nnvm::FInferType>("FInferType", QuantizedPoolingType)
    .set_attr<FInferStorageType>("FInferStorageType", DefaultStorageType)
    .set_attr<FNeedRequantize>("FNeedRequantize",
                               [](const NodeAttrs& attrs) {
                                 const auto& param = nnvm::get<PoolingParam>(attrs.parsed);
                                 CHECK(param.pool_type == pool_enum::kMaxPooling ||
                                       param.pool_type == pool_enum::kAvgPooling)
                                     << "QuantizedPoolingOp only supports pool_type=max/avg for now";
                                 return false;
                               })
    .set_attr<FCompute>("FCompute<gpu>", QuantizedPoolingForwardGPU)
    .add_argument("data", "NDArray-or-Symbol", "Input data.")
    .add_argument("min_data", "NDArray-or-Symbol", "Minimum value of data.")
    .add_argument("max_data", "NDArray-or-Symbol", "Maximum value of data.")
    .add_arguments(PoolingParam::__FIELDS__());

NNVM_REGISTER_OP(_contrib_quantized_flatten)
    .add_alias("_npx_quantized_flatten")
    .set_num_inputs(3)
    .set_num_outputs(3)
    .set_attr<mxnet::FInferShape>("FInferShape", QuantizedFlattenShape)
    .set_attr<nnvm::FInferType>("FInferType", QuantizedFlattenType)
    .set_attr<nnvm::FListInputNames>("FListInputNames",
                                     [](const NodeAttrs&) {
                                       return std::vector<std::string>{"data", "min_data",
                                                                       "max_data"};
                                     })
    .set_attr<nnvm::FListOutputNames>("FListOutputNames",
                                      [](const NodeAttrs&) {
                                        return std::vector<std::string>{"output", "min_output",
                                                                        "max_output"};
                                      })
    .set_attr<nnvm::FInplaceOption>("FInplaceOption",
                                    [](const NodeAttrs&) {
                                      return std::vector<std::pair<int, int>>{{0, 0}, {1, 1}, {2, 2}};
                                    })
    .set_attr<FCompute>("FCompute<gpu>", QuantizedFlattenComputeGPU)
    .add_argument("data", "NDArray-or-Symbol", "A ndarray/symbol of type `float32`")
    .add_argument("min_data", "NDArray-or-Symbol",
                  "The minimum scalar value possibly produced for the data")
    .add_argument("max_data", "NDArray-or-Symbol",
                  "The maximum scalar value possibly produced for the data");

// quantized_elemwise_add.cc:89-122 (+ the parser and argument fields the oneDNN file
// attaches, dnnl_quantized_elemwise_add.cc:270-275)
NNVM_REGISTER_OP(_contrib_quantized_elemwise_add)
    .add_alias("_npx_quantized_elemwise_add")
    .describe("elemwise_add operator for input dataA and input dataB data type of int8, and "
              "accumulates in type int32 for the output.")
    .set_num_inputs(6)
    .set_num_outputs(3)
    .set_attr_parser(ParamParser<QuantizeElemwiseAddParam>)
    .set_attr<nnvm::FListInputNames>("FListInputNames",
                                     [](const NodeAttrs&) {
                                       return std::vector<std::string>{"lhs",     "rhs",
                                                                       "lhs_min", "lhs_max",
                                                                       "rhs_min", "rhs_max"};
                                     })
    .set_attr<nnvm::FListOutputNames>("FListOutputNames",
                                      [](const NodeAttrs&) {
                                        return std::vector<std::string>{"output", "min_output",
                                                                        "max_output"};
                                      })
    .set_attr<nnvm::FInferType>("FInferType", ElemwiseAddType)
    .set_attr<mxnet::FInferShape>("FInferShape", ElemwiseAddShape)
    .set_attr<FInferStorageType>("FInferStorageType", DefaultStorageType)
    .set_attr<FNeedRequantize>("FNeedRequantize", [](const NodeAttrs&) { return true; })
    .set_attr<FCompute>("FCompute<gpu>", QuantizedElemwiseAddForwardGPU)
    .add_argument("lhs", "NDArray-or-Symbol", "first input")
    .add_argument("rhs", "NDArray-or-Symbol", "second input")
    .add_argument("lhs_min", "NDArray-or-Symbol", "3rd input")
    .add_argument("lhs_max", "NDArray-or-Symbol", "4th input")
    .add_argument("rhs_min", "NDArray-or-Symbol", "5th input")
    .add_argument("rhs_max", "NDArray-or-Symbol", "6th input")
    .add_arguments(QuantizeElemwiseAddParam::__FIELDS__());

// quantized_elemwise_add.cc:141-178 (+ dnnl_quantized_elemwise_add.cc:276-281)
NNVM_REGISTER_OP(_contrib_quantized_npi_add)
    .add_alias("_npx_quantized_npi_add")
    .describe("elemwise_add operator with numpy broadcasting for input dataA and input dataB "
              "data type of int8, and accumulates in type int32 for the output.")
    .set_num_inputs(6)
    .set_num_outputs(3)
    .set_attr_parser(ParamParser<QuantizeElemwiseAddParam>)
    .set_attr<nnvm::FListInputNames>("FListInputNames",
                                     [](const NodeAttrs&) {
                                       return std::vector<std::string>{"lhs",     "rhs",
                                                                       "lhs_min", "lhs_max",
                                                                       "rhs_min", "rhs_max"};
                                     })
    .set_attr<nnvm::FListOutputNames>("FListOutputNames",
                                      [](const NodeAttrs&) {
                                        return std::vector<std::string>{"output", "min_output",
                                                                        "max_output"};
                                      })
    .set_attr<nnvm::FInferType>("FInferType", ElemwiseAddType)
    .set_attr<mxnet::FInferShape>("FInferShape", QuantizedBinaryBroadcastShape)
    .set_attr<FInferStorageType>("FInferStorageType", DefaultStorageType)
    .set_attr<FNeedRequantize>("FNeedRequantize", [](const NodeAttrs&) { return true; })
    .set_attr<FCompute>("FCompute<gpu>", QuantizedNpiAddForwardGPU)
    .add_argument("lhs", "NDArray-or-Symbol", "first input")
    .add_argument("rhs", "NDArray-or-Symbol", "second input")
    .add_argument("lhs_min", "NDArray-or-Symbol", "3rd input")
    .add_argument("lhs_max", "NDArray-or-Symbol", "4th input")
    .add_argument("rhs_min", "NDArray-or-Symbol", "5th input")
    .add_argument("rhs_max", "NDArray-or-Symbol", "6th input")
    .add_arguments(QuantizeElemwiseAddParam::__FIELDS__());

// quantized_concat.cc:105-141
NNVM_REGISTER_OP(_contrib_quantized_concat)
    .describe("Joins input arrays along a given axis.  All inputs with different min/max will "
              "be rescaled by using largest [min, max] pairs.  If any input holds int8, then "
              "the output will be int8. Otherwise output will be uint8.")
    .set_num_inputs([](const NodeAttrs& attrs) {
      return static_cast<uint32_t>(nnvm::get<ConcatParam>(attrs.parsed).num_args * 3);
    })
    .set_num_outputs(3)
    .set_attr_parser(ParamParser<ConcatParam>)
    .set_attr<nnvm::FListInputNames>(
        "FListInputNames",
        [](const NodeAttrs& attrs) {
          const ConcatParam& params = nnvm::get<ConcatParam>(attrs.parsed);
          std::vector<std::string> ret;
          for (int i = 0; i < params.num_args; ++i) ret.push_back("arg" + std::to_string(i));
          for (int i = 0; i < params.num_args; ++i) {
            ret.push_back("arg" + std::to_string(i) + "_min");
            ret.push_back("arg" + std::to_string(i) + "_max");
          }
          return ret;
        })
    .set_attr<nnvm::FListOutputNames>("FListOutputNames",
                                      [](const NodeAttrs&) {
                                        return std::vector<std::string>{"output", "min_output",
                                                                        "max_output"};
                                      })
    .set_attr<nnvm::FInferType>("FInferType", QuantizedConcatType)
    .set_attr<mxnet::FInferShape>("FInferShape", QuantizedConcatShape)
    .set_attr<FInferStorageType>("FInferStorageType", DefaultStorageType)
    .set_attr<std::string>("key_var_num_args", "num_args")
    .set_attr<FCompute>("FCompute<gpu>", QuantizedConcatForwardGPU)
    .add_argument("data", "NDArray-or-Symbol[]", "List of arrays to concatenate")
    .add_arguments(ConcatParam::__FIELDS__());

}  // namespace op
}  // namespace mxnet
