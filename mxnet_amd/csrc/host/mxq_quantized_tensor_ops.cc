// Host side of the quantized operators that surround FC / conv in BERT-like and
// embedding graphs, for the gpu device: attribute parsing, shape / type inference and
// FCompute<gpu> functions under the reference's operator names.  As in
// mxq_quantization_ops.cc every compute function only unpacks TBlobs and calls the C ABI
// of libmxq_hip.so.
//
// Reference registrations this file mirrors (all under src/operator/quantization/):
//   _contrib_quantized_elemwise_mul   quantized_elemwise_mul.cc:33-89,208-245
//   _contrib_quantized_embedding      quantized_indexing_op.cc:30-73,124-160
//   _contrib_quantized_reshape        quantized_reshape.cc:48-100, quantized_reshape-inl.h:38-68
//   _contrib_quantized_transpose      quantized_transpose.cc:31-104
//   _contrib_quantize_asym            quantize_asym.cc:36-157
//   _contrib_quantized_batch_norm     quantized_batch_norm.cc:34-122
//   _contrib_quantized_batch_norm_relu  quantized_batch_norm_relu.cc:33-121
// The reference computes all five on the cpu only (quantize_asym also has a gpu class
// but registers no gpu attribute); here they are attached as "<gpu>" attributes.
#include <algorithm>
#include <iostream>
#include <string>
#include <vector>

#include "../../../include/mxq.h"
#include "mxq_params.h"
#include "mxq_shim.h"

namespace mxnet {
namespace op {

using mshadow::gpu;

namespace {

inline void MXQ_CALL(int rc) {
  if (rc != 0) throw dmlc::Error(std::string("libmxq_hip: ") + mxq_last_error());
}

inline void* raw_stream(const OpContext& ctx) {
  mshadow::Stream<gpu>* s = ctx.get_stream<gpu>();
  return s ? s->stream_ : nullptr;
}

const TShape kScalarShape{1};

bool AllDefaultStorage(const NodeAttrs&, const int, DispatchMode* dispatch_mode,
                       std::vector<int>* in_attrs, std::vector<int>* out_attrs) {
  *dispatch_mode = DispatchMode::kFCompute;
  for (auto& v : *in_attrs) v = kDefaultStorage;
  for (auto& v : *out_attrs) v = kDefaultStorage;
  return true;
}

std::vector<std::string> DataMinMax(const NodeAttrs&) { return {"data", "min_data", "max_data"}; }
std::vector<std::string> OutputMinMax(const NodeAttrs&) {
  return {"output", "min_output", "max_output"};
}

}  // namespace

// ---- _contrib_quantized_elemwise_mul ------------------------------------------------------

// quantized_elemwise_mul.cc:33-60
static bool ElemwiseMulShape(const NodeAttrs& attrs, ShapeVector* in_attrs,
                             ShapeVector* out_attrs) {
  const auto& params = nnvm::get<QuantizeElemwiseMulParam>(attrs.parsed);
  const TShape& lshape = (*in_attrs)[0];
  const TShape& rshape = (*in_attrs)[1];
  if (!ndim_is_known(lshape) || !ndim_is_known(rshape)) return false;
  CHECK_EQ(lshape.ndim(), rshape.ndim())
      << "Currently, quantized elemwise multiply doesn't support broadcast.";
  for (int i = 0; i < lshape.ndim(); ++i) CHECK_EQ(lshape[i], rshape[i]);
  for (int i = 2; i < 6; ++i) SHAPE_ASSIGN_CHECK(*in_attrs, i, kScalarShape);
  SHAPE_ASSIGN_CHECK(*out_attrs, 0, lshape);
  if (!params.enable_float_output) {
    SHAPE_ASSIGN_CHECK(*out_attrs, 1, kScalarShape);
    SHAPE_ASSIGN_CHECK(*out_attrs, 2, kScalarShape);
  }
  return true;
}

// quantized_elemwise_mul.cc:62-89
static bool ElemwiseMulType(const NodeAttrs& attrs, std::vector<int>* in_type,
                            std::vector<int>* out_type) {
  const auto& params = nnvm::get<QuantizeElemwiseMulParam>(attrs.parsed);
  for (int i = 0; i < 2; ++i) {
    if (in_type->at(i) == mshadow::kInt8) {
      TYPE_ASSIGN_CHECK(*in_type, i, mshadow::kInt8);
    } else {
      std::cerr << "currently, quantized elemwise mul only support int8 inputs." << std::endl;
    }
  }
  for (int i = 2; i < 6; ++i) TYPE_ASSIGN_CHECK(*in_type, i, mshadow::kFloat32);
  int dtype = mshadow::kInt32;
  if (params.max_calib_range.has_value() && params.min_calib_range.has_value())
    dtype = mshadow::kInt8;
  if (!params.enable_float_output) {
    TYPE_ASSIGN_CHECK(*out_type, 0, dtype);
    TYPE_ASSIGN_CHECK(*out_type, 1, mshadow::kFloat32);
    TYPE_ASSIGN_CHECK(*out_type, 2, mshadow::kFloat32);
  } else {
    TYPE_ASSIGN_CHECK(*out_type, 0, mshadow::kFloat32);
  }
  return true;
}

// quantized_elemwise_mul.cc:114-206
static void QuantizedElemwiseMulForwardGPU(const NodeAttrs& attrs, const OpContext& ctx,
                                           const std::vector<TBlob>& inputs,
                                           const std::vector<OpReqType>&,
                                           const std::vector<TBlob>& outputs) {
  const auto& params = nnvm::get<QuantizeElemwiseMulParam>(attrs.parsed);
  CHECK_EQ(inputs.size(), 6U);
  CHECK_EQ(outputs.size(), params.enable_float_output ? 1U : 3U);
  CHECK(inputs[0].type_flag_ == mshadow::kInt8 && inputs[1].type_flag_ == mshadow::kInt8)
      << "lhs and rhs only support iny8 dtype.";
  CHECK_EQ(inputs[0].Size(), inputs[1].Size());
  const bool calibrated = params.max_calib_range.has_value() && params.min_calib_range.has_value();
  MXQ_CALL(mxq_quantized_elemwise_mul(
      raw_stream(ctx), inputs[0].dptr<int8_t>(), inputs[1].dptr<int8_t>(),
      inputs[2].dptr<float>(), inputs[3].dptr<float>(), inputs[4].dptr<float>(),
      inputs[5].dptr<float>(), outputs[0].dptr_, outputs[0].type_flag_,
      params.enable_float_output ? nullptr : outputs[1].dptr<float>(),
      params.enable_float_output ? nullptr : outputs[2].dptr<float>(), outputs[0].Size(),
      calibrated ? 1 : 0, calibrated ? params.min_calib_range.value() : 0.f,
      calibrated ? params.max_calib_range.value() : 0.f));
}

// ---- _contrib_quantized_embedding -----------------------------------------------------------

// quantized_indexing_op.cc:30-52
static bool QuantizedEmbeddingShape(const NodeAttrs& attrs, ShapeVector* in_attrs,
                                    ShapeVector* out_attrs) {
  const TShape& dshape = (*in_attrs)[0];
  if (!ndim_is_known(dshape)) return false;
  const EmbeddingParam& param = nnvm::get<EmbeddingParam>(attrs.parsed);
  SHAPE_ASSIGN_CHECK(*in_attrs, 1, Shape2(param.input_dim, param.output_dim));
  SHAPE_ASSIGN_CHECK(*in_attrs, 2, kScalarShape);
  SHAPE_ASSIGN_CHECK(*in_attrs, 3, kScalarShape);
  out_attrs->clear();
  TShape oshape(dshape.ndim() + 1, -1);
  for (int i = 0; i < dshape.ndim(); ++i) oshape[i] = dshape[i];
  oshape[dshape.ndim()] = param.output_dim;
  out_attrs->push_back(oshape);
  out_attrs->push_back(kScalarShape);
  out_attrs->push_back(kScalarShape);
  return shape_is_known(oshape);
}

// quantized_indexing_op.cc:54-71 (the two range outputs are float32 = type flag 0)
static bool QuantizedEmbeddingType(const NodeAttrs&, std::vector<int>* in_type,
                                   std::vector<int>* out_type) {
  CHECK_EQ(in_type->size(), 4U);
  CHECK_GE(out_type->size(), 3U);
  const int itype = (*in_type)[0];
  CHECK_NE(itype, -1) << "First input must have specified type";
  TYPE_ASSIGN_CHECK(*in_type, 1, mshadow::kInt8);
  TYPE_ASSIGN_CHECK(*in_type, 2, mshadow::kFloat32);
  TYPE_ASSIGN_CHECK(*in_type, 3, mshadow::kFloat32);
  out_type->clear();
  out_type->push_back(mshadow::kInt8);
  out_type->push_back(mshadow::kFloat32);
  out_type->push_back(mshadow::kFloat32);
  return true;
}

// quantized_indexing_op.cc:103-122
static void QuantizedEmbeddingForwardGPU(const NodeAttrs&, const OpContext& ctx,
                                         const std::vector<TBlob>& inputs,
                                         const std::vector<OpReqType>& req,
                                         const std::vector<TBlob>& outputs) {
  CHECK_EQ(req[0], kWriteTo);
  CHECK_EQ(inputs.size(), 4U);
  CHECK_EQ(outputs.size(), 3U);
  CHECK_EQ(inputs[1].shape_.ndim(), 2)
      << "Embedding layer expects its weight to be two-dimensional. " << inputs[1].shape_.ndim()
      << " dimensional input is given instead";
  CHECK_EQ(inputs[1].type_flag_, mshadow::kInt8);
  const TShape& w = inputs[1].shape_;
  MXQ_CALL(mxq_quantized_embedding(raw_stream(ctx), inputs[0].dptr_, inputs[0].type_flag_,
                                   inputs[1].dptr<int8_t>(), inputs[2].dptr<float>(),
                                   inputs[3].dptr<float>(), outputs[0].dptr<int8_t>(),
                                   outputs[1].dptr<float>(), outputs[2].dptr<float>(),
                                   inputs[0].Size(), w[0], w[1]));
}

// ---- _contrib_quantized_reshape -------------------------------------------------------------

namespace {

// matrix_op-inl.h:95-182: the special values of `shape`
TShape InferReshapeShape(const TShape& shape, const TShape& dshape, bool reverse) {
  std::vector<index_t> dshape_vec, param_shape_vec;
  for (int i = 0; i < dshape.ndim(); ++i) dshape_vec.push_back(dshape[i]);
  for (int i = 0; i < shape.ndim(); ++i) param_shape_vec.push_back(shape[i]);
  std::vector<index_t> tmp;
  size_t src_idx = 0;
  int inf_idx = -1;
  if (reverse) {
    std::reverse(dshape_vec.begin(), dshape_vec.end());
    std::reverse(param_shape_vec.begin(), param_shape_vec.end());
  }
  const size_t dshape_len = dshape_vec.size(), params_len = param_shape_vec.size();
  for (size_t i = 0; i < params_len; ++i) {
    const index_t proposed_dim = param_shape_vec[i];
    if (proposed_dim == 0) {
      CHECK_LT(src_idx, dshape_len);
      tmp.push_back(dshape_vec[src_idx++]);
    } else if (proposed_dim == -1) {
      CHECK_LT(inf_idx, 0) << "One and only one dim can be inferred";
      inf_idx = static_cast<int>(i);
      tmp.push_back(1);
      src_idx++;
    } else if (proposed_dim == -2) {
      while (src_idx < dshape_len) tmp.push_back(dshape_vec[src_idx++]);
    } else if (proposed_dim == -3) {
      CHECK_LT(src_idx, dshape_len - 1);
      const index_t d1 = dshape_vec[src_idx++];
      const index_t d2 = dshape_vec[src_idx++];
      tmp.push_back((d1 < 0 || d2 < 0) ? -1 : d1 * d2);
    } else if (proposed_dim == -4) {
      CHECK_LT(i + 2, params_len);
      CHECK_LT(src_idx, dshape_len);
      const index_t d0 = dshape_vec[src_idx++];
      index_t d1 = param_shape_vec[++i];
      index_t d2 = param_shape_vec[++i];
      CHECK(d1 != -1 || d2 != -1) << "Split dims cannot both be -1.";
      if (d1 == -1 && d0 >= 0) d1 = d0 / d2;
      if (d2 == -1 && d0 >= 0) d2 = d0 / d1;
      CHECK(d1 * d2 == d0 || d0 == -1)
          << "Split dims " << d1 << ", " << d2 << " do not divide original dim " << d0;
      tmp.push_back(d1);
      tmp.push_back(d2);
    } else {
      tmp.push_back(proposed_dim);
      src_idx++;
    }
  }
  if (inf_idx >= 0) {
    if (shape_is_known(dshape)) {
      index_t new_size = 1;
      for (index_t x : tmp) new_size *= x;
      tmp[inf_idx] = static_cast<index_t>(dshape.Size()) / new_size;
    } else {
      tmp[inf_idx] = -1;
    }
  }
  if (reverse) std::reverse(tmp.begin(), tmp.end());
  return TShape(tmp);
}

// matrix_op-inl.h:184-205
bool ReverseReshapeInferShape(TShape* in, const TShape& out) {
  if (shape_is_known(*in) && shape_is_known(out)) return true;
  if (!shape_is_known(out)) return false;
  int zero_axis = -1;
  index_t known_dim_size_prod = 1;
  for (int i = 0; i < in->ndim(); i++) {
    if (!dim_size_is_known(*in, i)) {
      if (zero_axis != -1) return false;
      zero_axis = i;
    } else {
      known_dim_size_prod *= (*in)[i];
    }
  }
  (*in)[zero_axis] = static_cast<index_t>(out.Size()) / known_dim_size_prod;
  return true;
}

// matrix_op-inl.h:206-250
bool ReshapeShape(const NodeAttrs& attrs, ShapeVector* in_attrs, ShapeVector* out_attrs) {
  const ReshapeParam& param_ = nnvm::get<ReshapeParam>(attrs.parsed);
  CHECK_EQ(in_attrs->size(), 1U) << "Input: [data]";
  CHECK_EQ(out_attrs->size(), 1U);
  TShape& dshape = (*in_attrs)[0];
  if (!ndim_is_known(dshape)) return false;
  TShape oshape;
  if (param_.shape.ndim() != 0) {
    oshape = InferReshapeShape(param_.shape, dshape, param_.reverse);
  } else if (param_.target_shape.ndim() != 0) {
    oshape = param_.target_shape;
    int neg_count = 0;
    int inf_idx = 0;
    const int start_idx = param_.keep_highest ? 1 : 0;
    if (param_.keep_highest) oshape[0] = dshape[0];
    for (int i = start_idx; i < oshape.ndim(); ++i) {
      if (oshape[i] == 0) {
        neg_count++;
        inf_idx = i;
      }
    }
    if (neg_count == 1) {
      oshape[inf_idx] = 1;
      oshape[inf_idx] = static_cast<index_t>(dshape.Size() / oshape.Size());
    }
  } else {
    return shape_is_known((*out_attrs)[0]) &&
           ReverseReshapeInferShape(&(*in_attrs)[0], (*out_attrs)[0]);
  }
  ReverseReshapeInferShape(&dshape, oshape);
  SHAPE_ASSIGN_CHECK(*out_attrs, 0, oshape);
  return ReverseReshapeInferShape(&(*in_attrs)[0], (*out_attrs)[0]);
}

// np_matrix_op.cc:180-289
bool NumpyXReshapeInferShape(const TShape& src, const TShape& target, TShape* output,
                             const std::string& default_error_msg) {
  bool target_shape_is_known = true;
  index_t target_size = 1;
  for (int i = 0; i < target.ndim(); ++i) {
    if (target[i] < 0) {
      target_shape_is_known = false;
      target_size = -1;
      break;
    }
    target_size *= target[i];
  }
  if (shape_is_known(src) && target_shape_is_known) {
    CHECK_EQ(static_cast<index_t>(src.Size()), target_size) << default_error_msg;
    *output = target;
    return true;
  }
  if (!shape_is_known(src) || target.ndim() == -1) return false;
  int unknown_axis = -1;
  index_t known_dim_size_prod = 1;
  std::vector<index_t> out;
  int src_inx = 0;
  for (int i = 0; i < target.ndim(); ++i) {
    const index_t proposed_dim = target[i];
    CHECK(proposed_dim >= -6) << "Dimension size must be greater than -6, received "
                              << proposed_dim;
    if (proposed_dim == -1) {
      CHECK_LT(unknown_axis, 0) << "One and only one dim can be inferred";
      unknown_axis = static_cast<int>(out.size());
      out.push_back(-1);
      src_inx++;
    } else if (proposed_dim == -2) {
      CHECK_LT(src_inx, src.ndim()) << "Unmatching dimension of proposed new shape";
      known_dim_size_prod *= src[src_inx];
      out.push_back(src[src_inx++]);
    } else if (proposed_dim == -3) {
      CHECK_LT(src_inx, src.ndim()) << "Unmatching dimension of proposed new shape";
      CHECK_EQ(src[src_inx], 1) << "-3 index should only be used to skip dimension size 1";
      src_inx++;
    } else if (proposed_dim == -4) {
      while (src_inx < src.ndim()) {
        known_dim_size_prod *= src[src_inx];
        out.push_back(src[src_inx++]);
      }
    } else if (proposed_dim == -5) {
      CHECK_LT(src_inx, src.ndim() - 1) << "Not enough dimensions left for the product";
      const index_t d1 = src[src_inx++];
      const index_t d2 = src[src_inx++];
      known_dim_size_prod *= d1 * d2;
      out.push_back(d1 * d2);
    } else if (proposed_dim == -6) {
      CHECK_LT(i + 2, target.ndim());
      CHECK_LT(src_inx, src.ndim());
      const index_t d0 = src[src_inx++];
      index_t d1 = target[++i];
      index_t d2 = target[++i];
      CHECK(d1 != -1 || d2 != -1) << "Split dims cannot both be -1.";
      CHECK(d1 != 0 && d2 != 0) << "Split dims " << d1 << ", " << d2
                                << " do not divide original dim " << d0;
      if (d1 == -1) d1 = d0 / d2;
      if (d2 == -1) d2 = d0 / d1;
      CHECK(d1 * d2 == d0) << "Split dims " << d1 << ", " << d2
                           << " do not divide original dim " << d0;
      known_dim_size_prod *= d0;
      out.push_back(d1);
      out.push_back(d2);
    } else {
      known_dim_size_prod *= proposed_dim;
      out.push_back(proposed_dim);
      src_inx++;
    }
  }
  if (unknown_axis > -1) {
    CHECK_NE(known_dim_size_prod, 0) << default_error_msg;
    CHECK(static_cast<index_t>(src.Size()) % known_dim_size_prod == 0) << default_error_msg;
    out[unknown_axis] = static_cast<index_t>(src.Size()) / known_dim_size_prod;
  }
  *output = TShape(out);
  CHECK_EQ(output->Size(), src.Size()) << default_error_msg;
  return true;
}

// np_matrix_op.cc:291-327
bool NumpyXReshapeShape(const NodeAttrs& attrs, ShapeVector* in_attrs, ShapeVector* out_attrs) {
  CHECK_EQ(in_attrs->size(), 1U) << "Input: [data]";
  CHECK_EQ(out_attrs->size(), 1U);
  const NumpyXReshapeParam& param = nnvm::get<NumpyXReshapeParam>(attrs.parsed);
  CHECK(param.order == "C") << "only C-like index order is supported, got " << param.order;
  bool has_unknown_dim_size = false;
  for (int i = 0; i < param.newshape.ndim(); ++i) {
    if (param.newshape[i] < 0) {
      CHECK_GE(param.newshape[i], -6) << "Dimension size must be greater than or equal to -6";
      if (param.newshape[i] == -1) {
        CHECK(!has_unknown_dim_size) << "Can only specify one unknown dimension";
        has_unknown_dim_size = true;
      }
    }
  }
  TShape output_shape;
  bool success;
  std::ostringstream ss;
  ss << "Cannot reshape array of shape " << in_attrs->at(0) << " into shape " << param.newshape
     << " , reverse = " << param.reverse;
  if (!param.reverse) {
    success = NumpyXReshapeInferShape(in_attrs->at(0), param.newshape, &output_shape, ss.str());
  } else {
    std::vector<index_t> rin, rnew;
    for (int i = in_attrs->at(0).ndim() - 1; i >= 0; --i) rin.push_back(in_attrs->at(0)[i]);
    for (int i = param.newshape.ndim() - 1; i >= 0; --i) rnew.push_back(param.newshape[i]);
    if (!ndim_is_known(in_attrs->at(0))) return false;
    success = NumpyXReshapeInferShape(TShape(rin), TShape(rnew), &output_shape, ss.str());
    if (success) {
      std::vector<index_t> rev;
      for (int i = output_shape.ndim() - 1; i >= 0; --i) rev.push_back(output_shape[i]);
      output_shape = TShape(rev);
    }
  }
  if (!success) return false;
  SHAPE_ASSIGN_CHECK(*out_attrs, 0, output_shape);
  return true;
}

}  // namespace

// quantized_reshape-inl.h:38-56
template <bool (*Inner)(const NodeAttrs&, ShapeVector*, ShapeVector*)>
static bool QuantizedReshapeShape(const NodeAttrs& attrs, ShapeVector* in_attrs,
                                  ShapeVector* out_attrs) {
  CHECK_EQ(in_attrs->size(), 3U);
  CHECK_EQ(out_attrs->size(), 3U);
  ShapeVector input = {in_attrs->at(0)};
  ShapeVector output = {out_attrs->at(0)};
  const bool ret = Inner(attrs, &input, &output);
  SHAPE_ASSIGN_CHECK(*in_attrs, 1, kScalarShape);
  SHAPE_ASSIGN_CHECK(*in_attrs, 2, kScalarShape);
  SHAPE_ASSIGN_CHECK(*out_attrs, 0, output[0]);
  SHAPE_ASSIGN_CHECK(*out_attrs, 1, kScalarShape);
  SHAPE_ASSIGN_CHECK(*out_attrs, 2, kScalarShape);
  return ret;
}

// quantized_reshape-inl.h:58-68 and quantized_transpose.cc:31-42: the data keeps its type
static bool PassThroughType(const NodeAttrs&, std::vector<int>* in_attrs,
                            std::vector<int>* out_attrs) {
  CHECK_EQ(in_attrs->size(), 3U);
  CHECK_EQ(out_attrs->size(), 3U);
  TYPE_ASSIGN_CHECK(*in_attrs, 1, mshadow::kFloat32);
  TYPE_ASSIGN_CHECK(*in_attrs, 2, mshadow::kFloat32);
  TYPE_ASSIGN_CHECK(*out_attrs, 0, (*in_attrs)[0]);
  TYPE_ASSIGN_CHECK(*out_attrs, 1, mshadow::kFloat32);
  TYPE_ASSIGN_CHECK(*out_attrs, 2, mshadow::kFloat32);
  return (*in_attrs)[0] != -1;
}

// quantized_reshape.cc:31-46: an identity copy unless the engine runs it in place
static void QuantizedReshapeComputeGPU(const NodeAttrs&, const OpContext& ctx,
                                       const std::vector<TBlob>& inputs,
                                       const std::vector<OpReqType>& req,
                                       const std::vector<TBlob>& outputs) {
  CHECK_EQ(inputs.size(), 3U);
  CHECK_EQ(outputs.size(), 3U);
  CHECK_EQ(req.size(), 3U);
  CHECK(inputs[0].type_flag_ == mshadow::kInt8 || inputs[0].type_flag_ == mshadow::kUint8)
      << "quantized_reshape takes int8 or uint8 data";
  CHECK_EQ(inputs[0].Size(), outputs[0].Size());
  // in place: mxq_quantized_flatten copies nothing where in == out
  MXQ_CALL(mxq_quantized_flatten(raw_stream(ctx), inputs[0].dptr_, inputs[1].dptr<float>(),
                                 inputs[2].dptr<float>(),
                                 req[0] == kWriteInplace ? inputs[0].dptr_ : outputs[0].dptr_,
                                 outputs[1].dptr<float>(), outputs[2].dptr<float>(),
                                 outputs[0].Size()));
}

// ---- _contrib_quantized_transpose -----------------------------------------------------------

namespace {

// matrix_op-inl.h:579-613
bool TransposeShape(const NodeAttrs& attrs, ShapeVector* in_attrs, ShapeVector* out_attrs) {
  const TransposeParam& param = nnvm::get<TransposeParam>(attrs.parsed);
  CHECK_EQ(in_attrs->size(), 1U);
  CHECK_EQ(out_attrs->size(), 1U);
  TShape& shp = (*in_attrs)[0];
  TShape& out_shp = (*out_attrs)[0];
  if (!ndim_is_known(shp) && !ndim_is_known(out_shp)) return false;
  if (out_shp.ndim() >= 0 && shp.ndim() >= 0) CHECK_EQ(out_shp.ndim(), shp.ndim());
  const int nd = std::max(shp.ndim(), out_shp.ndim());
  TShape get(nd, -1), ret(nd, -1);
  if (param.axes.ndim() == 0) {
    for (int i = 0; i < shp.ndim(); ++i) ret[i] = shp[shp.ndim() - 1 - i];
    for (int i = 0; i < out_shp.ndim(); ++i) get[nd - 1 - i] = out_shp[i];
  } else {
    CHECK_EQ(nd, param.axes.ndim());
    for (int i = 0; i < shp.ndim(); ++i) {
      CHECK(param.axes[i] < static_cast<index_t>(shp.ndim()));
      ret[i] = shp[static_cast<int>(param.axes[i])];
    }
    for (int i = 0; i < out_shp.ndim(); ++i) get[static_cast<int>(param.axes[i])] = out_shp[i];
  }
  SHAPE_ASSIGN_CHECK(*in_attrs, 0, get);
  SHAPE_ASSIGN_CHECK(*out_attrs, 0, ret);
  return shape_is_known(ret);
}

// src/common/utils.h:917-929
TShape CanonicalizeAxes(const TShape& src) {
  const int ndim = src.ndim();
  TShape axes = src;
  for (int i = 0; i < ndim; ++i) {
    if (axes[i] < 0) axes[i] += ndim;
    CHECK(axes[i] >= 0 && axes[i] < ndim)
        << "axes[" << i << "]=" << axes[i] << " exceeds the range [" << 0 << ", " << ndim << ")";
  }
  return axes;
}

// np_matrix_op-inl.h:179-234
bool NumpyTransposeShape(const NodeAttrs& attrs, ShapeVector* in_attrs, ShapeVector* out_attrs) {
  const NumpyTransposeParam& param = nnvm::get<NumpyTransposeParam>(attrs.parsed);
  CHECK_EQ(in_attrs->size(), 1U);
  CHECK_EQ(out_attrs->size(), 1U);
  TShape& shp = (*in_attrs)[0];
  TShape& out_shp = (*out_attrs)[0];
  int ndim = -1;
  if (ndim_is_known(shp)) {
    ndim = shp.ndim();
  } else if (ndim_is_known(out_shp)) {
    ndim = out_shp.ndim();
  }
  if (ndim < 0) return false;
  if (out_shp.ndim() >= 0 && shp.ndim() >= 0) CHECK_EQ(out_shp.ndim(), shp.ndim());
  TShape get(ndim, -1), ret(ndim, -1);
  if (ndim_is_known(param.axes)) {
    CHECK_EQ(ndim, param.axes.ndim())
        << "The number of axes does not match the dimension of the tensor. axes = " << param.axes
        << ", input tensor shape = " << shp;
    const TShape axes = CanonicalizeAxes(param.axes);
    std::vector<bool> seen(ndim, false);
    for (int i = 0; i < ndim; ++i) {
      CHECK(!seen[axes[i]]) << "ValueError: Repeated axis in transpose. param.axes = "
                            << param.axes;
      seen[axes[i]] = true;
    }
    if (ndim_is_known(shp))
      for (int i = 0; i < ndim; ++i) ret[i] = shp[static_cast<int>(axes[i])];
    if (ndim_is_known(out_shp))
      for (int i = 0; i < ndim; ++i) get[static_cast<int>(axes[i])] = out_shp[i];
  } else {
    if (ndim_is_known(shp))
      for (int i = 0; i < ndim; ++i) ret[i] = shp[ndim - 1 - i];
    if (ndim_is_known(out_shp))
      for (int i = 0; i < ndim; ++i) get[ndim - 1 - i] = out_shp[i];
  }
  SHAPE_ASSIGN_CHECK(*in_attrs, 0, get);
  SHAPE_ASSIGN_CHECK(*out_attrs, 0, ret);
  return shape_is_known((*in_attrs)[0]) && shape_is_known((*out_attrs)[0]);
}

// the permutation an operator instance applies to data of `ndim` axes; empty = reverse
std::vector<int> transpose_axes(const TransposeParam& param, int) {
  std::vector<int> axes(param.axes.ndim());
  for (int i = 0; i < param.axes.ndim(); ++i) axes[i] = static_cast<int>(param.axes[i]);
  return axes;
}
std::vector<int> transpose_axes(const NumpyTransposeParam& param, int ndim) {
  std::vector<int> axes;
  if (!ndim_is_known(param.axes)) return axes;
  CHECK_EQ(param.axes.ndim(), ndim);
  const TShape canon = CanonicalizeAxes(param.axes);
  for (int i = 0; i < ndim; ++i) axes.push_back(static_cast<int>(canon[i]));
  if (axes.empty()) axes.push_back(0);  // never reached with data: 0-d has nothing to permute
  return axes;
}

}  // namespace

// quantized_transpose.cc:49-66
template <bool (*Inner)(const NodeAttrs&, ShapeVector*, ShapeVector*)>
static bool QuantizedTransposeShape(const NodeAttrs& attrs, ShapeVector* in_attrs,
                                    ShapeVector* out_attrs) {
  CHECK_EQ(in_attrs->size(), 3U);
  CHECK_EQ(out_attrs->size(), 3U);
  ShapeVector qin_attrs(1), qout_attrs(1);
  SHAPE_ASSIGN_CHECK(qin_attrs, 0, (*in_attrs)[0]);
  SHAPE_ASSIGN_CHECK(qout_attrs, 0, (*out_attrs)[0]);
  const bool ret = Inner(attrs, &qin_attrs, &qout_attrs);
  SHAPE_ASSIGN_CHECK(*in_attrs, 0, qin_attrs[0]);
  SHAPE_ASSIGN_CHECK(*out_attrs, 0, qout_attrs[0]);
  SHAPE_ASSIGN_CHECK(*in_attrs, 1, kScalarShape);
  SHAPE_ASSIGN_CHECK(*in_attrs, 2, kScalarShape);
  SHAPE_ASSIGN_CHECK(*out_attrs, 1, kScalarShape);
  SHAPE_ASSIGN_CHECK(*out_attrs, 2, kScalarShape);
  return ret;
}

// dnnl_quantized_transpose.cc: the float transpose on one-byte elements, ranges copied
template <typename Param>
static void QuantizedTransposeForwardGPU(const NodeAttrs& attrs, const OpContext& ctx,
                                         const std::vector<TBlob>& inputs,
                                         const std::vector<OpReqType>& req,
                                         const std::vector<TBlob>& outputs) {
  const Param& param = nnvm::get<Param>(attrs.parsed);
  CHECK_EQ(inputs.size(), 3U);
  CHECK_EQ(outputs.size(), 3U);
  CHECK(req[0] == kWriteTo) << "Transpose does not support inplace";
  CHECK(inputs[0].type_flag_ == mshadow::kInt8 || inputs[0].type_flag_ == mshadow::kUint8)
      << "quantized_transpose takes int8 or uint8 data";
  const TShape& shp = inputs[0].shape_;
  std::vector<int64_t> dims(shp.ndim());
  for (int i = 0; i < shp.ndim(); ++i) dims[i] = shp[i];
  std::vector<int> axes = transpose_axes(param, shp.ndim());
  if (shp.ndim() == 0) axes.clear();
  if (!axes.empty()) CHECK_EQ(axes.size(), dims.size());
  MXQ_CALL(mxq_quantized_transpose(raw_stream(ctx), inputs[0].dptr_, inputs[1].dptr<float>(),
                                   inputs[2].dptr<float>(), outputs[0].dptr_,
                                   outputs[1].dptr<float>(), outputs[2].dptr<float>(),
                                   shp.ndim(), dims.data(), axes.empty() ? nullptr : axes.data()));
}

// ---- _contrib_quantize_asym -----------------------------------------------------------------

// quantize_asym.cc:36-54
static bool QuantizeAsymShape(const NodeAttrs&, ShapeVector* in_attrs, ShapeVector* out_attrs) {
  CHECK_EQ(in_attrs->size(), 1U);
  CHECK_EQ(out_attrs->size(), 3U);
  TShape dshape = in_attrs->at(0);
  SHAPE_ASSIGN_CHECK(*out_attrs, 0, dshape);
  SHAPE_ASSIGN_CHECK(*out_attrs, 1, kScalarShape);
  SHAPE_ASSIGN_CHECK(*out_attrs, 2, kScalarShape);
  if (out_attrs->at(0).ndim() > 0) {
    dshape[0] = out_attrs->at(0)[0];
    SHAPE_ASSIGN_CHECK(*in_attrs, 0, dshape);
  }
  return !shape_is_none(out_attrs->at(0));
}

// quantize_asym.cc:56-69
static bool QuantizeAsymType(const NodeAttrs&, std::vector<int>* in_attrs,
                             std::vector<int>* out_attrs) {
  CHECK_EQ(in_attrs->size(), 1U);
  CHECK_EQ(out_attrs->size(), 3U);
  CHECK_EQ(in_attrs->at(0), mshadow::kFloat32);
  TYPE_ASSIGN_CHECK(*out_attrs, 0, mshadow::kUint8);
  TYPE_ASSIGN_CHECK(*out_attrs, 1, mshadow::kFloat32);
  TYPE_ASSIGN_CHECK(*out_attrs, 2, mshadow::kFloat32);
  return out_attrs->at(0) != -1;
}

// quantize_asym-inl.h:78-160.  The operator state only carries the attributes.
class QuantizeAsymOperatorGPU {
 public:
  explicit QuantizeAsymOperatorGPU(const NodeAttrs& attrs) : attrs_(attrs) {}
  void Forward(const OpContext& ctx, const std::vector<TBlob>& inputs,
               const std::vector<OpReqType>&, const std::vector<TBlob>& outputs) {
    CHECK_EQ(outputs[0].type_flag_, mshadow::kUint8)
        << "Asymmetric quantization only supports uint8 outputs.";
    const auto& param = nnvm::get<QuantizeAsymParam>(attrs_.parsed);
    const bool calibrated = param.min_calib_range.has_value() && param.max_calib_range.has_value();
    void* ws = nullptr;
    size_t ws_bytes = 0;
    if (inputs[0].type_flag_ == mshadow::kFloat32 && !calibrated) {
      CHECK(!ctx.requested.empty()) << "uncalibrated quantize_asym needs its temp space resource";
      ws_bytes = mxq_quantize_asym_workspace(inputs[0].Size());
      ws = ctx.requested[0].get_space(ws_bytes);
    }
    MXQ_CALL(mxq_quantize_asym(raw_stream(ctx), inputs[0].dptr_, inputs[0].type_flag_,
                               outputs[0].dptr<uint8_t>(), outputs[1].dptr<float>(),
                               outputs[2].dptr<float>(), inputs[0].Size(), calibrated ? 1 : 0,
                               calibrated ? param.min_calib_range.value() : 0.f,
                               calibrated ? param.max_calib_range.value() : 0.f, ws, ws_bytes));
  }

 private:
  NodeAttrs attrs_;
};

static OpStatePtr CreateQuantizeAsymState(const NodeAttrs& attrs, Context ctx, const ShapeVector&,
                                          const std::vector<int>&) {
  CHECK(ctx.dev_type == Context::kGPU) << "this build only provides the gpu operator";
  return OpStatePtr::Create<QuantizeAsymOperatorGPU>(attrs);
}

static void QuantizeAsymForwardGPU(const OpStatePtr& state, const OpContext& ctx,
                                   const std::vector<TBlob>& inputs,
                                   const std::vector<OpReqType>& req,
                                   const std::vector<TBlob>& outputs) {
  state.get_state<QuantizeAsymOperatorGPU>().Forward(ctx, inputs, req, outputs);
}

// ---- _contrib_quantized_batch_norm(_relu) -----------------------------------------------------

// quantized_batch_norm.cc:34-61
static bool QuantizedBatchNormShape(const NodeAttrs& attrs, ShapeVector* in_shape,
                                    ShapeVector* out_shape) {
  const BatchNormParam& param = nnvm::get<BatchNormParam>(attrs.parsed);
  CHECK_EQ(in_shape->size(), 7U)
      << "Input:[data, gamma, beta, moving_mean, moving_var, min_data, max_data]";
  CHECK_EQ(out_shape->size(), 3U);
  const TShape& dshape = in_shape->at(0);
  if (!ndim_is_known(dshape)) return false;
  const int channelAxis = param.axis < 0 ? dshape.ndim() + param.axis : param.axis;
  CHECK(channelAxis >= 0 && channelAxis < dshape.ndim())
      << "Channel axis out of range: " << param.axis;
  const index_t channelCount = dshape[channelAxis];
  for (int i = 1; i < 5; ++i) SHAPE_ASSIGN_CHECK(*in_shape, i, Shape1(channelCount));
  SHAPE_ASSIGN_CHECK(*in_shape, 5, kScalarShape);
  SHAPE_ASSIGN_CHECK(*in_shape, 6, kScalarShape);
  SHAPE_ASSIGN_CHECK(*out_shape, 0, dshape);
  SHAPE_ASSIGN_CHECK(*out_shape, 1, kScalarShape);
  SHAPE_ASSIGN_CHECK(*out_shape, 2, kScalarShape);
  return true;
}

// quantized_batch_norm.cc:63-87 (the oneDNN branch: int8 or uint8 data)
static bool QuantizedBatchNormType(const NodeAttrs&, std::vector<int>* in_type,
                                   std::vector<int>* out_type) {
  CHECK_EQ(in_type->size(), 7U);
  CHECK_EQ(out_type->size(), 3U);
  CHECK(in_type->at(0) == mshadow::kInt8 || in_type->at(0) == mshadow::kUint8)
      << "QuantizedBatchNorm only supports int8/uint8 input, while " << in_type->at(0)
      << " is given.";
  for (size_t i = 1; i < 7; ++i) TYPE_ASSIGN_CHECK(*in_type, i, mshadow::kFloat32);
  TYPE_ASSIGN_CHECK(*out_type, 0, mshadow::kInt8);
  TYPE_ASSIGN_CHECK(*out_type, 1, mshadow::kFloat32);
  TYPE_ASSIGN_CHECK(*out_type, 2, mshadow::kFloat32);
  return true;
}

// dnnl_quantized_batch_norm.cc:34-130
template <bool fuse_relu>
static void QuantizedBatchNormForwardGPU(const NodeAttrs& attrs, const OpContext& ctx,
                                         const std::vector<TBlob>& inputs,
                                         const std::vector<OpReqType>&,
                                         const std::vector<TBlob>& outputs) {
  CHECK_EQ(inputs.size(), 7U);
  CHECK_EQ(outputs.size(), 3U);
  const BatchNormParam& param = nnvm::get<BatchNormParam>(attrs.parsed);
  CHECK(param.min_calib_range.has_value() && param.max_calib_range.has_value())
      << "min_calib_range or max_calib_range is not available. Quantized BN currently "
         "don't support calib_mode=None";
  const TShape& shp = inputs[0].shape_;
  const int axis = param.axis < 0 ? shp.ndim() + param.axis : param.axis;
  CHECK(axis >= 0 && axis < shp.ndim()) << "Channel axis out of range: " << param.axis;
  int64_t outer = 1, inner = 1;
  for (int i = 0; i < axis; ++i) outer *= shp[i];
  for (int i = axis + 1; i < shp.ndim(); ++i) inner *= shp[i];
  CHECK(!ctx.requested.empty()) << "quantized batch norm needs its temp space resource";
  const size_t ws_bytes = mxq_quantized_batch_norm_workspace(shp[axis]);
  void* ws = ctx.requested[0].get_space(ws_bytes);
  MXQ_CALL(mxq_quantized_batch_norm(
      raw_stream(ctx), inputs[0].dptr_, inputs[0].type_flag_, inputs[1].dptr<float>(),
      inputs[2].dptr<float>(), inputs[3].dptr<float>(), inputs[4].dptr<float>(),
      inputs[5].dptr<float>(), inputs[6].dptr<float>(), outputs[0].dptr<int8_t>(),
      outputs[1].dptr<float>(), outputs[2].dptr<float>(), outer, shp[axis], inner, param.eps,
      param.min_calib_range.value(), param.max_calib_range.value(), fuse_relu ? 1 : 0, ws,
      ws_bytes));
}

// Temp space of the operators of this file, in bytes.
size_t MXQTensorOpsTempSpaceBytes(const NodeAttrs& attrs, const ShapeVector& in) {
  if (attrs.op->name == "_contrib_quantized_batch_norm" ||
      attrs.op->name == "_contrib_quantized_batch_norm_relu") {
    const BatchNormParam& param = nnvm::get<BatchNormParam>(attrs.parsed);
    const int axis = param.axis < 0 ? in[0].ndim() + param.axis : param.axis;
    return mxq_quantized_batch_norm_workspace(in[0][axis]);
  }
  if (attrs.op->name == "_contrib_quantize_asym") {
    const auto& param = nnvm::get<QuantizeAsymParam>(attrs.parsed);
    if (param.min_calib_range.has_value() && param.max_calib_range.has_value()) return 0;
    return mxq_quantize_asym_workspace(in[0].Size());
  }
  return 0;
}

// ---- registration ---------------------------------------------------------------------------

// quantized_elemwise_mul.cc:208-245
NNVM_REGISTER_OP(_contrib_quantized_elemwise_mul)
    .add_alias("_npx_quantized_elemwise_mul")
    .describe("Multiplies arguments int8 element-wise.")
    .set_num_inputs(6)
    .set_num_outputs([](const NodeAttrs& attrs) {
      return nnvm::get<QuantizeElemwiseMulParam>(attrs.parsed).enable_float_output ? 1U : 3U;
    })
    .set_attr_parser(ParamParser<QuantizeElemwiseMulParam>)
    .set_attr<nnvm::FListInputNames>("FListInputNames",
                                     [](const NodeAttrs&) {
                                       return std::vector<std::string>{"lhs",     "rhs",
                                                                       "lhs_min", "lhs_max",
                                                                       "rhs_min", "rhs_max"};
                                     })
    .set_attr<mxnet::FInferShape>("FInferShape", ElemwiseMulShape)
    .set_attr<nnvm::FInferType>("FInferType", ElemwiseMulType)
    .set_attr<FInferStorageType>("FInferStorageType", AllDefaultStorage)
    .set_attr<FCompute>("FCompute<gpu>", QuantizedElemwiseMulForwardGPU)
    .set_attr<FNeedRequantize>("FNeedRequantize", [](const NodeAttrs&) { return true; })
    .add_argument("lhs", "NDArray-or-Symbol", "first input")
    .add_argument("rhs", "NDArray-or-Symbol", "second input")
    .add_argument("lhs_min", "NDArray-or-Symbol", "Minimum value of first input.")
    .add_argument("lhs_max", "NDArray-or-Symbol", "Maximum value of first input.")
    .add_argument("rhs_min", "NDArray-or-Symbol", "Minimum value of second input.")
    .add_argument("rhs_max", "NDArray-or-Symbol", "Maximum value of second input.")
    .add_arguments(QuantizeElemwiseMulParam::__FIELDS__());

// quantized_indexing_op.cc:124-160
NNVM_REGISTER_OP(_contrib_quantized_embedding)
    .add_alias("_npx_quantized_embedding")
    .describe("Maps integer indices to int8 vector representations (embeddings).")
    .set_num_inputs(4)
    .set_num_outputs(3)
    .set_attr_parser(ParamParser<EmbeddingParam>)
    .set_attr<nnvm::FListInputNames>("FListInputNames",
                                     [](const NodeAttrs&) {
                                       return std::vector<std::string>{"data", "weight",
                                                                       "min_weight",
                                                                       "max_weight"};
                                     })
    .set_attr<nnvm::FListOutputNames>("FListOutputNames", OutputMinMax)
    .set_attr<mxnet::FInferShape>("FInferShape", QuantizedEmbeddingShape)
    .set_attr<nnvm::FInferType>("FInferType", QuantizedEmbeddingType)
    .set_attr<FInferStorageType>("FInferStorageType", AllDefaultStorage)
    .set_attr<FCompute>("FCompute<gpu>", QuantizedEmbeddingForwardGPU)
    .add_argument("data", "NDArray-or-Symbol", "The input array to the embedding operator.")
    .add_argument("weight", "NDArray-or-Symbol", "The embedding weight matrix.")
    .add_argument("min_weight", "NDArray-or-Symbol", "Minimum value of data.")
    .add_argument("max_weight", "NDArray-or-Symbol", "Maximum value of data.")
    .add_arguments(EmbeddingParam::__FIELDS__());

// quantized_reshape.cc:48-100
NNVM_REGISTER_OP(_contrib_quantized_reshape)
    .add_alias("quantized_reshape")
    .set_num_inputs(3)
    .set_num_outputs(3)
    .set_attr_parser(ParamParser<ReshapeParam>)
    .set_attr<nnvm::FListInputNames>("FListInputNames", DataMinMax)
    .set_attr<nnvm::FListOutputNames>("FListOutputNames", OutputMinMax)
    .set_attr<nnvm::FInplaceOption>("FInplaceOption",
                                    [](const NodeAttrs&) {
                                      return std::vector<std::pair<int, int>>{{0, 0}, {1, 1}, {2, 2}};
                                    })
    .set_attr<mxnet::FInferShape>("FInferShape", QuantizedReshapeShape<ReshapeShape>)
    .set_attr<nnvm::FInferType>("FInferType", PassThroughType)
    .set_attr<FCompute>("FCompute<gpu>", QuantizedReshapeComputeGPU)
    .set_attr<FQuantizable>("FQuantizable",
                            [](const NodeAttrs&) { return QuantizeType::kSupport; })
    .add_argument("data", "NDArray-or-Symbol", "Array to be reshaped.")
    .add_argument("min_data", "NDArray-or-Symbol",
                  "The minimum scalar value possibly produced for the data")
    .add_argument("max_data", "NDArray-or-Symbol",
                  "The maximum scalar value possibly produced for the data")
    .add_arguments(ReshapeParam::__FIELDS__());

// quantized_transpose.cc:68-104
NNVM_REGISTER_OP(_contrib_quantized_transpose)
    .add_alias("quantized_transpose")
    .set_num_inputs(3)
    .set_num_outputs(3)
    .set_attr_parser(ParamParser<TransposeParam>)
    .set_attr<nnvm::FListInputNames>("FListInputNames", DataMinMax)
    .set_attr<nnvm::FListOutputNames>("FListOutputNames", OutputMinMax)
    .set_attr<mxnet::FInferShape>("FInferShape", QuantizedTransposeShape<TransposeShape>)
    .set_attr<nnvm::FInferType>("FInferType", PassThroughType)
    .set_attr<FCompute>("FCompute<gpu>", QuantizedTransposeForwardGPU<TransposeParam>)
    .set_attr<FQuantizable>("FQuantizable",
                            [](const NodeAttrs&) { return QuantizeType::kSupport; })
    .add_argument("data", "NDArray-or-Symbol", "Array to be transposed.")
    .add_argument("min_data", "NDArray-or-Symbol",
                  "The minimum scalar value possibly produced for the data")
    .add_argument("max_data", "NDArray-or-Symbol",
                  "The maximum scalar value possibly produced for the data")
    .add_arguments(TransposeParam::__FIELDS__());

// quantized_reshape.cc:91-100: the numpy-namespace form, newshape with -1 ... -6
NNVM_REGISTER_OP(_npx_quantized_reshape)
    .set_num_inputs(3)
    .set_num_outputs(3)
    .set_attr_parser(ParamParser<NumpyXReshapeParam>)
    .set_attr<nnvm::FListInputNames>("FListInputNames", DataMinMax)
    .set_attr<nnvm::FListOutputNames>("FListOutputNames", OutputMinMax)
    .set_attr<nnvm::FInplaceOption>("FInplaceOption",
                                    [](const NodeAttrs&) {
                                      return std::vector<std::pair<int, int>>{{0, 0}, {1, 1}, {2, 2}};
                                    })
    .set_attr<mxnet::FInferShape>("FInferShape", QuantizedReshapeShape<NumpyXReshapeShape>)
    .set_attr<nnvm::FInferType>("FInferType", PassThroughType)
    .set_attr<FCompute>("FCompute<gpu>", QuantizedReshapeComputeGPU)
    .set_attr<FQuantizable>("FQuantizable",
                            [](const NodeAttrs&) { return QuantizeType::kSupport; })
    .add_argument("data", "NDArray-or-Symbol", "Array to be reshaped.")
    .add_argument("min_data", "NDArray-or-Symbol",
                  "The minimum scalar value possibly produced for the data")
    .add_argument("max_data", "NDArray-or-Symbol",
                  "The maximum scalar value possibly produced for the data")
    .add_arguments(NumpyXReshapeParam::__FIELDS__());

// quantized_transpose.cc:96-99: the numpy-namespace form, negative axes allowed
NNVM_REGISTER_OP(_npx_quantized_transpose)
    .set_num_inputs(3)
    .set_num_outputs(3)
    .set_attr_parser(ParamParser<NumpyTransposeParam>)
    .set_attr<nnvm::FListInputNames>("FListInputNames", DataMinMax)
    .set_attr<nnvm::FListOutputNames>("FListOutputNames", OutputMinMax)
    .set_attr<mxnet::FInferShape>("FInferShape", QuantizedTransposeShape<NumpyTransposeShape>)
    .set_attr<nnvm::FInferType>("FInferType", PassThroughType)
    .set_attr<FCompute>("FCompute<gpu>", QuantizedTransposeForwardGPU<NumpyTransposeParam>)
    .set_attr<FQuantizable>("FQuantizable",
                            [](const NodeAttrs&) { return QuantizeType::kSupport; })
    .add_argument("data", "NDArray-or-Symbol", "Array to be transposed.")
    .add_argument("min_data", "NDArray-or-Symbol",
                  "The minimum scalar value possibly produced for the data")
    .add_argument("max_data", "NDArray-or-Symbol",
                  "The maximum scalar value possibly produced for the data")
    .add_arguments(NumpyTransposeParam::__FIELDS__());

// quantize_asym.cc:100-157
NNVM_REGISTER_OP(_contrib_quantize_asym)
    .describe("Quantize a input tensor from float to uint8_t.  Output `scale` and `shift` are "
              "scalar floats that specify the quantization parameters for the input data: "
              "`out[i] = in[i] * scale + shift + 0.5` with `scale = uint8_range / (max_range - "
              "min_range)` and `shift = numeric_limits<T>::max - max_range * scale`.")
    .set_attr_parser(ParamParser<QuantizeAsymParam>)
    .set_num_inputs(1)
    .set_num_outputs(3)
    .set_attr<nnvm::FListInputNames>("FListInputNames",
                                     [](const NodeAttrs&) {
                                       return std::vector<std::string>{"data"};
                                     })
    .set_attr<nnvm::FListOutputNames>("FListOutputNames",
                                      [](const NodeAttrs&) {
                                        return std::vector<std::string>{"output", "scale",
                                                                        "shift"};
                                      })
    .set_attr<mxnet::FInferShape>("FInferShape", QuantizeAsymShape)
    .set_attr<nnvm::FInferType>("FInferType", QuantizeAsymType)
    .set_attr<FInferStorageType>("FInferStorageType", AllDefaultStorage)
    .set_attr<FCreateOpState>("FCreateOpState", CreateQuantizeAsymState)
    .set_attr<FStatefulCompute>("FStatefulCompute<gpu>", QuantizeAsymForwardGPU)
    .set_attr<FNeedCalibrateInput>("FNeedCalibrateInput",
                                   [](const NodeAttrs&) { return std::vector<int>{0}; })
    .set_attr<FResourceRequest>("FResourceRequest",
                                [](const NodeAttrs& attrs) {
                                  const auto& param =
                                      nnvm::get<QuantizeAsymParam>(attrs.parsed);
                                  if (param.max_calib_range.has_value() &&
                                      param.min_calib_range.has_value())
                                    return std::vector<ResourceRequest>();
                                  return std::vector<ResourceRequest>(
                                      1, ResourceRequest::kTempSpace);
                                })
    .add_argument("data", "NDArray-or-Symbol", "A ndarray/symbol of type `float32`")
    .add_arguments(QuantizeAsymParam::__FIELDS__());

// quantized_batch_norm.cc:89-122 and quantized_batch_norm_relu.cc:88-121, with the resource
// request the oneDNN files attach (dnnl_quantized_batch_norm.cc:150-167).  The reference
// stores its FNeedCalibrateOutput function under that key with the input variant's type.
#define MXQ_REGISTER_QUANTIZED_BATCH_NORM(name, relu, text)                                       \
  NNVM_REGISTER_OP(name)                                                                          \
      .describe(text)                                                                             \
      .set_num_inputs(7)                                                                          \
      .set_num_outputs(3)                                                                         \
      .set_attr_parser(ParamParser<BatchNormParam>)                                               \
      .set_attr<nnvm::FListInputNames>(                                                           \
          "FListInputNames",                                                                      \
          [](const NodeAttrs&) {                                                                  \
            return std::vector<std::string>{"data",       "gamma",    "beta",    "moving_mean",   \
                                            "moving_var", "min_data", "max_data"};                \
          })                                                                                      \
      .set_attr<nnvm::FListOutputNames>("FListOutputNames", OutputMinMax)                         \
      .set_attr<nnvm::FMutateInputs>("FMutateInputs",                                             \
                                     [](const NodeAttrs&) { return std::vector<uint32_t>{3, 4}; }) \
      .set_attr<mxnet::FInferShape>("FInferShape", QuantizedBatchNormShape)                       \
      .set_attr<nnvm::FInferType>("FInferType", QuantizedBatchNormType)                           \
      .set_attr<FInferStorageType>("FInferStorageType", AllDefaultStorage)                        \
      .set_attr<FNeedRequantize>("FNeedRequantize", [](const NodeAttrs&) { return false; })       \
      .set_attr<FNeedCalibrateOutput>("FNeedCalibrateOutput",                                     \
                                      [](const NodeAttrs&) { return std::vector<int>{0}; })       \
      .set_attr<FResourceRequest>("FResourceRequest",                                             \
                                  [](const NodeAttrs&) {                                          \
                                    return std::vector<ResourceRequest>{                          \
                                        ResourceRequest::kTempSpace};                             \
                                  })                                                              \
      .set_attr<FCompute>("FCompute<gpu>", QuantizedBatchNormForwardGPU<relu>)                    \
      .add_argument("data", "NDArray-or-Symbol", "Input data.")                                   \
      .add_argument("gamma", "NDArray-or-Symbol", "gamma.")                                       \
      .add_argument("beta", "NDArray-or-Symbol", "beta.")                                         \
      .add_argument("moving_mean", "NDArray-or-Symbol", "moving_mean.")                           \
      .add_argument("moving_var", "NDArray-or-Symbol", "moving_var.")                             \
      .add_argument("min_data", "NDArray-or-Symbol", "Minimum value of data.")                    \
      .add_argument("max_data", "NDArray-or-Symbol", "Maximum value of data.")                    \
      .add_arguments(BatchNormParam::__FIELDS__())

MXQ_REGISTER_QUANTIZED_BATCH_NORM(
    _contrib_quantized_batch_norm, false,
    "BatchNorm operator for input and output data type of int8.  The input and output data "
    "comes with min and max thresholds for quantizing the float32 data into int8.");
MXQ_REGISTER_QUANTIZED_BATCH_NORM(
    _contrib_quantized_batch_norm_relu, true,
    "BatchNorm with ReLU operator for input and output data type of int8.  The input and "
    "output data comes with min and max thresholds for quantizing the float32 data into int8.");

}  // namespace op
}  // namespace mxnet
