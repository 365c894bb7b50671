// Attribute structs of the quantization operators, parsed from the string dict of
// a node exactly as dmlc::Parameter<...>::Init does for the reference structs:
//   QuantizeV2Param        src/operator/quantization/quantize_v2-inl.h:39-63
//   QuantizeParam (v1)     src/operator/quantization/quantize-inl.h:39-48
//   RequantizeParam        src/operator/quantization/requantize-inl.h:39-65
//   DequantizeParam        src/operator/quantization/dequantize-inl.h:38-46
//   FullyConnectedParam    src/operator/nn/fully_connected-inl.h:70-82
//   ConvolutionParam       src/operator/nn/convolution-inl.h:56-112 (+ the defaults
//                          ConvolutionParamParser fills, src/operator/nn/convolution.cc:366-416)
//   ActivationParam        src/operator/nn/activation-inl.h (act_type only)
//   PoolingParam           src/operator/nn/pooling-inl.h:45-120 (+ PoolingParamParser,
//                          src/operator/nn/pooling.cc:35-64)
//   QuantizeElemwiseAddParam  src/operator/quantization/quantized_elemwise_add-inl.h:34-51
//   ConcatParam            src/operator/nn/concat-inl.h:48-64
//   QuantizeElemwiseMulParam  src/operator/quantization/quantized_elemwise_mul-inl.h:33-55
//   EmbeddingParam         src/operator/tensor/indexing_op.h:66-96
//   ReshapeParam           src/operator/tensor/matrix_op-inl.h:53-80
//   TransposeParam         src/operator/tensor/matrix_op-inl.h:269-280
//   QuantizeAsymParam      src/operator/quantization/quantize_asym-inl.h:41-59
//   BatchNormParam         src/operator/nn/batch_norm-inl.h:87-133
// Same field names, defaults, enum strings and error behaviour (unknown keys are
// errors unless they look like __hidden__ keys).
#ifndef MXQ_PARAMS_H_
#define MXQ_PARAMS_H_

#include <cctype>
#include <cstdlib>
#include <map>
#include <set>
#include <string>
#include <unordered_map>
#include <vector>

#include "mxq_shim.h"

namespace mxnet {
namespace op {

enum QuantizeOutType { kAuto = 0, kInt8, kUint8 };

namespace param_detail {

typedef std::unordered_map<std::string, std::string> Dict;

inline std::string trim(const std::string& s) {
  size_t b = 0, e = s.size();
  while (b < e && std::isspace(static_cast<unsigned char>(s[b]))) ++b;
  while (e > b && std::isspace(static_cast<unsigned char>(s[e - 1]))) --e;
  return s.substr(b, e - b);
}

inline bool is_hidden(const std::string& k) {
  return k.size() > 4 && k.compare(0, 2, "__") == 0 && k.compare(k.size() - 2, 2, "__") == 0;
}

// Fails for keys that no field consumed (dmlc::Parameter::Init, kAllowHidden).
inline void check_unknown(const Dict& d, const std::set<std::string>& known,
                          const char* struct_name) {
  for (const auto& kv : d) {
    if (known.count(kv.first) || is_hidden(kv.first)) continue;
    std::ostringstream os;
    os << "Cannot find argument '" << kv.first << "', Possible Arguments:\n----------------\n";
    for (const auto& k : known) os << k << "\n";
    os << "(in " << struct_name << ")";
    throw dmlc::ParamError(os.str());
  }
}

inline bool parse_float(const std::string& raw, float* out) {
  const std::string s = trim(raw);
  if (s.empty()) return false;
  char* end = nullptr;
  const float v = std::strtof(s.c_str(), &end);
  if (end == s.c_str()) return false;
  while (*end && std::isspace(static_cast<unsigned char>(*end))) ++end;
  if (*end == 'f' || *end == 'F') ++end;
  if (*end) return false;
  *out = v;
  return true;
}

inline bool parse_int(const std::string& raw, long long* out) {
  const std::string s = trim(raw);
  if (s.empty()) return false;
  char* end = nullptr;
  const long long v = std::strtoll(s.c_str(), &end, 10);
  if (end == s.c_str()) return false;
  if (*end == 'L' || *end == 'l') ++end;
  if (*end) return false;
  *out = v;
  return true;
}

inline void bad_value(const std::string& key, const std::string& value, const std::string& why) {
  std::ostringstream os;
  os << "Invalid Parameter format for " << key << " expect " << why << " but value='" << value
     << "'";
  throw dmlc::ParamError(os.str());
}

inline bool get_bool(const Dict& d, const std::string& key, bool def) {
  auto it = d.find(key);
  if (it == d.end()) return def;
  std::string s = trim(it->second);
  for (auto& c : s) c = static_cast<char>(std::tolower(static_cast<unsigned char>(c)));
  if (s == "true" || s == "1") return true;
  if (s == "false" || s == "0") return false;
  bad_value(key, it->second, "boolean");
  return def;
}

inline dmlc::optional<float> get_optional_float(const Dict& d, const std::string& key) {
  auto it = d.find(key);
  if (it == d.end()) return dmlc::optional<float>();
  const std::string s = trim(it->second);
  if (s == "None") return dmlc::optional<float>();
  float v;
  if (!parse_float(s, &v)) bad_value(key, it->second, "float or None");
  return dmlc::optional<float>(v);
}

inline int get_enum(const Dict& d, const std::string& key,
                    const std::vector<std::pair<std::string, int>>& names, bool has_def, int def,
                    bool* present = nullptr) {
  auto it = d.find(key);
  if (present) *present = it != d.end();
  if (it == d.end()) {
    if (!has_def) throw dmlc::ParamError("Required parameter " + key + " is not presented");
    return def;
  }
  const std::string s = trim(it->second);
  for (const auto& n : names)
    if (n.first == s) return n.second;
  std::ostringstream why;
  why << "{";
  for (size_t i = 0; i < names.size(); ++i) why << (i ? ", " : "") << "'" << names[i].first << "'";
  why << "}";
  bad_value(key, it->second, why.str());
  return def;
}

inline long long get_int(const Dict& d, const std::string& key, bool has_def, long long def,
                         bool has_lower, long long lower) {
  auto it = d.find(key);
  if (it == d.end()) {
    if (!has_def) throw dmlc::ParamError("Required parameter " + key + " is not presented");
    return def;
  }
  long long v;
  if (!parse_int(it->second, &v)) bad_value(key, it->second, "int");
  if (has_lower && v < lower) {
    std::ostringstream os;
    os << "value " << v << " for Parameter " << key << " should be greater equal to " << lower;
    throw dmlc::ParamError(os.str());
  }
  return v;
}

// Tuple text forms accepted by mxnet::Tuple's operator>> (include/mxnet/tuple.h:296-369):
// "(a, b)", "[a,b]", a bare integer, "None", "()" / "[]".
inline TShape get_shape(const Dict& d, const std::string& key, bool has_def) {
  auto it = d.find(key);
  if (it == d.end()) {
    if (!has_def) throw dmlc::ParamError("Required parameter " + key + " is not presented");
    return TShape(0, 0);
  }
  std::string s = trim(it->second);
  if (s == "None") return TShape();
  std::vector<index_t> v;
  if (!s.empty() && (s[0] == '(' || s[0] == '[')) {
    const char close = s[0] == '(' ? ')' : ']';
    if (s.back() != close) bad_value(key, it->second, "Shape(tuple)");
    s = s.substr(1, s.size() - 2);
    size_t pos = 0;
    while (pos <= s.size()) {
      size_t comma = s.find(',', pos);
      std::string tok = trim(s.substr(pos, comma == std::string::npos ? comma : comma - pos));
      if (!tok.empty()) {
        long long x;
        if (!parse_int(tok, &x)) bad_value(key, it->second, "Shape(tuple)");
        v.push_back(x);
      }
      if (comma == std::string::npos) break;
      pos = comma + 1;
    }
  } else {
    long long x;
    if (!parse_int(s, &x)) bad_value(key, it->second, "Shape(tuple)");
    v.push_back(x);
  }
  return TShape(v);
}

}  // namespace param_detail

static const std::vector<std::pair<std::string, int>> kQuantizeOutTypeNames = {
    {"auto", kAuto}, {"int8", kInt8}, {"uint8", kUint8}};

struct QuantizeV2Param {
  int out_type = kInt8;
  dmlc::optional<float> min_calib_range;
  dmlc::optional<float> max_calib_range;
  void Init(const param_detail::Dict& d) {
    using namespace param_detail;
    check_unknown(d, {"out_type", "min_calib_range", "max_calib_range"}, "QuantizeV2Param");
    out_type = get_enum(d, "out_type", kQuantizeOutTypeNames, true, kInt8);
    min_calib_range = get_optional_float(d, "min_calib_range");
    max_calib_range = get_optional_float(d, "max_calib_range");
  }
  static std::vector<nnvm::ParamFieldInfo> __FIELDS__() {
    return {{"out_type", "{'auto', 'int8', 'uint8'},optional, default='int8'",
             "Output data type. `auto` can be specified to automatically determine output type "
             "according to min_calib_range."},
            {"min_calib_range", "float or None, optional, default=None",
             "The minimum scalar value in the form of float32. If present, it will be used to "
             "quantize the fp32 data into int8 or uint8."},
            {"max_calib_range", "float or None, optional, default=None",
             "The maximum scalar value in the form of float32. If present, it will be used to "
             "quantize the fp32 data into int8 or uint8."}};
  }
};

struct RequantizeParam {
  int out_type = kInt8;
  dmlc::optional<float> min_calib_range;
  dmlc::optional<float> max_calib_range;
  void Init(const param_detail::Dict& d) {
    using namespace param_detail;
    check_unknown(d, {"out_type", "min_calib_range", "max_calib_range"}, "RequantizeParam");
    out_type = get_enum(d, "out_type", kQuantizeOutTypeNames, true, kInt8);
    min_calib_range = get_optional_float(d, "min_calib_range");
    max_calib_range = get_optional_float(d, "max_calib_range");
  }
  static std::vector<nnvm::ParamFieldInfo> __FIELDS__() {
    return {{"out_type", "{'auto', 'int8', 'uint8'},optional, default='int8'",
             "Output data type. `auto` can be specified to automatically determine output type "
             "according to min_calib_range."},
            {"min_calib_range", "float or None, optional, default=None",
             "The minimum scalar value in the form of float32 obtained through calibration. If "
             "present, it will be used to requantize the int32 data into int8."},
            {"max_calib_range", "float or None, optional, default=None",
             "The maximum scalar value in the form of float32 obtained through calibration. If "
             "present, it will be used to requantize the int32 data into int8."}};
  }
};

// v1 _contrib_quantize: out_type in {int8, uint8}, default uint8
struct QuantizeParam {
  int out_type = mshadow::kUint8;
  void Init(const param_detail::Dict& d) {
    using namespace param_detail;
    check_unknown(d, {"out_type"}, "QuantizeParam");
    out_type = get_enum(d, "out_type", {{"int8", mshadow::kInt8}, {"uint8", mshadow::kUint8}},
                        true, mshadow::kUint8);
  }
  static std::vector<nnvm::ParamFieldInfo> __FIELDS__() {
    return {{"out_type", "{'int8', 'uint8'},optional, default='uint8'", "Output data type."}};
  }
};

struct DequantizeParam {
  int out_type = mshadow::kFloat32;
  void Init(const param_detail::Dict& d) {
    using namespace param_detail;
    check_unknown(d, {"out_type"}, "DequantizeParam");
    out_type = get_enum(d, "out_type", {{"float32", mshadow::kFloat32}}, true, mshadow::kFloat32);
  }
  static std::vector<nnvm::ParamFieldInfo> __FIELDS__() {
    return {{"out_type", "{'float32'},optional, default='float32'", "Output data type."}};
  }
};

struct FullyConnectedParam {
  int num_hidden = 0;
  bool no_bias = false;
  bool flatten = true;
  void Init(const param_detail::Dict& d) {
    using namespace param_detail;
    check_unknown(d, {"num_hidden", "no_bias", "flatten"}, "FullyConnectedParam");
    num_hidden = static_cast<int>(get_int(d, "num_hidden", false, 0, true, 1));
    no_bias = get_bool(d, "no_bias", false);
    flatten = get_bool(d, "flatten", true);
  }
  static std::vector<nnvm::ParamFieldInfo> __FIELDS__() {
    return {{"num_hidden", "int, required", "Number of hidden nodes of the output."},
            {"no_bias", "boolean, optional, default=0", "Whether to disable bias parameter."},
            {"flatten", "boolean, optional, default=1",
             "Whether to collapse all but the first axis of the input data tensor."}};
  }
};

struct ConvolutionParam {
  TShape kernel, stride, dilate, pad;
  uint32_t num_filter = 0;
  uint32_t num_group = 1;
  uint64_t workspace = 1024;
  bool no_bias = false;
  dmlc::optional<int> cudnn_tune;
  bool cudnn_off = false;
  dmlc::optional<int> layout;
  void Init(const param_detail::Dict& d) {
    using namespace param_detail;
    check_unknown(d, {"kernel", "stride", "dilate", "pad", "num_filter", "num_group", "workspace",
                      "no_bias", "cudnn_tune", "cudnn_off", "layout"},
                  "ConvolutionParam");
    kernel = get_shape(d, "kernel", false);
    stride = get_shape(d, "stride", true);
    dilate = get_shape(d, "dilate", true);
    pad = get_shape(d, "pad", true);
    num_filter = static_cast<uint32_t>(get_int(d, "num_filter", false, 0, true, 1));
    num_group = static_cast<uint32_t>(get_int(d, "num_group", true, 1, false, 0));
    workspace = static_cast<uint64_t>(get_int(d, "workspace", true, 1024, true, 0));
    no_bias = get_bool(d, "no_bias", false);
    cudnn_off = get_bool(d, "cudnn_off", false);
    bool present = false;
    auto none_or = [&](const std::string& key,
                       const std::vector<std::pair<std::string, int>>& names) {
      auto it = d.find(key);
      if (it == d.end() || trim(it->second) == "None") return dmlc::optional<int>();
      return dmlc::optional<int>(get_enum(d, key, names, true, 0, &present));
    };
    cudnn_tune = none_or("cudnn_tune", {{"off", 0}, {"limited_workspace", 1}, {"fastest", 2}});
    layout = none_or("layout", {{"NCW", mshadow::kNCW},
                                {"NCHW", mshadow::kNCHW},
                                {"NCDHW", mshadow::kNCDHW},
                                {"NWC", mshadow::kNWC},
                                {"NHWC", mshadow::kNHWC},
                                {"NDHWC", mshadow::kNDHWC}});
  }
  index_t DilatedKernelSize(int dim) const { return 1 + (kernel[dim] - 1) * dilate[dim]; }
  static std::vector<nnvm::ParamFieldInfo> __FIELDS__() {
    return {{"kernel", "Shape(tuple), required", "Convolution kernel size: (w,), (h, w) or (d, h, w)"},
            {"stride", "Shape(tuple), optional, default=[]", "Convolution stride"},
            {"dilate", "Shape(tuple), optional, default=[]", "Convolution dilate"},
            {"pad", "Shape(tuple), optional, default=[]", "Zero pad for convolution"},
            {"num_filter", "int (non-negative), required", "Convolution filter(channel) number"},
            {"num_group", "int (non-negative), optional, default=1", "Number of group partitions."},
            {"workspace", "long (non-negative), optional, default=1024",
             "Maximum temporary workspace allowed (MB) in convolution."},
            {"no_bias", "boolean, optional, default=0", "Whether to disable bias parameter."},
            {"cudnn_tune", "{None, 'fastest', 'limited_workspace', 'off'},optional, default='None'",
             "Whether to pick convolution algo by running performance test."},
            {"cudnn_off", "boolean, optional, default=0", "Turn off cudnn for this layer."},
            {"layout", "{None, 'NCDHW', 'NCHW', 'NCW', 'NDHWC', 'NHWC', 'NWC'},optional, "
                       "default='None'",
             "Set layout for input, output and weight."}};
  }
};

namespace activation {
enum ActivationOpType { kReLU, kSigmoid, kTanh, kSoftReLU, kSoftSign };
}
struct ActivationParam {
  int act_type = activation::kReLU;
  void Init(const param_detail::Dict& d) {
    using namespace param_detail;
    check_unknown(d, {"act_type"}, "ActivationParam");
    act_type = get_enum(d, "act_type",
                        {{"relu", activation::kReLU},
                         {"sigmoid", activation::kSigmoid},
                         {"tanh", activation::kTanh},
                         {"softrelu", activation::kSoftReLU},
                         {"softsign", activation::kSoftSign}},
                        false, 0);
  }
  static std::vector<nnvm::ParamFieldInfo> __FIELDS__() {
    return {{"act_type", "{'relu', 'sigmoid', 'softrelu', 'softsign', 'tanh'}, required",
             "Activation function to be applied."}};
  }
};


namespace pool_enum {
enum PoolingOpType { kMaxPooling, kAvgPooling, kSumPooling, kLpPooling };
enum PoolingOpPadConventionType { kValid, kFull, kSame };
}  // namespace pool_enum

struct PoolingParam {
  TShape kernel, stride, pad;
  int pool_type = pool_enum::kMaxPooling;
  int pooling_convention = pool_enum::kValid;
  bool global_pool = false;
  bool cudnn_off = false;
  dmlc::optional<int> p_value;
  dmlc::optional<bool> count_include_pad;
  dmlc::optional<int> layout;
  bool has_output_size = false;  // adaptive pooling: recognised, not supported here
  void Init(const param_detail::Dict& d) {
    using namespace param_detail;
    check_unknown(d, {"kernel", "pool_type", "global_pool", "cudnn_off", "pooling_convention",
                      "stride", "pad", "p_value", "count_include_pad", "layout", "output_size"},
                  "PoolingParam");
    kernel = get_shape(d, "kernel", true);
    stride = get_shape(d, "stride", true);
    pad = get_shape(d, "pad", true);
    for (int i = 0; i < kernel.ndim(); ++i)
      if (kernel[i] == 0) bad_value("kernel", d.at("kernel"), "non-zero extents");
    for (int i = 0; i < stride.ndim(); ++i)
      if (stride[i] == 0) bad_value("stride", d.at("stride"), "non-zero extents");
    pool_type = get_enum(d, "pool_type",
                         {{"max", pool_enum::kMaxPooling},
                          {"avg", pool_enum::kAvgPooling},
                          {"sum", pool_enum::kSumPooling},
                          {"lp", pool_enum::kLpPooling}},
                         true, pool_enum::kMaxPooling);
    pooling_convention = get_enum(d, "pooling_convention",
                                  {{"full", pool_enum::kFull},
                                   {"valid", pool_enum::kValid},
                                   {"same", pool_enum::kSame}},
                                  true, pool_enum::kValid);
    global_pool = get_bool(d, "global_pool", false);
    cudnn_off = get_bool(d, "cudnn_off", false);
    auto it = d.find("p_value");
    if (it != d.end() && trim(it->second) != "None")
      p_value = dmlc::optional<int>(static_cast<int>(get_int(d, "p_value", false, 0, false, 0)));
    it = d.find("count_include_pad");
    if (it != d.end() && trim(it->second) != "None")
      count_include_pad = dmlc::optional<bool>(get_bool(d, "count_include_pad", true));
    it = d.find("layout");
    if (it != d.end() && trim(it->second) != "None")
      layout = dmlc::optional<int>(get_enum(d, "layout",
                                            {{"NCW", mshadow::kNCW},
                                             {"NCHW", mshadow::kNCHW},
                                             {"NCDHW", mshadow::kNCDHW},
                                             {"NWC", mshadow::kNWC},
                                             {"NHWC", mshadow::kNHWC},
                                             {"NDHWC", mshadow::kNDHWC}},
                                            true, 0));
    it = d.find("output_size");
    has_output_size = it != d.end() && trim(it->second) != "None";
  }
  // pooling-inl.h:122-140
  int GetLayout(int input_dim) const {
    if (layout.has_value()) return layout.value();
    switch (input_dim) {
      case 3: return mshadow::kNCW;
      case 4: return mshadow::kNCHW;
      case 5: return mshadow::kNCDHW;
      default: LOG_FATAL << "Unsupported input data dimension " << input_dim;
    }
    return mshadow::kNCHW;
  }
  static std::vector<nnvm::ParamFieldInfo> __FIELDS__() {
    return {{"kernel", "Shape(tuple), optional, default=[]", "Pooling kernel size: (y, x) or (d, y, x)"},
            {"pool_type", "{'avg', 'lp', 'max', 'sum'},optional, default='max'",
             "Pooling type to be applied."},
            {"global_pool", "boolean, optional, default=0",
             "Ignore kernel size, do global pooling based on current input feature map. "},
            {"cudnn_off", "boolean, optional, default=0",
             "Turn off cudnn pooling and use MXNet pooling operator. "},
            {"pooling_convention", "{'full', 'same', 'valid'},optional, default='valid'",
             "Pooling convention to be applied."},
            {"stride", "Shape(tuple), optional, default=[]",
             "Stride: for pooling (y, x) or (d, y, x). Defaults to 1 for each dimension."},
            {"pad", "Shape(tuple), optional, default=[]",
             "Pad for pooling: (y, x) or (d, y, x). Defaults to no padding."},
            {"p_value", "int or None, optional, default='None'", "Value of p for Lp pooling."},
            {"count_include_pad", "boolean or None, optional, default=None",
             "Only used for AvgPool, specify whether to count padding elements for average"
             "calculation. Defaults to true."},
            {"layout", "{None, 'NCDHW', 'NCHW', 'NCW', 'NDHWC', 'NHWC', 'NWC'},optional, "
                       "default='None'",
             "Set layout for input and output."},
            {"output_size", "Shape(tuple) or None, optional", "Only used for Adaptive Pooling."}};
  }
};

// src/operator/operator_common.h:478-495
template <typename PType>
inline void ParamParser(nnvm::NodeAttrs* attrs) {
  PType param;
  try {
    param.Init(attrs->dict);
  } catch (const dmlc::ParamError& e) {
    std::ostringstream os;
    os << e.what();
    os << ", in operator " << attrs->op->name << "("
       << "name=\"" << attrs->name << "\"";
    for (const auto& k : attrs->dict) os << ", " << k.first << "=\"" << k.second << "\"";
    os << ")";
    throw dmlc::ParamError(os.str());
  }
  attrs->parsed = std::move(param);
}

// src/operator/nn/convolution.cc:366-416 (2-D and 1-D/3-D defaults)
inline void ConvolutionParamParser(nnvm::NodeAttrs* attrs) {
  ParamParser<ConvolutionParam>(attrs);
  ConvolutionParam param_ = nnvm::get<ConvolutionParam>(attrs->parsed);
  const int nd = param_.kernel.ndim();
  CHECK(nd >= 1 && nd <= 3) << nd << "D convolution not supported";
  const int def_layout = nd == 1 ? mshadow::kNCW : (nd == 2 ? mshadow::kNCHW : mshadow::kNCDHW);
  param_.layout = param_.layout ? param_.layout.value() : def_layout;
  if (param_.stride.ndim() == 0) param_.stride = TShape(nd, 1);
  if (param_.dilate.ndim() == 0) param_.dilate = TShape(nd, 1);
  if (param_.pad.ndim() == 0) param_.pad = TShape(nd, 0);
  CHECK_EQ(param_.kernel.ndim(), param_.stride.ndim())
      << "Stride must have the same number of dimensions with kernel_size,"
      << "but kernel_size is set to " << param_.kernel << " while stride is " << param_.stride;
  CHECK_EQ(param_.kernel.ndim(), param_.dilate.ndim())
      << "Dilate must have the same number of dimensions with kernel_size,"
      << "but kernel_size is set to " << param_.kernel << " while dilate is " << param_.dilate;
  CHECK_EQ(param_.kernel.ndim(), param_.pad.ndim())
      << "Padding must have the same number of dimensions with kernel_size,"
      << "but kernel_size is set to " << param_.kernel << " while padding is " << param_.pad;
  attrs->parsed = std::move(param_);
}

struct QuantizeElemwiseAddParam {
  dmlc::optional<float> min_calib_range;
  dmlc::optional<float> max_calib_range;
  void Init(const param_detail::Dict& d) {
    using namespace param_detail;
    check_unknown(d, {"min_calib_range", "max_calib_range"}, "QuantizeElemwiseAddParam");
    min_calib_range = get_optional_float(d, "min_calib_range");
    max_calib_range = get_optional_float(d, "max_calib_range");
  }
  static std::vector<nnvm::ParamFieldInfo> __FIELDS__() {
    return {{"min_calib_range", "float or None, optional, default=None",
             "The minimum scalar value in the form of float32 obtained through calibration. If "
             "present, it will be used to requantize the int8 output data."},
            {"max_calib_range", "float or None, optional, default=None",
             "The maximum scalar value in the form of float32 obtained through calibration. If "
             "present, it will be used to requantize the int8 output data."}};
  }
};

struct ConcatParam {
  int num_args = 0;
  dmlc::optional<int> dim = dmlc::optional<int>(1);
  void Init(const param_detail::Dict& d) {
    using namespace param_detail;
    check_unknown(d, {"num_args", "dim"}, "ConcatParam");
    num_args = static_cast<int>(get_int(d, "num_args", false, 0, true, 1));
    auto it = d.find("dim");
    if (it != d.end()) {
      if (trim(it->second) == "None")
        dim = dmlc::optional<int>();
      else
        dim = dmlc::optional<int>(static_cast<int>(get_int(d, "dim", true, 1, false, 0)));
    }
  }
  static std::vector<nnvm::ParamFieldInfo> __FIELDS__() {
    return {{"num_args", "int, required", "Number of inputs to be concated."},
            {"dim", "int or None, optional, default='1'", "the dimension to be concated."}};
  }
};

struct QuantizeElemwiseMulParam {
  dmlc::optional<float> min_calib_range;
  dmlc::optional<float> max_calib_range;
  bool enable_float_output = false;
  void Init(const param_detail::Dict& d) {
    using namespace param_detail;
    check_unknown(d, {"min_calib_range", "max_calib_range", "enable_float_output"},
                  "QuantizeElemwiseMulParam");
    min_calib_range = get_optional_float(d, "min_calib_range");
    max_calib_range = get_optional_float(d, "max_calib_range");
    enable_float_output = get_bool(d, "enable_float_output", false);
  }
  static std::vector<nnvm::ParamFieldInfo> __FIELDS__() {
    return {{"min_calib_range", "float or None, optional, default=None",
             "The minimum scalar value in the form of float32 obtained through calibration. If "
             "present, it will be used to requantize the int8 output data."},
            {"max_calib_range", "float or None, optional, default=None",
             "The maximum scalar value in the form of float32 obtained through calibration. If "
             "present, it will be used to requantize the int8 output data."},
            {"enable_float_output", "boolean, optional, default=0",
             "Whether to enable float32 output"}};
  }
};

struct QuantizeAsymParam {
  dmlc::optional<float> min_calib_range;
  dmlc::optional<float> max_calib_range;
  void Init(const param_detail::Dict& d) {
    using namespace param_detail;
    check_unknown(d, {"min_calib_range", "max_calib_range"}, "QuantizeAsymParam");
    min_calib_range = get_optional_float(d, "min_calib_range");
    max_calib_range = get_optional_float(d, "max_calib_range");
  }
  static std::vector<nnvm::ParamFieldInfo> __FIELDS__() {
    return {{"min_calib_range", "float or None, optional, default=None",
             "The minimum scalar value in the form of float32. If present, it will be used to "
             "quantize the fp32 data."},
            {"max_calib_range", "float or None, optional, default=None",
             "The maximum scalar value in the form of float32. If present, it will be used to "
             "quantize the fp32 data."}};
  }
};

static const std::vector<std::pair<std::string, int>> kAllTypeNames = {
    {"bfloat16", 12}, {"float16", mshadow::kFloat16}, {"float32", mshadow::kFloat32},
    {"float64", mshadow::kFloat64}, {"int32", mshadow::kInt32}, {"int64", mshadow::kInt64},
    {"int8", mshadow::kInt8}, {"uint8", mshadow::kUint8}};

struct EmbeddingParam {
  index_t input_dim = 0;
  index_t output_dim = 0;
  int dtype = mshadow::kFloat32;
  bool sparse_grad = false;
  void Init(const param_detail::Dict& d) {
    using namespace param_detail;
    check_unknown(d, {"input_dim", "output_dim", "dtype", "sparse_grad"}, "EmbeddingParam");
    input_dim = get_int(d, "input_dim", false, 0, true, 1);
    output_dim = get_int(d, "output_dim", false, 0, true, 1);
    dtype = get_enum(d, "dtype", kAllTypeNames, true, mshadow::kFloat32);
    sparse_grad = get_bool(d, "sparse_grad", false);
  }
  static std::vector<nnvm::ParamFieldInfo> __FIELDS__() {
    return {{"input_dim", "long, required", "Vocabulary size of the input indices."},
            {"output_dim", "long, required", "Dimension of the embedding vectors."},
            {"dtype",
             "{'bfloat16', 'float16', 'float32', 'float64', 'int32', 'int64', 'int8', "
             "'uint8'},optional, default='float32'",
             "Data type of weight."},
            {"sparse_grad", "boolean, optional, default=0",
             "Compute row sparse gradient in the backward calculation. If set to True, the "
             "grad's storage type is row_sparse."}};
  }
};

struct ReshapeParam {
  TShape target_shape = TShape(0, -1);  // deprecated form; ndim 0 = not given
  bool keep_highest = false;
  TShape shape = TShape(0, -1);         // with the special values 0, -1, -2, -3, -4
  bool reverse = false;
  void Init(const param_detail::Dict& d) {
    using namespace param_detail;
    check_unknown(d, {"shape", "reverse", "target_shape", "keep_highest"}, "ReshapeParam");
    shape = get_shape(d, "shape", true);
    if (shape.ndim() < 0) shape = TShape(0, -1);
    reverse = get_bool(d, "reverse", false);
    target_shape = get_shape(d, "target_shape", true);
    if (target_shape.ndim() < 0) target_shape = TShape(0, -1);
    keep_highest = get_bool(d, "keep_highest", false);
  }
  static std::vector<nnvm::ParamFieldInfo> __FIELDS__() {
    return {{"shape", "Shape(tuple), optional, default=[]", "The target shape"},
            {"reverse", "boolean, optional, default=0",
             "If true then the special values are inferred from right to left"},
            {"target_shape", "Shape(tuple), optional, default=[]",
             "(Deprecated! Use ``shape`` instead.) Target new shape. One and only one dim can "
             "be 0, in which case it will be inferred from the rest of dims"},
            {"keep_highest", "boolean, optional, default=0",
             "(Deprecated! Use ``shape`` instead.) Whether keep the highest dim unchanged.If set "
             "to true, then the first dim in target_shape is ignored,and always fixed as input"}};
  }
};

inline double get_double(const param_detail::Dict& d, const std::string& key, double def) {
  auto it = d.find(key);
  if (it == d.end()) return def;
  const std::string s = param_detail::trim(it->second);
  char* end = nullptr;
  const double v = std::strtod(s.c_str(), &end);
  if (end == s.c_str() || *end) param_detail::bad_value(key, it->second, "double");
  return v;
}

struct BatchNormParam {
  double eps = 1e-3f;  // the reference's default is the float literal
  float momentum = 0.9f;
  bool fix_gamma = true;
  bool use_global_stats = false;
  bool output_mean_var = false;
  int axis = 1;
  bool cudnn_off = false;
  dmlc::optional<float> min_calib_range;
  dmlc::optional<float> max_calib_range;
  void Init(const param_detail::Dict& d) {
    using namespace param_detail;
    check_unknown(d, {"eps", "momentum", "fix_gamma", "use_global_stats", "output_mean_var",
                      "axis", "cudnn_off", "min_calib_range", "max_calib_range"},
                  "BatchNormParam");
    eps = get_double(d, "eps", 1e-3f);
    float m = 0.9f;
    auto it = d.find("momentum");
    if (it != d.end() && !parse_float(it->second, &m)) bad_value("momentum", it->second, "float");
    momentum = m;
    fix_gamma = get_bool(d, "fix_gamma", true);
    use_global_stats = get_bool(d, "use_global_stats", false);
    output_mean_var = get_bool(d, "output_mean_var", false);
    axis = static_cast<int>(get_int(d, "axis", true, 1, false, 0));
    cudnn_off = get_bool(d, "cudnn_off", false);
    min_calib_range = get_optional_float(d, "min_calib_range");
    max_calib_range = get_optional_float(d, "max_calib_range");
  }
  static std::vector<nnvm::ParamFieldInfo> __FIELDS__() {
    return {{"eps", "double, optional, default=0.0010000000474974513",
             "Epsilon to prevent div 0. Must be no less than CUDNN_BN_MIN_EPSILON defined in "
             "cudnn.h when using cudnn (usually 1e-5)"},
            {"momentum", "float, optional, default=0.899999976", "Momentum for moving average"},
            {"fix_gamma", "boolean, optional, default=1", "Fix gamma while training"},
            {"use_global_stats", "boolean, optional, default=0",
             "Whether use global moving statistics instead of local batch-norm. This will force "
             "change batch-norm into a scale shift operator."},
            {"output_mean_var", "boolean, optional, default=0", "Output the mean and inverse std "},
            {"axis", "int, optional, default='1'",
             "Specify which shape axis the channel is specified"},
            {"cudnn_off", "boolean, optional, default=0",
             "Do not select CUDNN operator, if available"},
            {"min_calib_range", "float or None, optional, default=None",
             "The minimum scalar value in the form of float32 obtained through calibration. If "
             "present, it will be used to by quantized batch norm op to calculate primitive "
             "scale.Note: this calib_range is to calib bn output."},
            {"max_calib_range", "float or None, optional, default=None",
             "The maximum scalar value in the form of float32 obtained through calibration. If "
             "present, it will be used to by quantized batch norm op to calculate primitive "
             "scale.Note: this calib_range is to calib bn output."}};
  }
};

struct TransposeParam {
  TShape axes = TShape(0, -1);
  void Init(const param_detail::Dict& d) {
    using namespace param_detail;
    check_unknown(d, {"axes"}, "TransposeParam");
    axes = get_shape(d, "axes", true);
    if (axes.ndim() < 0) axes = TShape(0, -1);
  }
  static std::vector<nnvm::ParamFieldInfo> __FIELDS__() {
    return {{"axes", "Shape(tuple), optional, default=[]",
             "Target axis order. By default the axes will be inverted."}};
  }
};

// src/operator/numpy/np_matrix_op-inl.h:44-62: unknown axes (the default) reverse the
// dimensions; negative axes count from the end
struct NumpyTransposeParam {
  TShape axes;  // ndim -1: not given
  void Init(const param_detail::Dict& d) {
    using namespace param_detail;
    check_unknown(d, {"axes"}, "NumpyTransposeParam");
    axes = d.count("axes") ? get_shape(d, "axes", true) : TShape();
  }
  static std::vector<nnvm::ParamFieldInfo> __FIELDS__() {
    return {{"axes", "Shape(tuple), optional, default=None",
             "By default, reverse the dimensions, otherwise permute the axes according to the "
             "values given."}};
  }
};

// src/operator/numpy/np_matrix_op-inl.h:109-146
struct NumpyXReshapeParam {
  TShape newshape;  // with the special values -1 ... -6
  bool reverse = false;
  std::string order = "C";
  void Init(const param_detail::Dict& d) {
    using namespace param_detail;
    check_unknown(d, {"newshape", "reverse", "order"}, "NumpyXReshapeParam");
    newshape = get_shape(d, "newshape", false);
    reverse = get_bool(d, "reverse", false);
    auto it = d.find("order");
    if (it != d.end()) order = trim(it->second);
  }
  static std::vector<nnvm::ParamFieldInfo> __FIELDS__() {
    return {{"newshape", "Shape(tuple), required",
             "The new shape should be compatible with the original shape. One shape dimension "
             "can be -1 (inferred); -2 copies a dimension, -3 skips a dimension of size one, -4 "
             "copies all remaining dimensions, -5 merges two dimensions, -6 splits one dimension "
             "into the two that follow."},
            {"reverse", "boolean, optional, default=0",
             "If true then the special values are inferred from right to left"},
            {"order", "string, optional, default='C'",
             "Only C-like index order is supported"}};
  }
};

// src/operator/tensor/broadcast_reduce_op.h:240-249: a negative axis counts from the end
inline int CheckAxis(const int axis, const int ndim) {
  if (ndim == 0) {
    CHECK(axis == 0 || axis == -1) << "axis " << axis << " is out of bounds for 0-dimension tensor";
    return 0;
  }
  CHECK(axis < ndim && axis >= -ndim)
      << "axis " << axis << " exceeds the input dimension of " << ndim;
  return (axis + ndim) % ndim;
}

// src/operator/nn/pooling.cc:35-64
inline void PoolingParamParser(nnvm::NodeAttrs* attrs) {
  ParamParser<PoolingParam>(attrs);
  PoolingParam param = nnvm::get<PoolingParam>(attrs->parsed);
  if (param.kernel.ndim() > 0) param.layout = param.GetLayout(param.kernel.ndim() + 2);
  if (param.kernel.ndim() == 1) {
    if (param.stride.ndim() == 0) param.stride = TShape(std::vector<index_t>{1});
    if (param.pad.ndim() == 0) param.pad = TShape(std::vector<index_t>{0});
  } else if (param.kernel.ndim() == 2) {
    if (param.stride.ndim() == 0) param.stride = TShape(std::vector<index_t>{1, 1});
    if (param.pad.ndim() == 0) param.pad = TShape(std::vector<index_t>{0, 0});
  } else {
    if (!param.global_pool && !param.has_output_size)
      CHECK_EQ(param.kernel.ndim(), 3) << param.kernel.ndim() << "D pooling not supported";
    if (param.stride.ndim() == 0) param.stride = TShape(std::vector<index_t>{1, 1, 1});
    if (param.pad.ndim() == 0) param.pad = TShape(std::vector<index_t>{0, 0, 0});
  }
  attrs->parsed = std::move(param);
}

}  // namespace op
}  // namespace mxnet

#endif  // MXQ_PARAMS_H_
