// Minimal stand-ins for the parts of dmlc-core, NNVM, mshadow and MXNet's operator
// interface that the quantization operators touch, so that the registration
// translation unit (mxq_quantization_ops.cc) compiles and runs without MXNet.
// Names, namespaces, signatures and semantics follow the reference so that the
// same operator code reads as it would inside the MXNet tree:
//   include/mxnet/op_attr_types.h:45-58 (OpReqType), :66-95 (OpContext),
//   :148-201 (OpStatePtr), :215-371 (attribute typedefs);
//   include/mxnet/tensor_blob.h:65-75 (TBlob); include/mxnet/base.h:90-166,343-380
//   (Context, RunContext); include/mxnet/resource.h:38-63,177-188 (Resource);
//   include/mxnet/tuple.h (TShape, unknown = -1);
//   src/operator/operator_common.h:155-250 (shape/type assign checks);
//   3rdparty/mshadow/mshadow/base.h:351-364 (TypeFlag).
// NNVM and dmlc-core are not vendored in the reference tree; their surface here is
// reconstructed from the call sites in src/operator/quantization/*.cc.
#ifndef MXQ_SHIM_H_
#define MXQ_SHIM_H_

#include <any>
#include <cstdint>
#include <functional>
#include <memory>
#include <sstream>
#include <stdexcept>
#include <string>
#include <unordered_map>
#include <utility>
#include <vector>

namespace dmlc {

struct Error : public std::runtime_error {
  explicit Error(const std::string& s) : std::runtime_error(s) {}
};
struct ParamError : public Error {
  explicit ParamError(const std::string& s) : Error(s) {}
};

template <typename T>
class optional {
 public:
  optional() : has_(false), v_() {}
  optional(const T& v) : has_(true), v_(v) {}  // NOLINT
  bool has_value() const { return has_; }
  explicit operator bool() const { return has_; }
  const T& value() const {
    if (!has_) throw Error("bad optional access");
    return v_;
  }
  bool operator==(const optional& o) const { return has_ == o.has_ && (!has_ || v_ == o.v_); }

 private:
  bool has_;
  T v_;
};

}  // namespace dmlc

// CHECK / LOG(FATAL) of dmlc/logging.h: throw dmlc::Error (the engine rethrows it at
// the next synchronisation point, src/engine/threaded_engine.h:383-400).
#define MXQ_THROW(msg)                 \
  do {                                 \
    std::ostringstream mxq_os_;        \
    mxq_os_ << msg;                    \
    throw ::dmlc::Error(mxq_os_.str()); \
  } while (0)
#define CHECK(cond) \
  if (!(cond)) ::mxq_shim::FatalStream(__FILE__, __LINE__).stream() << "Check failed: " #cond " "
#define CHECK_EQ(a, b) CHECK((a) == (b)) << "(" << (a) << " vs. " << (b) << ") "
#define CHECK_NE(a, b) CHECK((a) != (b)) << "(" << (a) << " vs. " << (b) << ") "
#define CHECK_LT(a, b) CHECK((a) < (b)) << "(" << (a) << " vs. " << (b) << ") "
#define CHECK_GE(a, b) CHECK((a) >= (b)) << "(" << (a) << " vs. " << (b) << ") "
#define LOG_FATAL ::mxq_shim::FatalStream(__FILE__, __LINE__).stream()

namespace mxq_shim {
// Collects the message and throws from the destructor of the full expression.
class FatalStream {
 public:
  FatalStream(const char* file, int line) { os_ << file << ":" << line << ": "; }
  std::ostringstream& stream() { return os_; }
  ~FatalStream() noexcept(false) { throw ::dmlc::Error(os_.str()); }

 private:
  std::ostringstream os_;
};
}  // namespace mxq_shim

namespace mshadow {

enum TypeFlag {
  kFloat32 = 0,
  kFloat64 = 1,
  kFloat16 = 2,
  kUint8 = 3,
  kInt32 = 4,
  kInt8 = 5,
  kInt64 = 6,
  kBool = 7,
  kBfloat16 = 12
};
enum LayoutFlag { kNCHW = 0, kNHWC, kCHWN, kNCW = 1 << 3, kNWC, kCWN, kNCDHW = 1 << 5, kNDHWC, kCDHWN };

struct cpu {
  static constexpr int kDevMask = 1;
};
struct gpu {
  static constexpr int kDevMask = 2;
};

// The reference's Stream<gpu> owns a cudaStream_t plus cuBLAS/cuDNN handles
// (3rdparty/mshadow/mshadow/stream_gpu-inl.h:36-253); here it is just the raw
// hipStream_t that is handed to the C-ABI launcher.
template <typename xpu>
struct Stream {
  void* stream_ = nullptr;
};

template <typename T>
struct DataType;
template <>
struct DataType<float> {
  static const int kFlag = kFloat32;
};
template <>
struct DataType<uint8_t> {
  static const int kFlag = kUint8;
};
template <>
struct DataType<int32_t> {
  static const int kFlag = kInt32;
};
template <>
struct DataType<int8_t> {
  static const int kFlag = kInt8;
};

}  // namespace mshadow

namespace mxnet {

typedef int64_t index_t;

// Shape with numpy semantics: ndim() == -1 is an unknown shape, a dimension of
// -1 an unknown extent (include/mxnet/tuple.h).
class TShape {
 public:
  TShape() : ndim_(-1) {}
  TShape(int ndim, index_t value) : ndim_(ndim), d_(ndim > 0 ? ndim : 0, value) {}
  TShape(std::initializer_list<index_t> l) : ndim_(static_cast<int>(l.size())), d_(l) {}
  explicit TShape(const std::vector<index_t>& v) : ndim_(static_cast<int>(v.size())), d_(v) {}
  int ndim() const { return ndim_; }
  index_t& operator[](int i) { return d_.at(i); }
  const index_t& operator[](int i) const { return d_.at(i); }
  size_t Size() const {
    size_t s = 1;
    for (int i = 0; i < ndim_; ++i) s *= static_cast<size_t>(d_[i]);
    return ndim_ < 0 ? 0 : s;
  }
  index_t ProdShape(int b, int e) const {
    index_t s = 1;
    for (int i = b; i < e; ++i) s *= d_[i];
    return s;
  }
  bool operator==(const TShape& o) const { return ndim_ == o.ndim_ && d_ == o.d_; }
  bool operator!=(const TShape& o) const { return !(*this == o); }
  const std::vector<index_t>& data() const { return d_; }

 private:
  int ndim_;
  std::vector<index_t> d_;
};
inline std::ostream& operator<<(std::ostream& os, const TShape& s) {
  if (s.ndim() < 0) return os << "None";
  os << '[';
  for (int i = 0; i < s.ndim(); ++i) os << (i ? "," : "") << s[i];
  return os << ']';
}
typedef std::vector<TShape> ShapeVector;

inline bool ndim_is_known(const TShape& s) { return s.ndim() >= 0; }
inline bool dim_size_is_known(const TShape& s, int i) { return s[i] >= 0; }
inline bool shape_is_known(const TShape& s) {
  if (!ndim_is_known(s)) return false;
  for (int i = 0; i < s.ndim(); ++i)
    if (!dim_size_is_known(s, i)) return false;
  return true;
}
inline bool shape_is_none(const TShape& s) { return !shape_is_known(s); }

inline TShape Shape1(index_t a) { return TShape{a}; }
inline TShape Shape2(index_t a, index_t b) { return TShape{a, b}; }

enum OpReqType { kNullOp, kWriteTo, kWriteInplace, kAddTo };
enum NDArrayStorageType { kUndefinedStorage = -1, kDefaultStorage, kRowSparseStorage, kCSRStorage };
enum class DispatchMode { kUndefined = -1, kFCompute, kFComputeEx, kFComputeFallback, kVariable };

struct Context {
  enum DeviceType { kCPU = 1, kGPU = 2, kCPUPinned = 3, kCPUShared = 5 };
  DeviceType dev_type = kGPU;
  int32_t dev_id = 0;
  int dev_mask() const { return dev_type == kGPU ? mshadow::gpu::kDevMask : mshadow::cpu::kDevMask; }
};

struct RunContext {
  Context ctx;
  void* stream = nullptr;  // mshadow::Stream<xpu>*
  template <typename xpu>
  mshadow::Stream<xpu>* get_stream() const {
    return static_cast<mshadow::Stream<xpu>*>(stream);
  }
};

struct ResourceRequest {
  enum Type { kRandom, kTempSpace, kParallelRandom };
  Type type;
  ResourceRequest(Type t) : type(t) {}  // NOLINT
};

// Temp space handed to the operator by the framework; owned by the caller.
struct Resource {
  ResourceRequest req{ResourceRequest::kTempSpace};
  void* ptr_ = nullptr;
  size_t capacity = 0;
  // the reference returns an mshadow::Tensor whose dptr_ is used; the byte
  // pointer is all the quantization operators need
  char* get_space(size_t bytes) const {
    if (bytes > capacity)
      MXQ_THROW("temp space too small: need " << bytes << " bytes, have " << capacity);
    return static_cast<char*>(ptr_);
  }
};

class TBlob {
 public:
  void* dptr_ = nullptr;
  TShape shape_;
  int type_flag_ = mshadow::kFloat32;
  TBlob() {}
  TBlob(void* p, const TShape& s, int dev_mask, int type_flag, int dev_id = -1)
      : dptr_(p), shape_(s), type_flag_(type_flag) {
    (void)dev_mask;
    (void)dev_id;
  }
  size_t Size() const { return shape_.Size(); }
  template <typename DType>
  DType* dptr() const {
    CHECK(mshadow::DataType<DType>::kFlag == type_flag_)
        << "TBlob.get_with_shape: data type do not match specified type. Expected: "
        << mshadow::DataType<DType>::kFlag << " v.s. given " << type_flag_;
    return static_cast<DType*>(dptr_);
  }
};

struct OpContext {
  bool need_grad = false;
  bool is_train = false;
  RunContext run_ctx;
  std::vector<Resource> requested;
  template <typename xpu>
  mshadow::Stream<xpu>* get_stream() const {
    return run_ctx.get_stream<xpu>();
  }
};

class OpStatePtr {
 public:
  template <typename T, typename... Args>
  static OpStatePtr Create(Args&&... args) {
    OpStatePtr p;
    p.state_ = std::shared_ptr<void>(new T(std::forward<Args>(args)...),
                                     [](void* q) { delete static_cast<T*>(q); });
    return p;
  }
  template <typename T>
  T& get_state() const {
    return *static_cast<T*>(state_.get());
  }
  explicit operator bool() const { return static_cast<bool>(state_); }

 private:
  std::shared_ptr<void> state_;
};

}  // namespace mxnet

namespace nnvm {

class Op;

struct NodeAttrs {
  const Op* op = nullptr;
  std::string name;
  std::unordered_map<std::string, std::string> dict;
  std::any parsed;
};

template <typename T>
inline const T& get(const std::any& a) {
  return std::any_cast<const T&>(a);
}

template <typename ValueType>
class OpMap {
 public:
  int count(const Op* op) const { return data_ && data_->count(op) ? 1 : 0; }
  const ValueType& operator[](const Op* op) const {
    auto it = data_ ? data_->find(op) : decltype(data_->find(op))();
    if (!data_ || it == data_->end()) throw dmlc::Error("attribute not registered for the op");
    return std::any_cast<const ValueType&>(it->second);
  }
  const ValueType& get(const Op* op, const ValueType& def) const {
    if (!count(op)) return def;
    return (*this)[op];
  }

 private:
  friend class Op;
  const std::unordered_map<const Op*, std::any>* data_ = nullptr;
};

struct ParamFieldInfo {
  std::string name, type, description;
};

class Op {
 public:
  std::string name;
  std::string description;
  std::vector<ParamFieldInfo> arguments;
  uint32_t num_inputs = 1;
  uint32_t num_outputs = 1;
  std::function<uint32_t(const NodeAttrs&)> get_num_inputs;
  std::function<void(NodeAttrs*)> attr_parser;

  Op& describe(const std::string& d) {
    description = d;
    return *this;
  }
  Op& add_alias(const std::string& alias);
  Op& add_argument(const std::string& n, const std::string& t, const std::string& d) {
    arguments.push_back({n, t, d});
    return *this;
  }
  Op& add_arguments(const std::vector<ParamFieldInfo>& a) {
    arguments.insert(arguments.end(), a.begin(), a.end());
    return *this;
  }
  Op& set_num_inputs(uint32_t n) {
    num_inputs = n;
    return *this;
  }
  Op& set_num_inputs(std::function<uint32_t(const NodeAttrs&)> fn) {
    get_num_inputs = fn;
    return *this;
  }
  Op& set_num_outputs(uint32_t n) {
    num_outputs = n;
    return *this;
  }
  Op& set_attr_parser(std::function<void(NodeAttrs*)> fn) {
    attr_parser = fn;
    return *this;
  }
  template <typename ValueType>
  Op& set_attr(const std::string& key, const ValueType& value, int plevel = 10) {
    (void)plevel;
    AttrTable()[key][this] = std::any(value);
    return *this;
  }
  Op& set_num_outputs(std::function<uint32_t(const NodeAttrs&)> fn) {
    get_num_outputs = fn;
    return *this;
  }
  uint32_t NumInputs(const NodeAttrs& attrs) const {
    return get_num_inputs ? get_num_inputs(attrs) : num_inputs;
  }
  uint32_t NumOutputs(const NodeAttrs& attrs) const {
    return get_num_outputs ? get_num_outputs(attrs) : num_outputs;
  }
  std::function<uint32_t(const NodeAttrs&)> get_num_outputs;

  static const Op* Get(const std::string& name);   // throws when the name is unknown
  static const Op* Find(const std::string& name);  // nullptr when the name is unknown
  static Op& RegisterOrGet(const std::string& name);
  static std::vector<std::string> ListAllNames();
  template <typename ValueType>
  static OpMap<ValueType> GetAttr(const std::string& key) {
    OpMap<ValueType> m;
    auto it = AttrTable().find(key);
    if (it != AttrTable().end()) m.data_ = &it->second;
    return m;
  }

 private:
  static std::unordered_map<std::string, std::unordered_map<const Op*, std::any>>& AttrTable();
};

typedef std::function<std::vector<std::string>(const NodeAttrs&)> FListInputNames;
typedef std::function<std::vector<std::string>(const NodeAttrs&)> FListOutputNames;
typedef std::function<bool(const NodeAttrs&, std::vector<int>*, std::vector<int>*)> FInferType;
typedef std::function<std::vector<std::pair<int, int>>(const NodeAttrs&)> FInplaceOption;
typedef std::function<std::vector<bool>(const NodeAttrs&)> FInplaceIdentity;
typedef std::function<uint32_t(const NodeAttrs&)> FNumVisibleOutputs;
// include/nnvm/op_attr_types.h: indices of the inputs an operator writes (moving statistics)
typedef std::function<std::vector<uint32_t>(const NodeAttrs&)> FMutateInputs;

// What FQuantizedOp hands back in the reference is a graph node; only its attributes
// (operator, name, dict, parsed struct) are ever looked at.
struct Node;
typedef std::shared_ptr<Node> ObjectPtr;
// include/nnvm/node.h: output `index` of `node`
struct NodeEntry {
  ObjectPtr node;
  uint32_t index = 0;
  uint32_t version = 0;
};
struct Node {
  NodeAttrs attrs;
  std::vector<NodeEntry> inputs;
  std::vector<ObjectPtr> control_deps;
  const Op* op() const { return attrs.op; }
  uint32_t num_inputs() const {
    return attrs.op != nullptr ? attrs.op->NumInputs(attrs) : static_cast<uint32_t>(inputs.size());
  }
  static std::shared_ptr<Node> Create() { return std::make_shared<Node>(); }
};
// include/nnvm/op_attr_types.h: the gradient of a node as new nodes, one entry per input
typedef std::function<std::vector<NodeEntry>(const ObjectPtr&, const std::vector<NodeEntry>&)>
    FGradient;

}  // namespace nnvm

#define MXQ_CONCAT_(a, b) a##b
#define MXQ_CONCAT(a, b) MXQ_CONCAT_(a, b)
#define NNVM_REGISTER_OP(OpName)                                    \
  static ::nnvm::Op& MXQ_CONCAT(mxq_nnvm_op_##OpName##_, __COUNTER__) = \
      ::nnvm::Op::RegisterOrGet(#OpName)

namespace mxnet {

using nnvm::NodeAttrs;

typedef std::function<bool(const NodeAttrs&, ShapeVector*, ShapeVector*)> FInferShape;
typedef std::function<bool(const NodeAttrs&, const int, DispatchMode*, std::vector<int>*,
                           std::vector<int>*)>
    FInferStorageType;
typedef std::function<void(const NodeAttrs&, const OpContext&, const std::vector<TBlob>&,
                           const std::vector<OpReqType>&, const std::vector<TBlob>&)>
    FCompute;
typedef std::function<void(const OpStatePtr&, const OpContext&, const std::vector<TBlob>&,
                           const std::vector<OpReqType>&, const std::vector<TBlob>&)>
    FStatefulCompute;
typedef std::function<OpStatePtr(const NodeAttrs&, Context, const ShapeVector&,
                                 const std::vector<int>&)>
    FCreateOpState;
typedef std::function<std::vector<ResourceRequest>(const NodeAttrs&)> FResourceRequest;
typedef std::function<bool(const NodeAttrs&)> FNeedRequantize;
typedef std::function<std::vector<int>(const NodeAttrs&)> FNeedCalibrateInput;
typedef std::function<std::vector<int>(const NodeAttrs&)> FNeedCalibrateOutput;
// include/mxnet/op_attr_types.h:134-142, 318-357
enum class QuantizeType { kNone = 0, kMust, kSupport };
typedef std::function<QuantizeType(const NodeAttrs&)> FQuantizable;
typedef std::function<nnvm::ObjectPtr(const NodeAttrs&)> FQuantizedOp;
typedef std::function<bool(const NodeAttrs&, const size_t, const std::string)> FAvoidQuantizeInput;
typedef std::function<bool(const NodeAttrs&, const size_t)> FAvoidDequantizeOutput;

namespace op {

// src/operator/operator_common.h:430-444: the quantized operators are inference-only, their
// gradient with respect to every input is a zeros_like node named after the forward node.
inline std::vector<nnvm::NodeEntry> MakeZeroGradNodes(const nnvm::ObjectPtr& n,
                                                      const std::vector<nnvm::NodeEntry>&) {
  const uint32_t count = n->num_inputs();
  std::vector<nnvm::NodeEntry> grads;
  for (uint32_t i = 0; i < count; ++i) {
    nnvm::ObjectPtr z = nnvm::Node::Create();
    z->attrs.op = nnvm::Op::Find("zeros_like");
    z->attrs.name = n->attrs.name + (count == 1 ? std::string("_backward")
                                                 : "_in" + std::to_string(i) + "_backward");
    if (i < n->inputs.size()) z->inputs.push_back(n->inputs[i]);
    z->control_deps.push_back(n);
    nnvm::NodeEntry e;
    e.node = z;
    grads.push_back(e);
  }
  return grads;
}

struct InferShapeError : public dmlc::Error {
  int index;
  InferShapeError(const std::string& m, int i) : dmlc::Error(m), index(i) {}
};
struct InferTypeError : public dmlc::Error {
  int index;
  InferTypeError(const std::string& m, int i) : dmlc::Error(m), index(i) {}
};

inline std::string type_string(int t) {
  switch (t) {
    case mshadow::kFloat32: return "float32";
    case mshadow::kFloat64: return "float64";
    case mshadow::kFloat16: return "float16";
    case mshadow::kUint8: return "uint8";
    case mshadow::kInt32: return "int32";
    case mshadow::kInt8: return "int8";
    case mshadow::kInt64: return "int64";
    case mshadow::kBool: return "bool";
    case mshadow::kBfloat16: return "bfloat16";
    default: return "unknown";
  }
}

// src/operator/operator_common.h:155-196
inline bool shape_assign(TShape* y, const TShape& x) {
  if (!ndim_is_known(*y)) {
    *y = x;
    return true;
  } else if (y->ndim() != x.ndim()) {
    return !ndim_is_known(x);
  } else {
    for (int i = 0; i < y->ndim(); ++i) {
      if (!dim_size_is_known(*y, i)) {
        (*y)[i] = x[i];
      } else if ((*y)[i] != x[i] && x[i] >= 0) {
        return false;
      }
    }
    return true;
  }
}
inline bool type_assign(int* y, const int& x) {
  if (*y == -1) {
    *y = x;
    return true;
  } else if (*y != x && x != -1) {
    return false;
  }
  return true;
}

#define SHAPE_ASSIGN_CHECK(shape_array, index, shape)                                 \
  {                                                                                   \
    if (!::mxnet::op::shape_assign(&(shape_array)[index], ::mxnet::TShape(shape))) {  \
      std::ostringstream os;                                                          \
      os << "Shape inconsistent, Provided = " << (shape_array)[index] << ','          \
         << " inferred shape=" << ::mxnet::TShape(shape);                             \
      throw ::mxnet::op::InferShapeError(os.str(), index);                            \
    }                                                                                 \
  }
#define TYPE_ASSIGN_CHECK(type_array, index, type)                                            \
  {                                                                                           \
    if (!::mxnet::op::type_assign(&(type_array)[index], type)) {                              \
      std::ostringstream os;                                                                  \
      os << "Type inconsistent, Provided = " << ::mxnet::op::type_string((type_array)[index]) \
         << ',' << " inferred type = " << ::mxnet::op::type_string(type);                     \
      throw ::mxnet::op::InferTypeError(os.str(), index);                                     \
    }                                                                                         \
  }

}  // namespace op
}  // namespace mxnet

#endif  // MXQ_SHIM_H_
