// Imperative front door of libmxq_ops.so (include/mxq_ops.h): what
// MXImperativeInvoke + Imperative::InvokeOp do around an operator in the reference
// (src/imperative/imperative.cc:51-139, imperative_utils.h:653-712), reduced to
// parse -> infer -> build TBlobs / OpContext -> call the registered gpu function.
#include <cstring>
#include <string>
#include <vector>

#include "../../../include/mxq_ops.h"
#include "mxq_graph_pass.h"
#include "mxq_shim.h"

namespace mxnet {
namespace op {
size_t MXQTempSpaceBytes(const nnvm::NodeAttrs& attrs, const ShapeVector& in,
                         const ShapeVector& out);
}
}  // namespace mxnet

namespace {

thread_local std::string tl_error;

struct Node {
  nnvm::NodeAttrs attrs;
  mxnet::OpStatePtr state;
  std::string in_names, out_names, grad_names;
};

#define OPS_API_BEGIN() try {
#define OPS_API_END()                 \
  }                                   \
  catch (const std::exception& e) {   \
    tl_error = e.what();              \
    return -1;                        \
  }                                   \
  catch (...) {                       \
    tl_error = "unknown error";       \
    return -1;                        \
  }                                   \
  return 0;

mxnet::TShape to_shape(int ndim, const int64_t* dims) {
  if (ndim < 0) return mxnet::TShape();
  return mxnet::TShape(std::vector<mxnet::index_t>(dims, dims + ndim));
}

std::string join(const std::vector<std::string>& v) {
  std::string s;
  for (size_t i = 0; i < v.size(); ++i) s += (i ? "," : "") + v[i];
  return s;
}

}  // namespace

extern "C" {

const char* mxq_ops_last_error(void) { return tl_error.c_str(); }

// lets the other translation units of the library report through the same channel
void mxq_ops_set_error(const char* text) { tl_error = text ? text : ""; }

int mxq_op_count(void) { return static_cast<int>(nnvm::Op::ListAllNames().size()); }

const char* mxq_op_name(int index) {
  static thread_local std::string name;
  auto names = nnvm::Op::ListAllNames();
  if (index < 0 || index >= static_cast<int>(names.size())) return nullptr;
  name = names[index];
  return name.c_str();
}

int mxq_op_has_attr(const char* op, const char* key) {
  try {
    const nnvm::Op* o = nnvm::Op::Get(op);
    const std::string k(key);
    // the typed maps share one table; probe with the function types that can appear
    if (nnvm::Op::GetAttr<mxnet::FCompute>(k).count(o)) return 1;
    return 0;
  } catch (...) {
    return 0;
  }
}

int mxq_node_create(const char* op, const char* node_name, int num_attrs, const char** keys,
                    const char** values, void** out_node) {
  OPS_API_BEGIN();
  std::unique_ptr<Node> n(new Node());
  n->attrs.op = nnvm::Op::Get(op);
  n->attrs.name = node_name ? node_name : "";
  for (int i = 0; i < num_attrs; ++i) n->attrs.dict[keys[i]] = values[i];
  if (n->attrs.op->attr_parser) n->attrs.op->attr_parser(&n->attrs);
  auto in_names = nnvm::Op::GetAttr<nnvm::FListInputNames>("FListInputNames");
  if (in_names.count(n->attrs.op)) n->in_names = join(in_names[n->attrs.op](n->attrs));
  auto out_names = nnvm::Op::GetAttr<nnvm::FListOutputNames>("FListOutputNames");
  if (out_names.count(n->attrs.op)) n->out_names = join(out_names[n->attrs.op](n->attrs));
  *out_node = n.release();
  OPS_API_END();
}

int mxq_node_free(void* node) {
  delete static_cast<Node*>(node);
  return 0;
}

int mxq_node_num_inputs(void* node, int* out) {
  OPS_API_BEGIN();
  Node* n = static_cast<Node*>(node);
  *out = static_cast<int>(n->attrs.op->NumInputs(n->attrs));
  OPS_API_END();
}

int mxq_node_num_outputs(void* node, int* out) {
  OPS_API_BEGIN();
  Node* n = static_cast<Node*>(node);
  *out = static_cast<int>(n->attrs.op->NumOutputs(n->attrs));
  OPS_API_END();
}

int mxq_node_input_names(void* node, const char** out) {
  *out = static_cast<Node*>(node)->in_names.c_str();
  return 0;
}

int mxq_node_output_names(void* node, const char** out) {
  *out = static_cast<Node*>(node)->out_names.c_str();
  return 0;
}

int mxq_node_gradient_names(void* node, const char** out) {
  OPS_API_BEGIN();
  Node* n = static_cast<Node*>(node);
  static auto& fgrad = *new auto(nnvm::Op::GetAttr<nnvm::FGradient>("FGradient"));
  n->grad_names.clear();
  if (fgrad.count(n->attrs.op)) {
    nnvm::ObjectPtr fwd = nnvm::Node::Create();
    fwd->attrs = n->attrs;
    std::vector<std::string> names;
    for (const nnvm::NodeEntry& e : fgrad[n->attrs.op](fwd, {}))
      names.push_back((e.node->op() != nullptr ? e.node->op()->name : std::string("?")) + ":" +
                      e.node->attrs.name);
    n->grad_names = join(names);
  }
  *out = n->grad_names.c_str();
  OPS_API_END();
}

int mxq_node_infer_shape(void* node, int num_in, int* in_ndim, int64_t* in_shape, int num_out,
                         int* out_ndim, int64_t* out_shape) {
  OPS_API_BEGIN();
  Node* n = static_cast<Node*>(node);
  mxnet::ShapeVector in(num_in), out(num_out);
  for (int i = 0; i < num_in; ++i) in[i] = to_shape(in_ndim[i], in_shape + i * MXQ_MAX_NDIM);
  for (int i = 0; i < num_out; ++i) out[i] = to_shape(out_ndim[i], out_shape + i * MXQ_MAX_NDIM);
  auto fmap = nnvm::Op::GetAttr<mxnet::FInferShape>("FInferShape");
  if (!fmap.count(n->attrs.op)) throw dmlc::Error("op has no FInferShape");
  fmap[n->attrs.op](n->attrs, &in, &out);
  auto write = [](const mxnet::TShape& s, int* nd, int64_t* dims) {
    *nd = s.ndim();
    if (s.ndim() > MXQ_MAX_NDIM) throw dmlc::Error("too many dimensions");
    for (int d = 0; d < s.ndim(); ++d) dims[d] = s[d];
  };
  for (int i = 0; i < num_in; ++i) write(in[i], in_ndim + i, in_shape + i * MXQ_MAX_NDIM);
  if (static_cast<int>(out.size()) != num_out) throw dmlc::Error("output count changed");
  for (int i = 0; i < num_out; ++i) write(out[i], out_ndim + i, out_shape + i * MXQ_MAX_NDIM);
  OPS_API_END();
}

int mxq_node_infer_type(void* node, int num_in, int* in_type, int num_out, int* out_type) {
  OPS_API_BEGIN();
  Node* n = static_cast<Node*>(node);
  std::vector<int> in(in_type, in_type + num_in), out(out_type, out_type + num_out);
  auto fmap = nnvm::Op::GetAttr<nnvm::FInferType>("FInferType");
  if (!fmap.count(n->attrs.op)) throw dmlc::Error("op has no FInferType");
  fmap[n->attrs.op](n->attrs, &in, &out);
  std::copy(in.begin(), in.end(), in_type);
  std::copy(out.begin(), out.end(), out_type);
  OPS_API_END();
}

int mxq_node_temp_bytes(void* node, int num_in, const mxq_blob* in, int num_out,
                        const mxq_blob* out, size_t* bytes) {
  OPS_API_BEGIN();
  Node* n = static_cast<Node*>(node);
  *bytes = 0;
  auto fres = nnvm::Op::GetAttr<mxnet::FResourceRequest>("FResourceRequest");
  if (!fres.count(n->attrs.op) || fres[n->attrs.op](n->attrs).empty()) return 0;
  mxnet::ShapeVector si(num_in), so(num_out);
  for (int i = 0; i < num_in; ++i) si[i] = to_shape(in[i].ndim, in[i].shape);
  for (int i = 0; i < num_out; ++i) so[i] = to_shape(out[i].ndim, out[i].shape);
  *bytes = mxnet::op::MXQTempSpaceBytes(n->attrs, si, so);
  OPS_API_END();
}

int mxq_node_forward(void* node, void* stream, int dev_id, int num_in, const mxq_blob* in,
                     int num_out, const mxq_blob* out, void* temp_space, size_t temp_bytes) {
  OPS_API_BEGIN();
  Node* n = static_cast<Node*>(node);
  const nnvm::Op* op = n->attrs.op;
  if (num_in != static_cast<int>(op->NumInputs(n->attrs)))
    throw dmlc::Error("wrong number of inputs for " + op->name);
  if (num_out != static_cast<int>(op->NumOutputs(n->attrs)))
    throw dmlc::Error("wrong number of outputs for " + op->name);
  std::vector<mxnet::TBlob> ins, outs;
  mxnet::ShapeVector in_shapes;
  std::vector<int> in_types;
  for (int i = 0; i < num_in; ++i) {
    ins.emplace_back(in[i].data, to_shape(in[i].ndim, in[i].shape), mshadow::gpu::kDevMask,
                     in[i].dtype, dev_id);
    in_shapes.push_back(ins.back().shape_);
    in_types.push_back(in[i].dtype);
  }
  for (int i = 0; i < num_out; ++i)
    outs.emplace_back(out[i].data, to_shape(out[i].ndim, out[i].shape), mshadow::gpu::kDevMask,
                      out[i].dtype, dev_id);
  std::vector<mxnet::OpReqType> req(num_out, mxnet::kWriteTo);

  mshadow::Stream<mshadow::gpu> s;
  s.stream_ = stream;
  mxnet::OpContext ctx;
  ctx.run_ctx.ctx.dev_type = mxnet::Context::kGPU;
  ctx.run_ctx.ctx.dev_id = dev_id;
  ctx.run_ctx.stream = &s;
  auto fres = nnvm::Op::GetAttr<mxnet::FResourceRequest>("FResourceRequest");
  if (fres.count(op)) {
    for (const auto& r : fres[op](n->attrs)) {
      mxnet::Resource res;
      res.req = r;
      res.ptr_ = temp_space;
      res.capacity = temp_bytes;
      ctx.requested.push_back(res);
    }
  }

  // dispatch order of Imperative::InvokeOp: FCompute, else stateful
  auto fcompute = nnvm::Op::GetAttr<mxnet::FCompute>("FCompute<gpu>");
  if (fcompute.count(op)) {
    fcompute[op](n->attrs, ctx, ins, req, outs);
    return 0;
  }
  auto fcreate = nnvm::Op::GetAttr<mxnet::FCreateOpState>("FCreateOpState");
  auto fstate = nnvm::Op::GetAttr<mxnet::FStatefulCompute>("FStatefulCompute<gpu>");
  if (fcreate.count(op) && fstate.count(op)) {
    if (!n->state) n->state = fcreate[op](n->attrs, ctx.run_ctx.ctx, in_shapes, in_types);
    fstate[op](n->state, ctx, ins, req, outs);
    return 0;
  }
  throw dmlc::Error("Operator " + op->name + " is not implemented for GPU.");
  OPS_API_END();
}


namespace {
thread_local std::string tl_json;
thread_local std::vector<std::string> tl_names;
thread_local std::vector<const char*> tl_name_ptrs;
}  // namespace

int mxq_quantize_symbol(const char* symbol_json, int dev_type, int num_excluded_nodes,
                        const char** excluded_nodes, int num_excluded_ops,
                        const char** excluded_ops, int num_offline, const char** offline_params,
                        const char* quantized_dtype, const char* quantize_mode,
                        const char* quantize_granularity, const char** out_symbol_json,
                        int* out_num_calib_names, const char*** out_calib_names) {
  OPS_API_BEGIN();
  CHECK(symbol_json && quantized_dtype && quantize_mode && quantize_granularity &&
        out_symbol_json && out_num_calib_names && out_calib_names)
      << "null argument";
  mxq_graph::QuantizeOptions opt;
  for (int i = 0; i < num_excluded_nodes; ++i) opt.excluded_nodes.insert(excluded_nodes[i]);
  for (int i = 0; i < num_excluded_ops; ++i) opt.excluded_ops.insert(excluded_ops[i]);
  for (int i = 0; i < num_offline; ++i) opt.offline_params.insert(offline_params[i]);
  opt.quantized_dtype = quantized_dtype;
  opt.quantize_mode = quantize_mode;
  opt.quantize_granularity = quantize_granularity;
  opt.dev_type = dev_type;
  mxq_graph::QuantizeResult r = mxq_graph::QuantizeGraph(mxq_graph::LoadJSON(symbol_json), opt);
  tl_json = mxq_graph::SaveJSON(r.graph);
  tl_names = r.calib_nodes;
  tl_name_ptrs.clear();
  for (const std::string& n : tl_names) tl_name_ptrs.push_back(n.c_str());
  *out_symbol_json = tl_json.c_str();
  *out_num_calib_names = static_cast<int>(tl_names.size());
  *out_calib_names = tl_name_ptrs.data();
  OPS_API_END();
}

int mxq_set_calib_table(const char* qsymbol_json, int num_layers, const char** layer_names,
                        const float* min_ranges, const float* max_ranges,
                        const char** out_symbol_json) {
  OPS_API_BEGIN();
  CHECK(qsymbol_json && out_symbol_json) << "null argument";
  std::map<std::string, std::pair<float, float>> table;
  for (int i = 0; i < num_layers; ++i)
    table.emplace(layer_names[i], std::make_pair(min_ranges[i], max_ranges[i]));
  tl_json = mxq_graph::SaveJSON(mxq_graph::SetCalibTable(mxq_graph::LoadJSON(qsymbol_json), table));
  *out_symbol_json = tl_json.c_str();
  OPS_API_END();
}

int mxq_symbol_normalize(const char* symbol_json, const char** out_symbol_json) {
  OPS_API_BEGIN();
  CHECK(symbol_json && out_symbol_json) << "null argument";
  tl_json = mxq_graph::SaveJSON(mxq_graph::LoadJSON(symbol_json));
  *out_symbol_json = tl_json.c_str();
  OPS_API_END();
}

int mxq_calibrate_entropy(const float* hist, const float* hist_edges, size_t num_bins,
                          int num_quantized_bins, float* out_threshold, float* out_divergence) {
  OPS_API_BEGIN();
  CHECK(hist && hist_edges && out_threshold && out_divergence) << "null argument";
  mxq_graph::CalibrateEntropy(hist, hist_edges, num_bins, num_quantized_bins, out_threshold,
                              out_divergence);
  OPS_API_END();
}

}  // extern "C"
