// The two graph passes behind MXQuantizeSymbol / MXSetCalibTableToQuantizedSymbol
// (src/c_api/c_api_symbolic.cc:916-972, 1031-1050), restated over the index-based
// graph of mxq_graph.h:
//   QuantizeGraph                  src/operator/quantization/quantize_graph_pass.cc:286-610
//   SetCalibTableToQuantizedGraph  src/operator/quantization/quantize_graph_pass.cc:612-673
// The output has to be the reference's graph: same operators, same wiring, same node
// names (they are what calibration tables and offline-quantized parameters are keyed
// by), and the same list of tensors to calibrate.
#include <algorithm>
#include <deque>
#include <map>
#include <set>
#include <string>
#include <vector>

#include "mxq_graph.h"
#include "mxq_graph_pass.h"
#include "mxq_shim.h"

namespace mxq_graph {

using mxnet::QuantizeType;

namespace {

const char* const kQuantize = "_contrib_quantize_v2";
const char* const kDequantize = "_contrib_dequantize";
const char* const kRequantize = "_contrib_requantize";

// True if the operator has any compute function for the device
// (quantize_graph_pass.cc:128-141; 1 = cpu, 2 = gpu as in Context::DeviceType).
bool HasDeviceCompute(const nnvm::Op* op, int dev_type) {
  if (op == nullptr) return false;
  const std::string dev = dev_type == 2 ? "<gpu>" : "<cpu>";
  for (const char* key : {"FCompute", "FComputeEx", "FStatefulCompute", "FStatefulComputeEx"})
    if (nnvm::Op::GetAttr<mxnet::FCompute>(key + dev).count(op)) return true;
  return false;
}

// Outputs a consumer can address (FNumVisibleOutputs when registered,
// quantize_graph_pass.cc:64-75).
uint32_t VisibleOutputs(const Graph& g, int node) {
  static const auto visible = nnvm::Op::GetAttr<nnvm::FNumVisibleOutputs>("FNumVisibleOutputs");
  const GNode& n = g.nodes[node];
  if (n.reg != nullptr && visible.count(n.reg)) return visible[n.reg](n.attrs);
  return g.NumOutputs(node);
}

struct Twin {
  nnvm::NodeAttrs attrs;  // operator, name and dict of the quantized replacement
  int dst = -1;           // its node in the rewritten graph
};

// Which float nodes are replaced (MarkQuantizedNodes + NeedQuantize,
// quantize_graph_pass.cc:143-284).
std::map<int, Twin> ChooseQuantizedNodes(const Graph& src, const std::vector<int>& order,
                                         const QuantizeOptions& opt) {
  static const auto quantizable = nnvm::Op::GetAttr<mxnet::FQuantizable>("FQuantizable");
  static const auto quantized_op = nnvm::Op::GetAttr<mxnet::FQuantizedOp>("FQuantizedOp");
  std::map<int, Twin> twins;
  std::set<int> must;
  std::map<int, int> support;  // node -> bits: 1 feeds a must node, 2 is fed by one
  std::map<int, std::vector<int>> consumers;
  for (const int id : order) {
    const GNode& n = src.nodes[id];
    if (n.reg != nullptr && quantized_op.count(n.reg)) {
      const nnvm::ObjectPtr q = quantized_op[n.reg](n.attrs);
      // a replacement without a compute function on the target device, an excluded node
      // or operator, or "no replacement" (no operator on q) leave the float node alone
      const bool usable = HasDeviceCompute(q->op(), opt.dev_type) &&
                          !opt.excluded_nodes.count(n.name) && !opt.excluded_ops.count(n.op);
      if (usable) {
        Twin t;
        t.attrs = q->attrs;
        if (opt.quantize_granularity == "channel-wise" && n.op == "_sg_onednn_fully_connected")
          t.attrs.dict["channel_wise_quantize"] = "True";
        twins[id] = t;
        const QuantizeType kind =
            quantizable.count(n.reg) ? quantizable[n.reg](n.attrs) : QuantizeType::kSupport;
        if (kind == QuantizeType::kMust) must.insert(id);
        if (kind == QuantizeType::kSupport) support[id] = 0;
      }
    }
    for (const Entry& e : n.inputs) consumers[e.node].push_back(id);
  }
  if (opt.quantize_mode == "full") return twins;
  CHECK(opt.quantize_mode == "smart") << "unrecognized quantize mode: " << opt.quantize_mode;
  // "smart": an operator that merely supports int8 is replaced only when int8 data both
  // reaches it from and flows on to an operator that must be quantized, through a chain
  // of such supporting operators.
  for (const int bit : {1, 2}) {
    std::deque<int> queue(must.begin(), must.end());
    while (!queue.empty()) {
      const int id = queue.front();
      queue.pop_front();
      std::vector<int> next;
      if (bit == 1) {
        for (const Entry& e : src.nodes[id].inputs) next.push_back(e.node);
      } else {
        next = consumers[id];
      }
      for (const int m : next) {
        auto it = support.find(m);
        if (it == support.end()) continue;
        it->second |= bit;
        queue.push_back(m);
      }
    }
  }
  for (const auto& kv : support)
    if (kv.second != 3) twins.erase(kv.first);
  return twins;
}

}  // namespace

QuantizeResult QuantizeGraph(const Graph& src, const QuantizeOptions& opt) {
  static const auto need_requantize = nnvm::Op::GetAttr<mxnet::FNeedRequantize>("FNeedRequantize");
  static const auto avoid_quantize_input =
      nnvm::Op::GetAttr<mxnet::FAvoidQuantizeInput>("FAvoidQuantizeInput");
  static const auto avoid_dequantize =
      nnvm::Op::GetAttr<mxnet::FAvoidDequantizeOutput>("FAvoidDequantizeOutput");
  static const auto list_inputs = nnvm::Op::GetAttr<nnvm::FListInputNames>("FListInputNames");
  static const auto calib_input =
      nnvm::Op::GetAttr<mxnet::FNeedCalibrateInput>("FNeedCalibrateInput");
  static const auto calib_output =
      nnvm::Op::GetAttr<mxnet::FNeedCalibrateOutput>("FNeedCalibrateOutput");

  CHECK(!(opt.dev_type == 2 && opt.quantize_granularity == "channel-wise"))
      << "`channel-wise` quantization option is not supported yet by GPU,"
      << " please set quantize_granularity to `tensor-wise` when quantizing model.";

  const std::vector<int> order = src.PostOrder();
  std::map<int, Twin> twins = ChooseQuantizedNodes(src, order, opt);

  Graph dst;
  std::map<int, int> mirror;        // float node -> what stands for it in dst (so far)
  std::map<int, int> origin;        // dst node -> the float node it stands for
  std::map<Entry, Entry> quantize;  // float entry -> output 0 of the quantize node made for it

  auto keeps_float_output = [&](const Entry& e) {
    const GNode& p = src.nodes[e.node];
    return p.reg != nullptr && avoid_dequantize.count(p.reg) &&
           avoid_dequantize[p.reg](p.attrs, e.index);
  };
  // indices of the (min, max) outputs that belong to data output `index` of a quantized
  // node: data outputs first, then one (min, max) pair per data output
  auto range_outputs = [&](uint32_t visible, uint32_t index) {
    const uint32_t base = visible - 2 + 2 * index;
    return std::make_pair(base, base + 1);
  };
  auto add_dequantize = [&](int float_node, const Entry& value, uint32_t min_index,
                            uint32_t max_index) {
    const int dq = dst.AddNode(kDequantize, src.nodes[float_node].name + "_dequantize");
    dst.nodes[dq].inputs = {value, Entry{value.node, min_index, 0}, Entry{value.node, max_index, 0}};
    return dq;
  };

  for (const int id : order) {
    const GNode& n = src.nodes[id];
    int made;
    auto tw = twins.find(id);
    if (tw != twins.end()) {
      std::map<std::string, std::string> dict(tw->second.attrs.dict.begin(),
                                              tw->second.attrs.dict.end());
      const int q = dst.AddNode(tw->second.attrs.op->name, tw->second.attrs.name, dict);
      tw->second.dst = q;
      std::vector<Entry> data_inputs, range_inputs;
      for (size_t i = 0; i < n.inputs.size(); ++i) {
        const Entry& e = n.inputs[i];
        const int m = mirror.at(e.node);
        const bool stays_float = n.reg != nullptr && avoid_quantize_input.count(n.reg) &&
                                 avoid_quantize_input[n.reg](n.attrs, i, opt.quantize_granularity);
        if (stays_float) {
          data_inputs.push_back(Entry{m, e.index, e.version});
          continue;
        }
        const bool producer_is_int8 = twins.count(e.node) && !keeps_float_output(e);
        if (!producer_is_int8) {
          // float producer: one quantize node per float entry, shared by all consumers
          auto found = quantize.find(e);
          if (found == quantize.end()) {
            // Name: "<producer>_<output name>_quantize" behind an operator; behind a
            // variable "<consumer>_<argument name>_quantize", except parameters that are
            // quantized offline, which keep "<variable>_quantize".
            const GNode& producer = src.nodes[e.node];
            std::string base = producer.name, suffix;
            if (!producer.is_variable()) {
              suffix = "_" + OutputName(src, e.node, e.index);
            } else if (!opt.offline_params.count(base)) {
              if (n.reg != nullptr && list_inputs.count(n.reg))
                base = n.name + "_" + list_inputs[n.reg](n.attrs)[i];
              else
                base = n.name + "_" + producer.name;
            }
            const int qz = dst.AddNode(kQuantize, base + suffix + "_quantize",
                                       {{"out_type", opt.quantized_dtype}});
            dst.nodes[qz].inputs = {Entry{m, e.index, e.version}};
            found = quantize.emplace(e, Entry{qz, 0, e.version}).first;
            data_inputs.push_back(Entry{qz, 0, 0});
          } else {
            data_inputs.push_back(found->second);
          }
        } else if (dst.nodes[m].op == kDequantize) {
          // the producer already got a dequantize node for a float consumer: go around it
          data_inputs.push_back(Entry{dst.nodes[m].inputs[0].node, e.index, e.version});
        } else {
          data_inputs.push_back(Entry{m, e.index, e.version});
        }
      }
      // the ranges follow all data inputs: min1, max1, min2, max2, ...
      for (size_t i = 0; i < n.inputs.size(); ++i) {
        const Entry& e = n.inputs[i];
        if (n.reg != nullptr && avoid_quantize_input.count(n.reg) &&
            avoid_quantize_input[n.reg](n.attrs, i, opt.quantize_granularity))
          continue;
        int m = mirror.at(e.node);
        if (dst.nodes[m].op == kDequantize) m = dst.nodes[m].inputs[0].node;
        std::pair<uint32_t, uint32_t> mm(1, 2);  // outputs of a quantize node
        const auto found = quantize.find(e);
        if (twins.count(e.node))
          mm = range_outputs(VisibleOutputs(dst, m), e.index);
        else
          CHECK(found != quantize.end()) << "The input is not quantize or quantized_op";
        const int from = found != quantize.end() ? found->second.node : m;
        range_inputs.push_back(Entry{from, mm.first, 0});
        range_inputs.push_back(Entry{from, mm.second, 0});
      }
      data_inputs.insert(data_inputs.end(), range_inputs.begin(), range_inputs.end());
      dst.nodes[q].inputs = data_inputs;
      made = q;
      // int32 accumulators are brought back to int8 right away
      const GNode& qn = dst.nodes[q];
      if (qn.reg != nullptr && need_requantize.count(qn.reg) && need_requantize[qn.reg](qn.attrs)) {
        const int r = dst.AddNode(kRequantize, "requantize_" + n.name,
                                  {{"out_type", opt.quantized_dtype}});
        dst.nodes[r].inputs = {Entry{q, 0, 0}, Entry{q, 1, 0}, Entry{q, 2, 0}};
        made = r;
      }
    } else {
      // float node: copied; int8 producers get one dequantize node each, which from then
      // on stands for the producer
      const int c = dst.AddNode(n.op, n.name, n.dict);
      std::vector<Entry> inputs;
      for (const Entry& e : n.inputs) {
        const int m = mirror.at(e.node);
        const auto found = quantize.find(e);
        if (twins.count(e.node) && dst.nodes[m].op != kDequantize && !keeps_float_output(e)) {
          const auto mm = range_outputs(VisibleOutputs(dst, m), e.index);
          const int dq = add_dequantize(e.node, Entry{m, e.index, e.version}, mm.first, mm.second);
          inputs.push_back(Entry{dq, 0, 0});
          mirror[e.node] = dq;
          origin[dq] = e.node;
        } else if (found != quantize.end()) {
          // a quantize node exists for this float entry: read what it reads
          inputs.push_back(Entry{dst.nodes[found->second.node].inputs[0].node, e.index, e.version});
        } else {
          inputs.push_back(Entry{m, e.index, e.version});
        }
      }
      dst.nodes[c].inputs = inputs;
      made = c;
    }
    mirror[id] = made;
    origin[made] = id;
  }

  // graph outputs come back as float
  for (const Entry& e : src.heads) {
    const int m = mirror.at(e.node);
    if (twins.count(e.node) && !keeps_float_output(e) && dst.nodes[m].op != kDequantize) {
      const auto mm = range_outputs(VisibleOutputs(src, e.node) + 2, e.index);
      const int dq = add_dequantize(e.node, Entry{m, e.index, e.version}, mm.first, mm.second);
      dst.heads.push_back(Entry{dq, 0, 0});
    } else if (twins.count(e.node) && dst.nodes[m].op == kDequantize) {
      dst.heads.push_back(Entry{m, 0, 0});
    } else {
      dst.heads.push_back(Entry{m, e.index, e.version});
    }
  }

  // Parameters quantized offline: the quantize node over such a variable disappears and
  // its three outputs become variables "<node>", "<node>_min", "<node>_max"
  // (OfflineParams, quantize_graph_pass.cc:103-126).
  if (!opt.offline_params.empty()) {
    static const char* const kSuffix[3] = {"", "_min", "_max"};
    std::map<Entry, int> variable_of;
    auto is_offline_quantize = [&](int node) {
      const GNode& qz = dst.nodes[node];
      if (qz.op != kQuantize || qz.inputs.empty()) return false;
      const GNode& in = dst.nodes[qz.inputs[0].node];
      return in.is_variable() && opt.offline_params.count(in.name) > 0;
    };
    for (const int id : dst.PostOrder()) {
      for (size_t i = 0; i < dst.nodes[id].inputs.size(); ++i) {
        const Entry e = dst.nodes[id].inputs[i];
        if (!is_offline_quantize(e.node)) continue;
        CHECK(e.index < 3) << "a quantize node has three outputs";
        auto found = variable_of.find(e);
        if (found == variable_of.end()) {
          const int v = dst.AddNode("null", dst.nodes[e.node].name + kSuffix[e.index]);
          found = variable_of.emplace(e, v).first;
        }
        dst.nodes[id].inputs[i] = Entry{found->second, 0, 0};
      }
    }
  }

  // Tensors whose range a calibration run has to observe, named the way the reference's
  // monitor callback names what it sees (quantize_graph_pass.cc:533-606).
  QuantizeResult result;
  std::set<int> pending;  // quantize nodes reading a variable: named when the consumer shows up
  std::map<int, int> float_of_twin;
  for (const auto& kv : twins) float_of_twin[kv.second.dst] = kv.first;
  auto float_output_name = [&](int float_node, uint32_t index) {
    return src.nodes[float_node].name + "_" + OutputName(src, float_node, index);
  };
  for (const int id : dst.PostOrder()) {
    const GNode& node = dst.nodes[id];
    if (!node.is_variable() && !pending.empty()) {
      for (size_t i = 0; i < node.inputs.size(); ++i) {
        const int in = node.inputs[i].node;
        if (!pending.count(in)) continue;
        const auto f = float_of_twin.find(id);
        if (f == float_of_twin.end()) continue;
        const GNode& fn = src.nodes[f->second];
        if (fn.reg != nullptr && list_inputs.count(fn.reg))
          result.calib_nodes.push_back(fn.name + "_" + list_inputs[fn.reg](fn.attrs)[i]);
        else
          result.calib_nodes.push_back(fn.name + "_" + dst.nodes[in].name);
        pending.erase(in);
      }
    }
    if (node.reg != nullptr && calib_input.count(node.reg)) {
      for (const int idx : calib_input[node.reg](node.attrs)) {
        const Entry& e = node.inputs.at(idx);
        const auto self = origin.find(id);
        if (self != origin.end()) {
          result.calib_nodes.push_back(float_output_name(self->second, e.index));
        } else if (dst.nodes[e.node].is_variable()) {
          pending.insert(id);
        } else {
          const auto producer = origin.find(e.node);
          CHECK(producer != origin.end()) << "Can't find calibration node for " << node.name;
          result.calib_nodes.push_back(float_output_name(producer->second, e.index));
        }
      }
    } else if (node.reg != nullptr && calib_output.count(node.reg)) {
      for (const int idx : calib_output[node.reg](node.attrs)) {
        const auto self = origin.find(id);
        if (self != origin.end())
          result.calib_nodes.push_back(float_output_name(self->second, static_cast<uint32_t>(idx)));
        else
          result.calib_nodes.push_back(node.name + "_" +
                                       OutputName(dst, id, static_cast<uint32_t>(idx)));
      }
    }
  }
  result.graph = std::move(dst);
  return result;
}

Graph SetCalibTable(const Graph& g_in, const std::map<std::string, std::pair<float, float>>& table) {
  static const auto calib_input =
      nnvm::Op::GetAttr<mxnet::FNeedCalibrateInput>("FNeedCalibrateInput");
  static const auto calib_output =
      nnvm::Op::GetAttr<mxnet::FNeedCalibrateOutput>("FNeedCalibrateOutput");
  Graph g = g_in;
  // The key of the tensor entry `e` observed for `node` (SetCalibTableForEntry,
  // quantize_graph_pass.cc:612-650): "<producer>_<output name>" behind an operator, with
  // a leading "quantized_" dropped; behind a variable the quantize node's own name minus
  // "_quantize".
  auto apply = [&](const Entry& e, int node_id) {
    GNode& node = g.nodes[node_id];
    const GNode& producer = g.nodes[e.node];
    std::string key = producer.name;
    if (!producer.is_variable()) {
      key += "_" + OutputName(g, e.node, e.index);
    } else {
      const std::string suffix = "_quantize";
      key = node.name;
      CHECK(key.size() >= suffix.size()) << "unexpected node name " << key;
      key.erase(key.size() - suffix.size());
    }
    const std::string prefix = "quantized_";
    if (producer.name.rfind(prefix, 0) == 0) key = key.substr(prefix.size());
    const auto it = table.find(key);
    if (it == table.end()) return;
    node.dict["min_calib_range"] = std::to_string(it->second.first);
    node.dict["max_calib_range"] = std::to_string(it->second.second);
    BindOp(&node);
  };
  for (const int id : g.PostOrder()) {
    const GNode& node = g.nodes[id];
    if (node.reg == nullptr) continue;
    if (calib_input.count(node.reg)) {
      const std::vector<int> idx = calib_input[node.reg](node.attrs);
      CHECK_EQ(idx.size(), 1U);
      apply(node.inputs.at(idx[0]), id);
    } else if (calib_output.count(node.reg)) {
      const std::vector<int> idx = calib_output[node.reg](node.attrs);
      CHECK_EQ(idx.size(), 1U);
      apply(Entry{id, static_cast<uint32_t>(idx[0]), 0}, id);
    }
  }
  return g;
}

}  // namespace mxq_graph
