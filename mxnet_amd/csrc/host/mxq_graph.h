// Symbol graphs for the quantization passes: an index-based arena instead of the
// reference's shared-pointer node graph, with the reader and writer of the NNVM
// symbol JSON (the `-symbol.json` files of the reference; nnvm::Graph <-> JSON is
// the un-vendored 3rdparty/tvm/nnvm/src/pass/saveload_json.cc, format visible in
// every model the reference exports: {"nodes": [{"op", "name", "attrs", "inputs":
// [[node, index, version], ...]}, ...], "arg_nodes", "node_row_ptr", "heads",
// "attrs": {"mxnet_version": ["int", N]}}).
#ifndef MXQ_GRAPH_H_
#define MXQ_GRAPH_H_

#include <cstdint>
#include <functional>
#include <map>
#include <string>
#include <utility>
#include <vector>

#include "mxq_shim.h"

namespace mxq_graph {

struct Entry {
  int node = -1;        // index into Graph::nodes
  uint32_t index = 0;   // which output of that node
  uint32_t version = 0;
  bool operator<(const Entry& o) const {
    return node != o.node ? node < o.node : index < o.index;  // version is not part of identity
  }
};

struct GNode {
  std::string op;    // "null" for a variable
  std::string name;
  std::map<std::string, std::string> dict;  // attributes as written in the JSON
  std::vector<Entry> inputs;
  const nnvm::Op* reg = nullptr;            // registry entry when the operator is known here
  nnvm::NodeAttrs attrs;                    // parsed attributes (only when reg != nullptr)
  bool is_variable() const { return op == "null"; }
};

struct Graph {
  std::vector<GNode> nodes;  // an arena: not every node needs to be reachable
  std::vector<Entry> heads;

  int AddNode(const std::string& op, const std::string& name,
              const std::map<std::string, std::string>& dict = {});
  // Post-order walk over everything reachable from the heads (inputs in order, a node
  // after its inputs, each node once): the visiting order of nnvm::DFSVisit.
  std::vector<int> PostOrder() const;
  // Outputs a node has: registry value, or 1 + the largest index any consumer uses.
  uint32_t NumOutputs(int node) const;
};

// Binds GNode::reg / attrs from the registry and runs the operator's attribute parser.
void BindOp(GNode* node);

Graph LoadJSON(const std::string& json);
// Writes the nodes reachable from the heads, renumbered in post-order.
std::string SaveJSON(const Graph& g);

// Name of output `index` of a node as the passes spell it: FListOutputNames when
// registered, the decimal index otherwise (quantize_graph_pass.cc:45-62).
std::string OutputName(const Graph& g, int node, uint32_t index);

}  // namespace mxq_graph

#endif  // MXQ_GRAPH_H_
