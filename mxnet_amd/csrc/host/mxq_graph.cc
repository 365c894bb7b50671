// Graph arena, symbol-JSON reader / writer (see mxq_graph.h).
#include "mxq_graph.h"

#include <algorithm>
#include <cctype>
#include <cstdio>
#include <cstring>
#include <cstdlib>
#include <memory>
#include <sstream>

namespace mxq_graph {

// ---- a small JSON value -------------------------------------------------------------
namespace {

struct JValue {
  enum Kind { kNull, kBool, kNumber, kString, kArray, kObject } kind = kNull;
  bool b = false;
  double num = 0;
  std::string str;  // string value, or the literal text of a number
  std::vector<JValue> arr;
  std::vector<std::pair<std::string, JValue>> obj;  // insertion order kept
  const JValue* find(const std::string& key) const {
    for (const auto& kv : obj)
      if (kv.first == key) return &kv.second;
    return nullptr;
  }
};

class JParser {
 public:
  explicit JParser(const std::string& s) : s_(s) {}
  JValue Parse() {
    JValue v = Value();
    Skip();
    if (pos_ != s_.size()) Fail("trailing characters");
    return v;
  }

 private:
  const std::string& s_;
  size_t pos_ = 0;
  [[noreturn]] void Fail(const std::string& why) const {
    std::ostringstream os;
    os << "symbol JSON: " << why << " at offset " << pos_;
    throw dmlc::Error(os.str());
  }
  void Skip() {
    while (pos_ < s_.size() && std::isspace(static_cast<unsigned char>(s_[pos_]))) ++pos_;
  }
  char Peek() {
    Skip();
    if (pos_ >= s_.size()) Fail("unexpected end");
    return s_[pos_];
  }
  void Expect(char c) {
    if (Peek() != c) Fail(std::string("expected '") + c + "'");
    ++pos_;
  }
  JValue Value() {
    const char c = Peek();
    JValue v;
    if (c == '{') {
      v.kind = JValue::kObject;
      ++pos_;
      if (Peek() == '}') {
        ++pos_;
        return v;
      }
      while (true) {
        std::string key = String();
        Expect(':');
        v.obj.emplace_back(std::move(key), Value());
        if (Peek() == ',') {
          ++pos_;
          continue;
        }
        Expect('}');
        return v;
      }
    }
    if (c == '[') {
      v.kind = JValue::kArray;
      ++pos_;
      if (Peek() == ']') {
        ++pos_;
        return v;
      }
      while (true) {
        v.arr.push_back(Value());
        if (Peek() == ',') {
          ++pos_;
          continue;
        }
        Expect(']');
        return v;
      }
    }
    if (c == '"') {
      v.kind = JValue::kString;
      v.str = String();
      return v;
    }
    if (s_.compare(pos_, 4, "true") == 0) {
      v.kind = JValue::kBool;
      v.b = true;
      pos_ += 4;
      return v;
    }
    if (s_.compare(pos_, 5, "false") == 0) {
      v.kind = JValue::kBool;
      pos_ += 5;
      return v;
    }
    if (s_.compare(pos_, 4, "null") == 0) {
      pos_ += 4;
      return v;
    }
    const size_t start = pos_;
    while (pos_ < s_.size() && (std::isdigit(static_cast<unsigned char>(s_[pos_])) ||
                                std::strchr("+-.eE", s_[pos_]) != nullptr))
      ++pos_;
    if (pos_ == start) Fail("unexpected character");
    v.kind = JValue::kNumber;
    v.str = s_.substr(start, pos_ - start);
    v.num = std::strtod(v.str.c_str(), nullptr);
    return v;
  }
  std::string String() {
    Expect('"');
    std::string out;
    while (true) {
      if (pos_ >= s_.size()) Fail("unterminated string");
      const char c = s_[pos_++];
      if (c == '"') return out;
      if (c != '\\') {
        out.push_back(c);
        continue;
      }
      if (pos_ >= s_.size()) Fail("unterminated escape");
      const char e = s_[pos_++];
      switch (e) {
        case '"': out.push_back('"'); break;
        case '\\': out.push_back('\\'); break;
        case '/': out.push_back('/'); break;
        case 'b': out.push_back('\b'); break;
        case 'f': out.push_back('\f'); break;
        case 'n': out.push_back('\n'); break;
        case 'r': out.push_back('\r'); break;
        case 't': out.push_back('\t'); break;
        case 'u': {
          if (pos_ + 4 > s_.size()) Fail("short \\u escape");
          const unsigned cp = static_cast<unsigned>(std::strtoul(s_.substr(pos_, 4).c_str(),
                                                                 nullptr, 16));
          pos_ += 4;
          if (cp < 0x80) {
            out.push_back(static_cast<char>(cp));
          } else if (cp < 0x800) {
            out.push_back(static_cast<char>(0xC0 | (cp >> 6)));
            out.push_back(static_cast<char>(0x80 | (cp & 0x3F)));
          } else {
            out.push_back(static_cast<char>(0xE0 | (cp >> 12)));
            out.push_back(static_cast<char>(0x80 | ((cp >> 6) & 0x3F)));
            out.push_back(static_cast<char>(0x80 | (cp & 0x3F)));
          }
          break;
        }
        default: Fail("bad escape");
      }
    }
  }
};

void WriteString(std::ostringstream& os, const std::string& s) {
  os << '"';
  for (const char c : s) {
    switch (c) {
      case '"': os << "\\\""; break;
      case '\\': os << "\\\\"; break;
      case '\n': os << "\\n"; break;
      case '\r': os << "\\r"; break;
      case '\t': os << "\\t"; break;
      default:
        if (static_cast<unsigned char>(c) < 0x20) {
          char buf[8];
          std::snprintf(buf, sizeof(buf), "\\u%04x", c);
          os << buf;
        } else {
          os << c;
        }
    }
  }
  os << '"';
}

int AsInt(const JValue& v, const char* what) {
  if (v.kind != JValue::kNumber) throw dmlc::Error(std::string("symbol JSON: ") + what);
  return static_cast<int>(v.num);
}

}  // namespace

// ---- graph ----------------------------------------------------------------------------

void BindOp(GNode* node) {
  node->reg = node->is_variable() ? nullptr : nnvm::Op::Find(node->op);
  node->attrs = nnvm::NodeAttrs();
  node->attrs.name = node->name;
  node->attrs.op = node->reg;
  for (const auto& kv : node->dict) node->attrs.dict[kv.first] = kv.second;
  if (node->reg != nullptr && node->reg->attr_parser) node->reg->attr_parser(&node->attrs);
}

int Graph::AddNode(const std::string& op, const std::string& name,
                   const std::map<std::string, std::string>& dict) {
  GNode n;
  n.op = op;
  n.name = name;
  n.dict = dict;
  BindOp(&n);
  nodes.push_back(std::move(n));
  return static_cast<int>(nodes.size()) - 1;
}

std::vector<int> Graph::PostOrder() const {
  std::vector<int> order;
  std::vector<char> seen(nodes.size(), 0);
  std::vector<std::pair<int, size_t>> stack;  // node, next input to look at
  for (const Entry& h : heads) {
    if (seen[h.node]) continue;
    seen[h.node] = 1;
    stack.emplace_back(h.node, 0);
    while (!stack.empty()) {
      auto& top = stack.back();
      const GNode& n = nodes[top.first];
      if (top.second < n.inputs.size()) {
        const int next = n.inputs[top.second++].node;
        if (!seen[next]) {
          seen[next] = 1;
          stack.emplace_back(next, 0);
        }
      } else {
        order.push_back(top.first);
        stack.pop_back();
      }
    }
  }
  return order;
}

uint32_t Graph::NumOutputs(int node) const {
  const GNode& n = nodes[node];
  if (n.is_variable()) return 1;
  if (n.reg != nullptr) return n.reg->NumOutputs(n.attrs);
  uint32_t most = 0;
  for (const GNode& c : nodes)
    for (const Entry& e : c.inputs)
      if (e.node == node) most = std::max(most, e.index);
  for (const Entry& e : heads)
    if (e.node == node) most = std::max(most, e.index);
  return most + 1;
}

std::string OutputName(const Graph& g, int node, uint32_t index) {
  static const auto flist = nnvm::Op::GetAttr<nnvm::FListOutputNames>("FListOutputNames");
  const GNode& n = g.nodes[node];
  if (n.reg != nullptr && flist.count(n.reg)) {
    const std::vector<std::string> names = flist[n.reg](n.attrs);
    CHECK(names.size() > index) << "output " << index << " of " << n.name << " has no name";
    return names[index];
  }
  return std::to_string(index);
}

Graph LoadJSON(const std::string& json) {
  const JValue root = JParser(json).Parse();
  if (root.kind != JValue::kObject) throw dmlc::Error("symbol JSON: top level is not an object");
  const JValue* jnodes = root.find("nodes");
  const JValue* jheads = root.find("heads");
  if (!jnodes || jnodes->kind != JValue::kArray || !jheads || jheads->kind != JValue::kArray)
    throw dmlc::Error("symbol JSON: missing \"nodes\" or \"heads\"");
  Graph g;
  auto entry = [&](const JValue& v, size_t limit) {
    if (v.kind != JValue::kArray || v.arr.size() < 2)
      throw dmlc::Error("symbol JSON: a node entry is [node, index, version]");
    Entry e;
    e.node = AsInt(v.arr[0], "entry node id");
    e.index = static_cast<uint32_t>(AsInt(v.arr[1], "entry index"));
    e.version = v.arr.size() > 2 ? static_cast<uint32_t>(AsInt(v.arr[2], "entry version")) : 0;
    if (e.node < 0 || static_cast<size_t>(e.node) >= limit)
      throw dmlc::Error("symbol JSON: entry refers to a later or missing node");
    return e;
  };
  for (const JValue& jn : jnodes->arr) {
    if (jn.kind != JValue::kObject) throw dmlc::Error("symbol JSON: node is not an object");
    const JValue* op = jn.find("op");
    const JValue* name = jn.find("name");
    if (!op || op->kind != JValue::kString || !name || name->kind != JValue::kString)
      throw dmlc::Error("symbol JSON: node without \"op\" or \"name\"");
    GNode n;
    n.op = op->str;
    n.name = name->str;
    // "attrs" today; "attr" and "param" in files written by older versions
    for (const char* key : {"param", "attr", "attrs"}) {
      const JValue* a = jn.find(key);
      if (!a || a->kind != JValue::kObject) continue;
      for (const auto& kv : a->obj) {
        if (kv.second.kind != JValue::kString)
          throw dmlc::Error("symbol JSON: attribute values are strings");
        n.dict[kv.first] = kv.second.str;
      }
    }
    const JValue* inputs = jn.find("inputs");
    if (inputs && inputs->kind == JValue::kArray)
      for (const JValue& ji : inputs->arr) n.inputs.push_back(entry(ji, g.nodes.size()));
    BindOp(&n);
    g.nodes.push_back(std::move(n));
  }
  for (const JValue& jh : jheads->arr) g.heads.push_back(entry(jh, g.nodes.size()));
  return g;
}

std::string SaveJSON(const Graph& g) {
  const std::vector<int> order = g.PostOrder();
  std::vector<int> new_id(g.nodes.size(), -1);
  for (size_t i = 0; i < order.size(); ++i) new_id[order[i]] = static_cast<int>(i);
  std::ostringstream os;
  os << "{\n  \"nodes\": [\n";
  std::vector<int> arg_nodes;
  std::vector<uint32_t> row_ptr(1, 0);
  for (size_t i = 0; i < order.size(); ++i) {
    const GNode& n = g.nodes[order[i]];
    if (n.is_variable()) arg_nodes.push_back(static_cast<int>(i));
    row_ptr.push_back(row_ptr.back() + g.NumOutputs(order[i]));
    os << "    {\n      \"op\": ";
    WriteString(os, n.op);
    os << ", \n      \"name\": ";
    WriteString(os, n.name);
    os << ", \n";
    if (!n.dict.empty()) {
      os << "      \"attrs\": {";
      bool first = true;
      for (const auto& kv : n.dict) {
        os << (first ? "\n        " : ", \n        ");
        first = false;
        WriteString(os, kv.first);
        os << ": ";
        WriteString(os, kv.second);
      }
      os << "\n      }, \n";
    }
    os << "      \"inputs\": [";
    for (size_t j = 0; j < n.inputs.size(); ++j) {
      const Entry& e = n.inputs[j];
      os << (j ? ", " : "") << "[" << new_id[e.node] << ", " << e.index << ", " << e.version << "]";
    }
    os << "]\n    }" << (i + 1 < order.size() ? ", " : "") << "\n";
  }
  os << "  ], \n  \"arg_nodes\": [";
  for (size_t i = 0; i < arg_nodes.size(); ++i) os << (i ? ", " : "") << arg_nodes[i];
  os << "], \n  \"node_row_ptr\": [";
  for (size_t i = 0; i < row_ptr.size(); ++i) os << (i ? ", " : "") << row_ptr[i];
  os << "], \n  \"heads\": [";
  for (size_t i = 0; i < g.heads.size(); ++i) {
    const Entry& e = g.heads[i];
    os << (i ? ", " : "") << "[" << new_id[e.node] << ", " << e.index << ", " << e.version << "]";
  }
  os << "], \n  \"attrs\": {\"mxnet_version\": [\"int\", 20000]}\n}";
  return os.str();
}

}  // namespace mxq_graph
