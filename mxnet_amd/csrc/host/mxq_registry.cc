// The operator registry behind NNVM_REGISTER_OP in the stand-alone build.
#include <map>
#include <mutex>

#include "mxq_shim.h"

namespace nnvm {

namespace {
struct Registry {
  std::map<std::string, std::unique_ptr<Op>> ops;
  std::map<std::string, Op*> by_name;  // names and aliases
  std::mutex mu;
  static Registry& Get() {
    static Registry* r = new Registry();  // never destroyed: ops are used from static dtors
    return *r;
  }
};
}  // namespace

std::unordered_map<std::string, std::unordered_map<const Op*, std::any>>& Op::AttrTable() {
  static auto* t = new std::unordered_map<std::string, std::unordered_map<const Op*, std::any>>();
  return *t;
}

Op& Op::RegisterOrGet(const std::string& name) {
  Registry& r = Registry::Get();
  std::lock_guard<std::mutex> lk(r.mu);
  auto it = r.by_name.find(name);
  if (it != r.by_name.end()) return *it->second;
  std::unique_ptr<Op> op(new Op());
  op->name = name;
  Op* p = op.get();
  r.ops[name] = std::move(op);
  r.by_name[name] = p;
  return *p;
}

Op& Op::add_alias(const std::string& alias) {
  Registry& r = Registry::Get();
  std::lock_guard<std::mutex> lk(r.mu);
  r.by_name[alias] = this;
  return *this;
}

const Op* Op::Get(const std::string& name) {
  Registry& r = Registry::Get();
  std::lock_guard<std::mutex> lk(r.mu);
  auto it = r.by_name.find(name);
  if (it == r.by_name.end()) throw dmlc::Error("Operator " + name + " is not registered");
  return it->second;
}

const Op* Op::Find(const std::string& name) {
  Registry& r = Registry::Get();
  std::lock_guard<std::mutex> lk(r.mu);
  auto it = r.by_name.find(name);
  return it == r.by_name.end() ? nullptr : it->second;
}

std::vector<std::string> Op::ListAllNames() {
  Registry& r = Registry::Get();
  std::lock_guard<std::mutex> lk(r.mu);
  std::vector<std::string> names;
  for (const auto& kv : r.ops) names.push_back(kv.first);
  return names;
}

}  // namespace nnvm
