#include "lite/core/optimizer/mir/graph.h"

#include <algorithm>
#include <set>

namespace paddle {
namespace lite {
namespace mir {

void Graph::Link(Node* from, Node* to) {
  from->outlinks.push_back(to);
  to->inlinks.push_back(from);
}

Graph::Graph(const std::vector<OpInfo>& ops, const Scope& scope) {
  for (size_t i = 0; i < ops.size(); ++i) {
    for (const auto& kv : ops[i].inputs()) {
      for (const std::string& name : kv.second) {
        Variable* v = scope.FindVar(name);
        RetrieveVarNode(name, v != nullptr && v->GetMutable<Tensor>()->persistable());
      }
    }
    CreateOpNode(ops[i], static_cast<int>(i));
  }
}

Graph::Node* Graph::RetrieveVarNode(const std::string& name, bool is_weight) {
  auto it = vars_.find(name);
  if (it != vars_.end()) return it->second;
  nodes_.emplace_back();
  Node* n = &nodes_.back();
  n->name = name;
  n->is_weight = is_weight;
  vars_[name] = n;
  return n;
}

Graph::Node* Graph::CreateOpNode(const OpInfo& op, int order) {
  nodes_.emplace_back();
  Node* n = &nodes_.back();
  n->is_op = true;
  n->op = op;
  n->order = order;
  for (const auto& kv : op.inputs())
    for (const std::string& name : kv.second) Link(RetrieveVarNode(name, false), n);
  for (const auto& kv : op.outputs()) {
    for (const std::string& name : kv.second) {
      Node* v = RetrieveVarNode(name, false);
      CHECK(v->inlinks.empty()) << "variable " << name << " is written by two ops: the graph must be in single-assignment form";
      Link(n, v);
    }
  }
  return n;
}

void Graph::RemoveNode(Node* n) {
  for (Node* in : n->inlinks) in->outlinks.erase(std::remove(in->outlinks.begin(), in->outlinks.end(), n), in->outlinks.end());
  for (Node* out : n->outlinks) out->inlinks.erase(std::remove(out->inlinks.begin(), out->inlinks.end(), n), out->inlinks.end());
  if (!n->is_op) vars_.erase(n->name);
  nodes_.remove_if([n](const Node& x) { return &x == n; });
}

std::vector<Graph::Node*> Graph::OpNodes() {
  std::vector<Node*> v;
  for (Node& n : nodes_)
    if (n.is_op) v.push_back(&n);
  std::stable_sort(v.begin(), v.end(), [](const Node* a, const Node* b) { return a->order < b->order; });
  return v;
}

std::vector<const Graph::Node*> Graph::OpNodes() const {
  std::vector<const Node*> v;
  for (const Node& n : nodes_)
    if (n.is_op) v.push_back(&n);
  std::stable_sort(v.begin(), v.end(), [](const Node* a, const Node* b) { return a->order < b->order; });
  return v;
}

Graph::Node* Graph::Var(const std::string& name) {
  auto it = vars_.find(name);
  return it == vars_.end() ? nullptr : it->second;
}

const Graph::Node* Graph::Var(const std::string& name) const {
  auto it = vars_.find(name);
  return it == vars_.end() ? nullptr : it->second;
}

const Graph::Node* Graph::Producer(const std::string& var) const {
  const Node* v = Var(var);
  return (v == nullptr || v->inlinks.empty()) ? nullptr : v->inlinks.front();
}

std::vector<const Graph::Node*> Graph::Consumers(const std::string& var) const {
  std::vector<const Node*> c;
  if (const Node* v = Var(var)) {
    for (const Node* o : v->outlinks)
      if (std::find(c.begin(), c.end(), o) == c.end()) c.push_back(o);
  }
  std::stable_sort(c.begin(), c.end(), [](const Node* a, const Node* b) { return a->order < b->order; });
  return c;
}

std::vector<OpInfo> Graph::TopologicalOps() const {
  std::vector<const Node*> pending = OpNodes();
  std::set<const Node*> done;
  std::vector<OpInfo> out;
  while (!pending.empty()) {
    bool progressed = false;
    for (auto it = pending.begin(); it != pending.end(); ++it) {
      bool ready = true;
      for (const Node* v : (*it)->inlinks)
        for (const Node* producer : v->inlinks) ready = ready && done.count(producer) != 0;
      if (!ready) continue;
      out.push_back((*it)->op);
      done.insert(*it);
      pending.erase(it);
      progressed = true;
      break;  // restart: the earliest ready op comes next
    }
    CHECK(progressed) << "the graph has a cycle";
  }
  return out;
}

}  // namespace mir
}  // namespace lite
}  // namespace paddle
