// A small SSA graph of op nodes and variable nodes with directed links, the
// part of the reference's mir::SSAGraph / mir::Node
// (lite/core/optimizer/mir/ssa_graph.h, node.h) that the passes of this slice
// need: who produces a variable, who consumes it, replacing an op node and
// dropping variable nodes nothing refers to any more.
#pragma once

#include <list>
#include <map>
#include <string>
#include <vector>

#include "lite/core/op_desc.h"
#include "lite/core/scope.h"

namespace paddle {
namespace lite {
namespace mir {

class Graph {
 public:
  struct Node {
    bool is_op = false;
    OpInfo op;               // op nodes
    std::string name;        // variable nodes
    bool is_weight = false;  // variable nodes: a persistable tensor of the scope
    int order = 0;           // op nodes: position in the list the graph was built from (or of the op it replaced)
    std::vector<Node*> inlinks, outlinks;
  };

  // One op node per op and one variable node per name; every input and
  // output argument becomes a link.  A variable written by two ops is
  // refused (the reference renames such variables when it builds its graph;
  // the programs of this slice are already in single-assignment form).
  Graph(const std::vector<OpInfo>& ops, const Scope& scope);
  Graph(const Graph&) = delete;
  Graph& operator=(const Graph&) = delete;

  // Op nodes in list order.
  std::vector<Node*> OpNodes();
  std::vector<const Node*> OpNodes() const;
  Node* Var(const std::string& name);
  const Node* Var(const std::string& name) const;
  // The op node that writes the variable (nullptr for feeds and weights) and
  // the op nodes that read it, in list order.
  const Node* Producer(const std::string& var) const;
  std::vector<const Node*> Consumers(const std::string& var) const;

  Node* RetrieveVarNode(const std::string& name, bool is_weight);
  // New op node linked to the variables its description names.
  Node* CreateOpNode(const OpInfo& op, int order);
  // Unlinks the node from its neighbours and deletes it.
  void RemoveNode(Node* n);

  // The ops in an order in which every variable is produced before it is
  // consumed; ops that are ready at the same time keep their list order.
  std::vector<OpInfo> TopologicalOps() const;

 private:
  static void Link(Node* from, Node* to);
  std::list<Node> nodes_;
  std::map<std::string, Node*> vars_;
};

}  // namespace mir
}  // namespace lite
}  // namespace paddle
