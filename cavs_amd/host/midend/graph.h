// Graph IR of the midend: scopes of nodes and edges built from OpDefs, shape inference,
// dynamic-edge marking for the vertex function, and the autograd pass that derives the
// backward program (including the backward vertex function).  Restates the parts of
// cavs/midend/{scope,node,edge,graph_util}.{h,cc} and cavs/backend/op_decl_*.cc that the
// F-over-G path needs, over plain structs.
#ifndef CAVS_HOST_MIDEND_GRAPH_H_
#define CAVS_HOST_MIDEND_GRAPH_H_

#include <map>
#include <memory>
#include <set>
#include <string>
#include <vector>

#include "cavs/proto/op_def.h"

namespace cavs {
namespace mid {

struct Node;
struct Scope;

struct Edge {
  std::string name;
  std::vector<int> shape;   // -1 = the batch's total vertex count (GraphOutput and what follows it)
  bool dynamic = false;     // inside F: one row per vertex of the round (graph_util.cc:309-318)
  Node *src = nullptr;
  std::vector<Node *> dst;
  Scope *scope = nullptr;
  // elements per row (dynamic / -1-shaped edges) or in total (static edges)
  long width() const {
    long w = 1;
    for (int d : shape) if (d > 0) w *= d;
    return w;
  }
  bool per_vertex() const {
    if (dynamic) return true;
    for (int d : shape) if (d < 0) return true;
    return false;
  }
};

struct Node {
  OpDef def;
  std::vector<Edge *> in, out;
  Scope *scope = nullptr;
  std::vector<std::string> after;  // control dependencies: edges that must be computed first
};

struct Scope {
  std::string name;
  Scope *parent = nullptr;
  std::vector<std::unique_ptr<Node>> nodes;  // creation order == a topological order
  std::map<std::string, std::unique_ptr<Edge>> edges;
  Edge *find(const std::string &n, bool upward = true) const;
  Edge *add_edge(const std::string &n, const std::vector<int> &shape);
};

struct OptimizerSpec {
  bool present = false;
  std::string output;          // the symbol that triggers a training step
  std::string loss;
  std::vector<std::string> vars;
  float lr = 1.f, clip = 0.f;
  int iters = 1;
  std::vector<OpDef> backward;  // main-scope backward program in execution order
};

struct Graph {
  Scope main;
  std::unique_ptr<Scope> func;            // "Node"
  std::vector<OpDef> func_backward;       // backward vertex function, per-round part
  std::vector<OpDef> func_deferred;       // weight-gradient part, run once over all rows
  std::vector<std::string> func_inputs;   // external edges F reads (weights etc.)
  std::vector<int> func_ret_shape;
  std::string graph_output;               // name of the GraphOutput edge, if any
  OptimizerSpec opt;
  int version = 0;                        // bumped on every change (sessions recompile)

  Graph() { main.name = "main"; }
  // returns the inferred shape of output 0
  std::vector<int> add_op(const OpDef &def);
  std::vector<int> add_function(const FunctionDef &def);
  void add_optimizer(const OpDef &def);
  void add_control_dependency(const OpDef &def);
  std::string dump() const;
};

Graph &global_graph();
void reset_global_graph();
// installs `g` as the process-wide graph and returns the previous one (used to declare
// template programs without disturbing the user's)
Graph *swap_global_graph(Graph *g);

// shape inference for one op; inputs are the input edges in order
std::vector<std::vector<int>> infer_shapes(const OpDef &def, const std::vector<const Edge *> &in);

[[noreturn]] void graph_error(const std::string &msg);

}  // namespace mid
}  // namespace cavs
#endif
