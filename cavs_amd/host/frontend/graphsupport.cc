// GraphSupport: records Node() into a FunctionDef named "Node", registers it, and emits
// the GraphOutput op (cavs/frontend/cxx/graphsupport.cc:10-93).
#include "cavs/frontend/cxx/graphsupport.h"

#include <cstdlib>

#include "cavs/util/op_def_builder.h"

GraphSupport::GraphSupport(const Sym &graph_placeholder, const Sym &vertex_placeholder)
    : graph_placeholder_(graph_placeholder), vertex_placeholder_(vertex_placeholder) {}

GraphSupport::~GraphSupport() = default;

Sym GraphSupport::Output() {
  FuncConf::FuncDefineBegin("Node");
  this->Node();
  FunctionDef func = FuncConf::FuncDefineEnd("Node");
  string bytes;
  func.SerializeToString(&bytes);
  int *dim = nullptr;
  size_t n = 0;
  C_AddFunction(bytes.data(), bytes.size(), &dim, &n);
  CHECK(n > 0) << "the vertex function pushes nothing";
  int width = 1;
  for (size_t i = 0; i < n; i++) width *= dim[i];
  std::free(dim);
  int max_nodes = 1;
  for (int d : graph_placeholder_.shape(0)) max_nodes *= d;
  return Sym(OpDefBuilder("GraphOutput").Input(graph_placeholder_.output(0)).Input(vertex_placeholder_.output(0))
                 .Dtype(vertex_placeholder_.type()).Device(vertex_placeholder_.device()).Shape({-1, width})
                 .AttrSingle("Wavefront", true).AttrSingle("MaxGraphNodeCount", max_nodes).Finalize());
}

Sym GraphSupport::Gather(int child, const std::vector<int> &shape) {
  CHECK(!shape.empty());
  return Sym(OpDefBuilder("Gather").Dtype(vertex_placeholder_.type()).Device(vertex_placeholder_.device()).Shape(shape)
                 .AttrSingle("Child", child).Finalize());
}

Sym GraphSupport::Pull(int offset, const std::vector<int> &shape) {
  return Sym(OpDefBuilder("Pull").Dtype(vertex_placeholder_.type()).Device(vertex_placeholder_.device()).Shape(shape)
                 .AttrSingle("Offset", offset).Finalize());
}

void GraphSupport::Push(const Sym &s) {
  Sym added(OpDefBuilder("Push").Input(s.output(0)).Dtype(s.type()).Device(s.device()).Finalize());
}

void GraphSupport::Scatter(const Sym &s) {
  // the reference hard-codes Child = 0 (graphsupport.cc:84-93)
  Sym added(OpDefBuilder("Scatter").Input(s.output(0)).Dtype(s.type()).Device(s.device()).AttrSingle("Child", 0).Finalize());
}
