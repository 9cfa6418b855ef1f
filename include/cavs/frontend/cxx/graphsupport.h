// Vertex-function declaration.  An application derives from GraphSupport and writes Node():
// the body every vertex of every instance graph runs, built from Pull (the vertex's own input
// row), Gather (the message of child i), Scatter (the message for the parent) and Push (the
// vertex's return value).  Output() declares the function and hands back the GraphOutput symbol,
// one row per vertex.  Same class, method names and argument meaning as
// cavs/frontend/cxx/graphsupport.h:9-27, so an application written against that header compiles
// against this one.
#pragma once

#include <vector>

#include "cavs/frontend/cxx/sym.h"

class GraphSupport {
 protected:
  // ---- what Node() is written with ----
  // row `column_offset` .. of this vertex in the vertex placeholder, viewed as `row_shape`
  Sym Pull(int column_offset, const std::vector<int> &row_shape);
  // message Scatter'ed by child `child_index` (zeros when there is no such child)
  Sym Gather(int child_index, const std::vector<int> &row_shape);
  void Scatter(const Sym &message);
  void Push(const Sym &result);

 public:
  GraphSupport(const Sym &graph_placeholder, const Sym &vertex_placeholder);
  virtual ~GraphSupport();
  // runs Node() once between the function's begin and end markers and returns GraphOutput
  Sym Output();
  virtual void Node() = 0;

 private:
  Sym graph_placeholder_, vertex_placeholder_;
};
