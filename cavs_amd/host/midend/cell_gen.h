// Lowering of a vertex function of the general shape onto generated round kernels:
// recognises  act(sum_i Gather_i * W_i + Pull * W + b)  with any elementwise tail over the
// pre-activations and the children's states, cuts a function whose products depend on each other
// into a chain of such cells, derives the elementwise part of each one's backward
// function, and writes the kernels' source (the product loops for this function's operands plus
// the two elementwise parts).  The counterpart of the reference's parser + code generator
// (cavs/midend/runtime_compiler/parser.cc:73-139, code_generator.cc:104-185) for a whole F.
#ifndef CAVS_HOST_MIDEND_CELL_GEN_H_
#define CAVS_HOST_MIDEND_CELL_GEN_H_

#include <map>
#include <memory>
#include <string>

#include "../cell.h"
#include "graph.h"

namespace cavs {
namespace mid {

struct CellSlot {
  std::string param;  // engine parameter
  long offset = 0, count = 0;
};

struct CellMatch {
  std::shared_ptr<CellSpec> spec;
  std::map<std::string, std::string> roles;  // role -> name of the main-scope edge that supplies it
  std::map<std::string, CellSlot> slots;     // role -> where it lives in the engine's parameters
};

// null when F is not of that shape; `why` then says what stood in the way
std::unique_ptr<CellMatch> match_cell(const Graph &g, std::string *why = nullptr);

// The elementwise parts alone as host C++ (cell_forward / cell_backward over plain structs), for
// checking the derived backward part against finite differences without a device.
// (stage: which cell of the chain a function of several stages is cut into; 0 for a function of one)
std::string cell_host_source(const Graph &g, int stage = 0);

// A main-scope edge traced back through aliasing ops to the Variable it views.
struct Resolved {
  std::string var;
  long offset = 0, count = 0;
  bool ok = false;
};
Resolved resolve_external(const Edge *e);

}  // namespace mid
}  // namespace cavs
#endif
