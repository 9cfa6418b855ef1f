// Recognition of the vertex functions the engine runs on fused round kernels.  A user's F is
// lowered onto cavs::Engine when its operator graph is the same computation as one of the
// templates with hand-written kernels (binary Tree-LSTM, chain LSTM, Tree-FC: same operators, same
// wiring, same attributes), or, failing that, when it has the general shape that
// generated kernels cover (cell_gen.h) -- everything else runs op by op.
#ifndef CAVS_HOST_MIDEND_LOWERING_H_
#define CAVS_HOST_MIDEND_LOWERING_H_

#include <map>
#include <memory>
#include <string>

#include "cell_gen.h"
#include "graph.h"

namespace cavs {
namespace mid {

struct Lowering {
  int model = 0;                  // CAVS_MODEL_*
  int H = 0, E = 0, V = 0;
  int act = 0, use_bias = 0, use_x = 0;
  // role -> name of the main-scope edge that supplies it
  std::map<std::string, std::string> roles;
  // model == CAVS_MODEL_CELL: the generated kernels and where each role lives in their parameters
  std::shared_ptr<CellSpec> cell;
  std::map<std::string, CellSlot> cell_slots;
};

// mode 1: the hand-written templates first, then the general shape; 2: the general shape only
std::unique_ptr<Lowering> match_vertex_function(const Graph &g, int mode = 1);

}  // namespace mid
}  // namespace cavs
#endif
