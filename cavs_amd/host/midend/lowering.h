// Recognition of the vertex functions the fused round kernels implement.  A user's F is
// lowered onto cavs::Engine only when its operator graph is the same computation as one
// of the templates (binary Tree-LSTM, chain LSTM, Tree-FC): same operators, same
// wiring, same attributes -- everything else runs op by op.
#ifndef CAVS_HOST_MIDEND_LOWERING_H_
#define CAVS_HOST_MIDEND_LOWERING_H_

#include <map>
#include <memory>
#include <string>

#include "graph.h"

namespace cavs {
namespace mid {

struct Lowering {
  int model = 0;                  // CAVS_MODEL_*
  int H = 0, E = 0, V = 0;
  int act = 0, use_bias = 0, use_x = 0;
  // role -> name of the main-scope edge that supplies it
  std::map<std::string, std::string> roles;
};

std::unique_ptr<Lowering> match_vertex_function(const Graph &g);

}  // namespace mid
}  // namespace cavs
#endif
