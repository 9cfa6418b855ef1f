// Runtime fusion pass (OPT_FUSION): groups connected elementwise operators of a program
// into FusedKernel nodes and generates one HIP kernel per group, which the backend
// compiles with its runtime compiler.  Restates cavs/midend/runtime_compiler/
// {parser,code_generator,statement_builder}.cc and expression.h: same fusable operator
// set, same kernel signature (outputs, const inputs, output counts, input counts,
// n_elements), inputs read as x[idx % x_count].
#ifndef CAVS_HOST_MIDEND_FUSION_H_
#define CAVS_HOST_MIDEND_FUSION_H_

#include <functional>
#include <set>
#include <string>
#include <vector>

#include "cavs/proto/op_def.h"

namespace cavs {
namespace mid {

struct FusionEnv {
  // true when the edge holds one row per vertex of the round (counts scale with the round)
  std::function<bool(const std::string &)> per_row;
  // elements per row (per-row edges) or in total
  std::function<long(const std::string &)> width;
  // edges that must stay materialised because something outside the program reads them
  std::set<std::string> live;
};

// Returns the program with every profitable group replaced by one FusedKernel OpDef
// (attributes KernelName, KernelSource) placed where the group's last member stood.
std::vector<OpDef> fuse_program(const std::vector<OpDef> &prog, const FusionEnv &env, int *groups_made = nullptr);

// operands of `d` that its implementation reads (the *_grad operators carry an unused one)
int operands_read(const OpDef &d);

// The backward vertex function after the pass.  Its deferred part (the gradient ops that run
// once over all rows after the round loop, cavs/midend/batch_weight_updater.h:12-84) holds ops
// that only add a per-row value up over the rows -- the gradient of an operand that was broadcast
// over the rows, e.g. a bias.  Such an op can ride in a per-round generated kernel as a reducing
// output: the kernel adds each round's rows onto the output, which is zeroed once before the
// loop (`zero_before_loop`).  They are offered to the pass behind the per-round program; those
// it does not take into a kernel stay deferred.  Only the sole writer of its output qualifies
// (another deferred writer would run after it and overwrite the sum).  `env.live` must hold what
// everything outside the backward function reads.
struct BackwardFusion {
  std::vector<OpDef> per_round, deferred;
  std::vector<std::string> zero_before_loop;
  int groups = 0;
};
BackwardFusion fuse_function_backward(const std::vector<OpDef> &per_round, const std::vector<OpDef> &deferred, FusionEnv env);

struct Graph;
// geometry callbacks over the declared program (the live set is left empty)
FusionEnv graph_env(const Graph &g);
// Text of the vertex function's programs and the main program after the pass, for tests
// and inspection; needs no device.
std::string dump_fused(const Graph &g);

}  // namespace mid
}  // namespace cavs
#endif
