#include "lowering.h"

#include "executor.h"

namespace cavs {
namespace mid {

std::unique_ptr<Lowering> match_vertex_function(const Graph &) { return nullptr; }

void Executor::lowered_forward(const int32_t *, int, int, float *) { fail(CAVS_EUNSUPPORTED, "no lowering"); }
void Executor::lowered_backward(const OpDef &) { fail(CAVS_EUNSUPPORTED, "no lowering"); }

}  // namespace mid
}  // namespace cavs
