// The front end's C API (include/cavs/frontend/c_api.h) over the midend.  The
// reference's functions have no error channel and CHECK-abort; here a failure prints
// the message, records it for C_LastError and aborts the same way.
#include "cavs/frontend/c_api.h"

#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>

#include "../midend/cell_gen.h"
#include "../midend/executor.h"
#include "../midend/fusion.h"
#include "../midend/graph.h"

using cavs::mid::Executor;
using cavs::mid::HostTensor;

struct C_Session {
  Executor exec;
  C_Session(int opt, const std::string &name) : exec(opt, name) {}
};
struct C_Tensor {
  HostTensor t;
};

namespace {
thread_local std::string g_err;

template <typename F>
bool guarded(const char *where, F &&f) {
  try {
    f();
    return true;
  } catch (const std::exception &e) {
    g_err = std::string(where) + ": " + e.what();
    return false;
  }
}
template <typename F>
void must(const char *where, F &&f) {
  if (!guarded(where, f)) {
    std::fprintf(stderr, "[cavs] fatal: %s\n", g_err.c_str());
    std::abort();
  }
}
void give_shape(const std::vector<int> &s, int **dim, size_t *n) {
  *n = s.size();
  *dim = static_cast<int *>(std::malloc(sizeof(int) * (s.empty() ? 1 : s.size())));
  for (size_t i = 0; i < s.size(); i++) (*dim)[i] = s[i];
}
}  // namespace

extern "C" {

const char *C_LastError(void) { return g_err.c_str(); }

C_Session *C_NewSession(const char *name, size_t name_len, int opt) {
  C_Session *s = nullptr;
  must("C_NewSession", [&] { s = new C_Session(opt, std::string(name ? name : "", name ? name_len : 0)); });
  return s;
}

void C_DeleteSession(C_Session *s) { delete s; }

C_Tensor *C_NewTensor(const char *name, size_t name_len, const int *shape, int dims, C_Dtype dtype) {
  auto *t = new C_Tensor;
  t->t.name.assign(name, name_len);
  t->t.shape.assign(shape, shape + dims);
  size_t n = 1;
  for (int i = 0; i < dims; i++) n *= (size_t)shape[i];
  t->t.data.resize(n * (dtype == C_DOUBLE ? 8 : 4));
  return t;
}

void C_DeleteTensor(C_Tensor *t) { delete t; }
void *C_TensorData(const C_Tensor *t) { return const_cast<char *>(t->t.data.data()); }
size_t C_TensorSize(const C_Tensor *t) { return t->t.data.size(); }

void C_AddOp(const void *def, size_t len, int **dim, size_t *dim_length) {
  must("C_AddOp", [&] {
    OpDef d;
    if (!d.ParseFromArray(def, len)) throw std::runtime_error("malformed OpDef bytes");
    give_shape(cavs::mid::global_graph().add_op(d), dim, dim_length);
  });
}

void C_AddFunction(const void *def, size_t len, int **dim, size_t *dim_length) {
  must("C_AddFunction", [&] {
    FunctionDef f;
    if (!f.ParseFromArray(def, len)) throw std::runtime_error("malformed FunctionDef bytes");
    give_shape(cavs::mid::global_graph().add_function(f), dim, dim_length);
  });
}

void C_AddOptimizerOp(const void *def, size_t len) {
  must("C_AddOptimizerOp", [&] {
    OpDef d;
    if (!d.ParseFromArray(def, len)) throw std::runtime_error("malformed OpDef bytes");
    cavs::mid::global_graph().add_optimizer(d);
  });
}

void C_AddControlDependency(const void *def, size_t len) {
  must("C_AddControlDependency", [&] {
    OpDef d;
    if (!d.ParseFromArray(def, len)) throw std::runtime_error("malformed OpDef bytes");
    cavs::mid::global_graph().add_control_dependency(d);
  });
}

static void run_impl(C_Session *s, const char **out_names, C_Tensor **out_tensors, int nout, const char **in_names,
                     C_Tensor *const *in_tensors, int nin) {
  std::vector<std::string> outs(out_names, out_names + nout);
  std::vector<std::pair<std::string, const HostTensor *>> feeds;
  for (int i = 0; i < nin; i++) feeds.emplace_back(in_names[i], &in_tensors[i]->t);
  std::vector<HostTensor *> res;
  s->exec.run(outs, &res, feeds);
  for (int i = 0; i < nout; i++) {
    out_tensors[i] = nullptr;
    if (!res[i]) continue;
    auto *t = new C_Tensor;
    t->t = std::move(*res[i]);
    delete res[i];
    out_tensors[i] = t;
  }
}

void C_Run(C_Session *s, const char **out_names, C_Tensor **out_tensors, int nout, const char **in_names,
           C_Tensor *const *in_tensors, int nin) {
  must("C_Run", [&] { run_impl(s, out_names, out_tensors, nout, in_names, in_tensors, nin); });
}

int C_TryRun(C_Session *s, const char **out_names, C_Tensor **out_tensors, int nout, const char **in_names,
             C_Tensor *const *in_tensors, int nin) {
  return guarded("C_Run", [&] { run_impl(s, out_names, out_tensors, nout, in_names, in_tensors, nin); }) ? 0 : -1;
}

size_t C_DumpGraph(char *buf, size_t cap) {
  std::string d = cavs::mid::global_graph().dump();
  if (buf && cap) {
    size_t n = std::min(cap - 1, d.size());
    std::memcpy(buf, d.data(), n);
    buf[n] = 0;
  }
  return d.size() + 1;
}

size_t C_DumpFusedGraph(char *buf, size_t cap) {
  std::string d = cavs::mid::dump_fused(cavs::mid::global_graph());
  if (buf && cap) {
    size_t n = std::min(cap - 1, d.size());
    std::memcpy(buf, d.data(), n);
    buf[n] = 0;
  }
  return d.size() + 1;
}

size_t C_DumpCell(char *buf, size_t cap, int what) {
  std::string d;
  const int stage = what / 10;
  if (what % 10 == 0) {
    d = cavs::mid::cell_host_source(cavs::mid::global_graph(), stage);
  } else {
    std::string why;
    auto m = cavs::mid::match_cell(cavs::mid::global_graph(), &why);
    std::shared_ptr<cavs::CellSpec> spec = m ? m->spec : nullptr;
    for (int i = 0; i < stage && spec; i++) spec = spec->next;
    d = spec ? spec->source : m ? std::string("// no such stage\n") : "// not a cell: " + why + "\n";
  }
  if (buf && cap) {
    size_t n = std::min(cap - 1, d.size());
    std::memcpy(buf, d.data(), n);
    buf[n] = 0;
  }
  return d.size() + 1;
}

void C_ResetGraph(void) { cavs::mid::reset_global_graph(); }

int C_SetVariable(C_Session *s, const char *name, const float *data, size_t n) {
  return guarded("C_SetVariable", [&] { s->exec.set_variable(name, data, n); }) ? 0 : -1;
}

long C_ReadTensor(C_Session *s, const char *name, float *out, size_t cap) {
  long r = 0;
  if (!guarded("C_ReadTensor", [&] { r = s->exec.read_tensor(name, out, cap); })) return 0;
  return r;
}

int C_SessionUsesFusedPath(C_Session *s) { return s->exec.fused_path_kind(); }
int C_SessionGeneratedKernels(C_Session *s) { return s->exec.fused_kernel_count(); }
void C_SessionAllowFusedPath(C_Session *s, int allow) { s->exec.set_lowering_mode(allow < 0 ? 0 : allow > 3 ? 3 : allow); }
void C_SessionSetPairing(C_Session *s, int pairing) { s->exec.set_pairing(pairing); }

}  // extern "C"
