#include "fusion.h"

#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <map>
#include <numeric>
#include <sstream>

#include "cavs/util/op_def_builder.h"
#include "graph.h"

namespace cavs {
namespace mid {

namespace {

// parser.cc:20-52: operators the generator can express; "deserved" ones pay for a fusion
// (aliases and plain copies do not)
bool fusable(const std::string &op) {
  static const std::set<std::string> k = {"Add", "Sub", "Mul", "Tanh", "Sigmoid", "Relu", "Mirror", "Assign",
                                          "Accumulate", "Neg", "Tanh_grad", "Sigmoid_grad", "Relu_grad"};
  return k.count(op) != 0;
}
bool deserved(const std::string &op) { return fusable(op) && op != "Mirror" && op != "Assign"; }

// operands the generated expression reads (the *_grad operators carry a third, unused one)
int arity(const std::string &op) {
  if (op == "Add" || op == "Sub" || op == "Mul" || op == "Tanh_grad" || op == "Sigmoid_grad" || op == "Relu_grad") return 2;
  return 1;
}

bool accumulates(const OpDef &d, int i) {
  auto *a = d.find_attr("Acc");
  return a && i < (int)a->value_.list_i.size() && a->value_.list_i[i] != 0;
}

// a float constant that reads back to the same value
std::string literal(float v) {
  char buf[48];
  std::snprintf(buf, sizeof buf, "%.9g", (double)v);
  std::string s(buf);
  if (s.find_first_of(".en") == std::string::npos) s += ".0";  // "n": inf/nan stay as they are
  return s + "f";
}

// expression.h:40-120: one C expression per operator
std::string expression(const OpDef &d, const std::vector<std::string> &in) {
  const std::string &op = d.name();
  std::ostringstream o;
  if (op == "Add") o << in[0] << " + " << in[1];
  else if (op == "Sub") o << in[0] << " - " << in[1];
  else if (op == "Mul") {
    o << in[0] << " * " << in[1];
    float s = GetSingleArg<float>(d, "Scale", 1.f);
    if (s != 1.f) o << " * " << literal(s);
  } else if (op == "Tanh") o << "tanhf(" << in[0] << ")";
  else if (op == "Sigmoid") o << "1.f / (1.f + expf(-" << in[0] << "))";
  else if (op == "Relu") o << "(" << in[0] << " > 0.f ? " << in[0] << " : 0.f)";
  else if (op == "Mirror" || op == "Assign" || op == "Accumulate") o << in[0];
  else if (op == "Neg") o << "-" << in[0];
  else if (op == "Tanh_grad") o << in[0] << " * (1.f - " << in[1] << " * " << in[1] << ")";
  else if (op == "Sigmoid_grad") o << in[0] << " * (" << in[1] << " * (1.f - " << in[1] << "))";
  else if (op == "Relu_grad") o << "(" << in[1] << " > 0.f ? " << in[0] << " : 0.f)";
  return o.str();
}

struct UnionFind {
  std::vector<int> p;
  explicit UnionFind(int n) : p(n) { std::iota(p.begin(), p.end(), 0); }
  int find(int x) { return p[x] == x ? x : p[x] = find(p[x]); }
  void unite(int a, int b) { p[find(a)] = find(b); }
};

}  // namespace

std::vector<OpDef> fuse_program(const std::vector<OpDef> &prog, const FusionEnv &env, int *groups_made) {
  const int n = (int)prog.size();
  static int kernel_id = 0;
  // The class of an op is the geometry of the element range it runs over, (per-row?, width)
  // encoded as +-width; 0 means "cannot be fused".  Operands have the same class or are static
  // rows that divide it.  The output normally covers the whole range.  A *reducing* op is one
  // whose operands are per-row slabs while its output is a static row whose width divides
  // theirs (the gradient of an operand that was broadcast over the rows: a bias): it runs over
  // its operands' range and every element is added onto out[idx % out_count] -- the
  // generator's atomicAdd form for outputs narrower than n_elements
  // (cavs/midend/runtime_compiler/code_generator.cc:84-100).
  std::vector<char> reducing(n, 0);
  auto full_count = [&](const OpDef &d, char *reduces) -> long {
    *reduces = 0;
    if (d.output_size() != 1 || d.input_size() < arity(d.name())) return 0;
    bool rows = env.per_row(d.output(0));
    long w = env.width(d.output(0));
    if (w <= 0) return 0;
    if (!rows) {
      long win = 0;
      for (int k = 0; k < arity(d.name()); k++)
        if (env.per_row(d.input(k))) win = std::max(win, env.width(d.input(k)));
      if (win > 0) {  // per-row operands, static output
        if (win % w != 0) return 0;
        *reduces = 1;
        rows = true;
        w = win;
      }
    }
    for (int k = 0; k < arity(d.name()); k++) {
      const std::string &i = d.input(k);
      long wi = env.width(i);
      if (wi <= 0) return 0;
      if (env.per_row(i)) {
        if (!rows || wi != w) return 0;
      } else if (w % wi != 0) {
        return 0;
      }
    }
    return rows ? w : -w;
  };
  std::vector<long> width(n, 0);
  std::map<std::string, int> producer;  // last writer of an edge within the program
  std::vector<std::vector<int>> readers_of(n);
  for (int i = 0; i < n; i++) {
    if (fusable(prog[i].name())) width[i] = full_count(prog[i], &reducing[i]);
    for (auto &o : prog[i].output()) producer[o] = i;
  }
  UnionFind uf(n);
  {
    std::map<std::string, int> last;  // producer seen so far, in program order
    for (int i = 0; i < n; i++) {
      for (int k = 0; k < prog[i].input_size() && (width[i] == 0 || k < arity(prog[i].name())); k++) {
        const std::string &in = prog[i].input(k);
        auto it = last.find(in);
        if (it == last.end()) continue;
        int p = it->second;
        // (what a reducing op produces is complete only when its kernel has finished: nobody
        // joins a group through it)
        if (width[i] != 0 && width[i] == width[p] && !reducing[p]) uf.unite(i, p);
      }
      for (auto &o : prog[i].output()) last[o] = i;
    }
  }
  std::map<int, std::vector<int>> groups;
  for (int i = 0; i < n; i++)
    if (width[i] != 0) groups[uf.find(i)].push_back(i);

  std::vector<int> group_of(n, -1);
  std::map<int, OpDef> fused_at;  // position of the last member -> FusedKernel
  int made = 0;
  // The kernel runs where the group's last member stood.  An outsider in between must not read
  // or write what the members above it produce, nor overwrite what they read: the group is cut
  // at the first outsider that does, and both halves are examined again.
  auto violation = [&](const std::vector<int> &m) -> int {
    std::set<int> in(m.begin(), m.end());
    std::set<std::string> produced, read_so_far;
    for (int j = m.front(); j < m.back(); j++) {
      if (in.count(j)) {
        for (int k = 0; k < arity(prog[j].name()); k++) read_so_far.insert(prog[j].input(k));
        for (auto &o : prog[j].output()) produced.insert(o);
        continue;
      }
      for (auto &x : prog[j].input())
        if (produced.count(x)) return j;
      for (auto &x : prog[j].output())
        if (produced.count(x) || read_so_far.count(x)) return j;
    }
    // an outsider above a later member may also write an edge that member accumulates onto: fine
    return -1;
  };
  std::vector<std::vector<int>> work;
  for (auto &kv : groups) work.push_back(kv.second);
  while (!work.empty()) {
    std::vector<int> members = work.back();
    work.pop_back();
    if (members.size() < 2) continue;
    int cut = violation(members);
    if (cut >= 0) {
      std::vector<int> above, below;
      for (int i : members) (i < cut ? above : below).push_back(i);
      work.push_back(above);
      work.push_back(below);
      continue;
    }
    {
      // a member must not read what a reducing member of the same group adds up
      std::set<std::string> reduced;
      int offender = -1;
      for (int i : members) {
        for (int k = 0; k < arity(prog[i].name()) && offender < 0; k++)
          if (reduced.count(prog[i].input(k))) offender = i;
        if (reducing[i]) reduced.insert(prog[i].output(0));
      }
      if (offender >= 0) {
        std::vector<int> above, below;
        for (int i : members) (i < offender ? above : below).push_back(i);
        work.push_back(above);
        work.push_back(below);
        continue;
      }
    }
    int benefit = 0;
    for (int i : members) benefit += deserved(prog[i].name()) || reducing[i];
    if (members.size() < 2 || benefit <= 1) continue;  // parser.cc:118-131: kept iff benefit > 1

    std::set<int> in(members.begin(), members.end());
    const long cls = width[members[0]];
    std::set<std::string> written;
    std::vector<std::string> inputs, outputs, stateful, zero_first;
    std::set<std::string> seen_in, reduced_out;
    std::ostringstream body;
    bool clash = false;
    for (int i : members) {
      const OpDef &d = prog[i];
      std::vector<std::string> args;
      for (int k = 0; k < arity(d.name()); k++) {
        const std::string &x = d.input(k);
        if (!written.count(x) && seen_in.insert(x).second) inputs.push_back(x);
        args.push_back("tmp_" + x);
      }
      const std::string &o = d.output(0);
      bool acc = accumulates(d, 0);
      if (reducing[i]) {
        // tmp_o holds this element's contribution only; the store adds it onto out[idx % count].
        // An output the group is the first writer of must be zero when the kernel first runs.
        if (written.count(o) && !reduced_out.count(o)) { clash = true; break; }
        if (seen_in.count(o)) { clash = true; break; }
        std::string e = expression(d, args);
        if (reduced_out.count(o)) body << "    tmp_" << o << " = tmp_" << o << " + (" << e << ");\n";
        else body << "    float tmp_" << o << " = " << e << ";\n";
        if (!acc && !reduced_out.count(o)) zero_first.push_back(o);
        reduced_out.insert(o);
        written.insert(o);
        continue;
      }
      if (reduced_out.count(o)) { clash = true; break; }
      if (acc && !written.count(o)) {  // accumulates onto a value produced outside the group
        if (seen_in.count(o)) { clash = true; break; }  // read as an operand and updated in place
        stateful.push_back(o);
      }
      std::string e = expression(d, args);
      if (written.count(o)) {
        body << "    tmp_" << o << " = " << (acc ? "tmp_" + o + " + (" + e + ")" : e) << ";\n";
      } else if (acc) {
        body << "    float tmp_" << o << " = " << o << "[idx] + (" << e << ");\n";
      } else {
        body << "    float tmp_" << o << " = " << e << ";\n";
      }
      written.insert(o);
    }
    if (clash) continue;
    // outputs: member results that anything outside the group reads, and results nobody
    // in the group consumes (they are somebody's final value)
    for (auto &o : written) {
      bool needed = env.live.count(o) != 0 || std::find(stateful.begin(), stateful.end(), o) != stateful.end();
      bool used_inside = false;
      for (int j = 0; j < n; j++) {
        const int lim = in.count(j) ? arity(prog[j].name()) : prog[j].input_size();
        for (int k = 0; k < lim; k++)
          if (prog[j].input(k) == o) (in.count(j) ? used_inside : needed) = true;
      }
      if (needed || !used_inside) outputs.push_back(o);
    }
    if (outputs.empty()) continue;
    std::string name = "FusedKernel_" + std::to_string(kernel_id++);
    std::ostringstream src;
    src << "extern \"C\" __global__ void " << name << "(";
    for (auto &o : outputs) src << "float *" << o << ", ";
    for (auto &x : inputs) src << "const float *" << x << ", ";
    for (auto &o : outputs) src << "const int " << o << "_count, ";
    for (auto &x : inputs) src << "const int " << x << "_count, ";
    src << "const int n_elements)\n{\n  const int idx = blockIdx.x * blockDim.x + threadIdx.x;\n  if (idx < n_elements) {\n";
    // operands of the group's own geometry hold n_elements values; only broadcast rows wrap
    auto index = [&](const std::string &x) {
      const bool same = env.per_row(x) == (cls > 0) && env.width(x) == std::labs(cls);
      return same ? std::string("[idx]") : "[idx % " + x + "_count]";
    };
    for (auto &x : inputs) src << "    float tmp_" << x << " = " << x << index(x) << ";\n";
    src << body.str();
    for (auto &o : outputs) {
      if (reduced_out.count(o)) src << "    atomicAdd(&" << o << "[idx % " << o << "_count], tmp_" << o << ");\n";
      else src << "    " << o << "[idx] = tmp_" << o << ";\n";
    }
    src << "  }\n}\n";
    // Stateful: outputs the kernel accumulates onto a value written before it; Reduced: outputs
    // narrower than the element range, added to with atomicAdd; ZeroEnforced: those of them the
    // kernel is the first writer of, which must hold zero before its first launch of an iteration
    // (code_generator.cc:155-164; the reference zeroes such buffers once per iteration,
    // cavs/midend/tensor.cc:283-300)
    OpDefBuilder b("FusedKernel");
    b.Input(inputs).Output(outputs).AttrSingle("KernelName", name).AttrSingle("KernelSource", src.str())
        .AttrList("Stateful", stateful).AttrList("Reduced", std::vector<std::string>(reduced_out.begin(), reduced_out.end()))
        .AttrList("ZeroEnforced", zero_first);
    fused_at[members.back()] = b.Finalize();
    for (int i : members) group_of[i] = members.back();
    made++;
  }
  std::vector<OpDef> out;
  for (int i = 0; i < n; i++) {
    if (group_of[i] < 0) out.push_back(prog[i]);
    else if (group_of[i] == i) out.push_back(fused_at[i]);
  }
  if (groups_made) *groups_made = made;
  return out;
}

BackwardFusion fuse_function_backward(const std::vector<OpDef> &per_round, const std::vector<OpDef> &deferred, FusionEnv env) {
  BackwardFusion out;
  std::vector<OpDef> offered = per_round;
  std::map<std::string, int> writers;
  for (auto &d : deferred)
    for (auto &o : d.output()) writers[o]++;
  std::vector<char> moved(deferred.size(), 0);
  for (size_t i = 0; i < deferred.size(); i++) {
    const OpDef &d = deferred[i];
    if (d.name() != "Assign" && d.name() != "Accumulate" && d.name() != "Neg") continue;
    if (d.output_size() != 1 || d.input_size() < 1 || accumulates(d, 0) || writers[d.output(0)] != 1) continue;
    if (env.per_row(d.output(0)) || !env.per_row(d.input(0))) continue;
    // right behind the op that produces its operand, so that nothing between them reads what the
    // group they may form produces
    int at = -1;
    for (size_t j = 0; j < offered.size(); j++)
      for (auto &o : offered[j].output())
        if (o == d.input(0)) at = (int)j;
    if (at < 0) continue;  // the operand does not come out of the per-round program
    moved[i] = 1;
    offered.insert(offered.begin() + at + 1, d);
  }
  for (size_t i = 0; i < deferred.size(); i++)
    if (!moved[i])
      for (int k = 0; k < operands_read(deferred[i]); k++) env.live.insert(deferred[i].input(k));
  std::vector<OpDef> fused = fuse_program(offered, env, &out.groups);
  std::set<std::string> came_back;  // offered ops the pass left as they were
  for (auto &d : fused) {
    bool was_deferred = false;
    for (size_t i = 0; i < deferred.size(); i++)
      if (moved[i] && d.name() == deferred[i].name() && d.output_size() == 1 && d.output(0) == deferred[i].output(0)) was_deferred = true;
    if (was_deferred) {
      came_back.insert(d.output(0));
    } else {
      out.per_round.push_back(d);
      if (d.name() == "FusedKernel")
        for (auto &z : GetListArgS(d, "ZeroEnforced")) out.zero_before_loop.push_back(z);
    }
  }
  for (size_t i = 0; i < deferred.size(); i++)
    if (!moved[i] || came_back.count(deferred[i].output(0))) out.deferred.push_back(deferred[i]);
  return out;
}

int operands_read(const OpDef &d) {
  return fusable(d.name()) ? std::min(arity(d.name()), d.input_size()) : d.input_size();
}

static const Edge *lookup(const Graph &g, const std::string &name) {
  const Edge *e = g.func ? g.func->find(name) : g.main.find(name);
  if (!e && IsGradientName(name)) e = lookup(g, GetOriginName(name));  // a gradient has its origin's geometry
  return e;
}

FusionEnv graph_env(const Graph &g) {
  FusionEnv env;
  const Graph *gp = &g;
  env.per_row = [gp](const std::string &n) { const Edge *e = lookup(*gp, n); return e && e->per_vertex(); };
  env.width = [gp](const std::string &n) -> long { const Edge *e = lookup(*gp, n); return e ? e->width() : 0; };
  return env;
}

std::string dump_fused(const Graph &g) {
  std::vector<OpDef> fwd, main_all;
  if (g.func)
    for (auto &n : g.func->nodes) fwd.push_back(n->def);
  for (auto &n : g.main.nodes) main_all.push_back(n->def);
  auto live_of = [&](const std::vector<const std::vector<OpDef> *> &others) {
    FusionEnv env = graph_env(g);
    for (auto *o : others)
      for (auto &d : *o)
        for (int k = 0; k < operands_read(d); k++) env.live.insert(d.input(k));
    for (auto &v : g.opt.vars) env.live.insert(GetGradientName(v));
    return env;
  };
  std::ostringstream o;
  auto emit = [&](const char *title, const std::vector<OpDef> &prog) {
    o << title << ":\n";
    for (auto &d : prog) {
      if (d.name() == "FusedKernel") {
        o << "  FusedKernel(";
        for (auto &x : d.input()) o << x << ",";
        o << ") -> (";
        for (auto &x : d.output()) o << x << ",";
        o << ")\n" << GetSingleArg<std::string>(d, "KernelSource", "");
      } else {
        o << "  " << d.DebugString() << "\n";
      }
    }
  };
  emit("main", fuse_program(main_all, live_of({&fwd, &g.func_backward, &g.func_deferred, &g.opt.backward})));
  if (g.func) {
    emit("function", fuse_program(fwd, live_of({&g.func_backward, &g.func_deferred, &main_all, &g.opt.backward})));
    BackwardFusion bf = fuse_function_backward(g.func_backward, g.func_deferred, live_of({&fwd, &main_all, &g.opt.backward}));
    emit("function_grad", bf.per_round);
    emit("function_grad_deferred", bf.deferred);
  }
  if (g.opt.present) emit("backward", fuse_program(g.opt.backward, live_of({&fwd, &g.func_backward, &g.func_deferred})));
  return o.str();
}

}  // namespace mid
}  // namespace cavs
