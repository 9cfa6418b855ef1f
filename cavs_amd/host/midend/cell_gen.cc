#include "cell_gen.h"

#include <algorithm>
#include <cstdio>
#include <cstring>
#include <functional>
#include <set>
#include <sstream>
#include <tuple>

#include "cavs/util/op_def_builder.h"

namespace cavs {
namespace mid {

namespace {

const char kTemplate[] =
#include "cell_template.inc"
    ;

// ---------------------------------------------------------------- the elementwise part as a DAG
// One node per value of one hidden unit of one vertex.  Nodes are created in evaluation order, so an
// operand's id is below its user's; equal nodes are shared.
enum Kind {
  N_XW, N_HU, N_BIAS, N_CS, N_XD,  // inputs of the forward part (i0, i1 index them)
  N_DST, N_DRET, N_ZERO,           // seeds of the backward part, and "no gradient"
  N_ADD, N_SUB, N_MUL, N_NEG, N_SIGM, N_TANH, N_RELU,
  N_DSIGM, N_DTANH, N_DRELU        // a = gradient, b = the activation's output
};

struct ENode {
  int kind, a, b, i0, i1;
  float scale;
};

struct Dag {
  std::vector<ENode> n;
  std::map<std::tuple<int, int, int, int, int, uint32_t>, int> memo;
  int make(int kind, int a = -1, int b = -1, int i0 = 0, int i1 = 0, float scale = 1.f) {
    uint32_t bits;
    std::memcpy(&bits, &scale, 4);
    auto key = std::make_tuple(kind, a, b, i0, i1, bits);
    auto it = memo.find(key);
    if (it != memo.end()) return it->second;
    n.push_back({kind, a, b, i0, i1, scale});
    return memo[key] = (int)n.size() - 1;
  }
};

std::string literal(float v) {
  char buf[48];
  std::snprintf(buf, sizeof buf, "%.9g", (double)v);
  std::string s(buf);
  if (s.find_first_of(".en") == std::string::npos) s += ".0";
  return s + "f";
}

bool alias_op(const std::string &op) { return op == "Mirror" || op == "Reshape" || op == "Flatten" || op == "Expand_dims"; }

struct Fail {
  std::string why;
};
[[noreturn]] void no(const std::string &why) { throw Fail{why}; }

// One cell: its description, its elementwise part, the nodes of its state blocks and of the value it pushes.
struct Body {
  CellSpec spec;
  Dag dag;
  std::vector<int> st;
  int ret = -1;
};

// ---------------------------------------------------------------- reading F
// A product as read: the nodes of its left operand's blocks, whatever they are.
struct RawTerm {
  int node;
  long brow;
};
struct RawProduct {
  std::vector<RawTerm> terms;
  CellParamRef B;
  int ldb = 0;
  long col = 0;
};

struct Reader : Body {
  const Graph &g;
  const Scope *func;
  std::map<const Edge *, std::vector<int>> val;  // H-wide blocks of a func-scope edge, as nodes
  std::set<const Edge *> raw_x, emb_x;           // the pulled id; its embedding row
  std::vector<RawProduct> raw;                   // by the index of their N_HU node
  std::map<std::string, int> param_of;           // Variable -> index in spec.params
  std::map<std::string, std::string> roles;
  std::map<std::string, CellSlot> slots;
  std::map<std::pair<int, long>, int> bias_of;   // (param, offset) -> index in spec.biases
  std::map<std::pair<int, int>, int> asrc_of;    // (mask, block) -> index in spec.asrc
  bool have_xw = false;

  explicit Reader(const Graph &graph) : g(graph), func(graph.func.get()) {}
  std::map<std::pair<int, long>, int> &biases_seen() { return bias_of; }

  int param_index(const Resolved &r, bool embedding) {
    auto it = param_of.find(r.var);
    if (it != param_of.end()) return it->second;
    const Edge *ve = g.main.find(r.var);
    if (!ve) no("no Variable edge " + r.var);
    CellParam p;
    p.name = embedding ? "Emb" : "P" + std::to_string(spec.params.size());
    p.size = ve->width();
    spec.params.push_back(p);
    if ((int)spec.params.size() > CA_MAX_PARAMS) no("more than " + std::to_string(CA_MAX_PARAMS) + " Variables");
    return param_of[r.var] = (int)spec.params.size() - 1;
  }

  // an operand that comes from the main scope: a view of a Variable, registered as a role
  CellParamRef external(const Edge *e, long *count, bool embedding = false) {
    Resolved r = resolve_external(e);
    if (!r.ok) no("external input " + e->name + " is not a view of a Variable");
    CellParamRef ref;
    ref.param = param_index(r, embedding);
    ref.offset = r.offset;
    *count = r.count;
    // the edge F consumes directly (the one the backward function returns a gradient for)
    const Edge *direct = e;
    while (direct->scope == func && direct->src && alias_op(direct->src->def.name())) direct = direct->src->in[0];
    if (direct->scope == func) no("external input " + e->name + " is reshaped inside F in a way that is not a plain alias");
    const std::string key = r.var + "@" + std::to_string(r.offset) + "+" + std::to_string(r.count);
    auto it = roles.find(key);
    if (it != roles.end() && it->second != direct->name) no("two main-scope edges view the same part of " + r.var);
    roles[key] = direct->name;
    slots[key] = {spec.params[ref.param].name, r.offset, r.count};
    return ref;
  }

  bool is_external(const Edge *e) const {
    while (e->scope == func && e->src && alias_op(e->src->def.name())) e = e->src->in[0];
    return e->scope != func;
  }

  const std::vector<int> &blocks(const Edge *e) {
    auto it = val.find(e);
    if (it != val.end()) return it->second;
    if (!is_external(e)) no("operand " + e->name + " is not made of H-wide blocks");
    long count;
    CellParamRef ref = external(e, &count);
    const int H = spec.H;
    if (count % H) no("external operand " + e->name + " is not a multiple of H wide");
    std::vector<int> b;
    for (long i = 0; i < count / H; i++) {
      auto key = std::make_pair(ref.param, ref.offset + i * H);
      if (!bias_of.count(key)) {
        bias_of[key] = (int)spec.biases.size();
        CellBias cb;
        cb.ref.param = ref.param;
        cb.ref.offset = ref.offset + i * H;
        spec.biases.push_back(cb);
      }
      b.push_back(dag.make(N_BIAS, -1, -1, bias_of[key]));
    }
    return val[e] = b;
  }

  // whether a node is a plain sum of one state block of distinct children (what the first stage's
  // products take as their left operand straight from the message pool)
  bool child_sum(int node, int *mask_out, int *block_out) const {
    int mask = 0, block = -1;
    std::vector<int> todo{node};
    while (!todo.empty()) {
      const ENode &q = dag.n[todo.back()];
      todo.pop_back();
      if (q.kind == N_ADD) {
        todo.push_back(q.a);
        todo.push_back(q.b);
      } else if (q.kind == N_CS) {
        if ((block >= 0 && block != q.i1) || (mask & (1 << q.i0))) return false;
        block = q.i1;
        mask |= 1 << q.i0;
      } else {
        return false;
      }
    }
    *mask_out = mask;
    *block_out = block;
    return true;
  }

  void read() {
    if (!func) no("no vertex function");
    CellSpec &s = spec;
    int pushes = 0, scatters = 0;
    for (auto &n : func->nodes) {
      if (n->def.name() == "Push") {
        s.H = (int)n->in[0]->width();
        pushes++;
      }
      scatters += n->def.name() == "Scatter";
    }
    if (pushes != 1 || scatters != 1) no("F must end in one Scatter and one Push");
    if (s.H <= 0 || s.H % 32) no("the pushed value's width is not a multiple of 32");
    const int H = s.H;
    for (auto &np : func->nodes) {
      const Node *n = np.get();
      const OpDef &d = n->def;
      const std::string &op = d.name();
      const Edge *out = n->out.empty() ? nullptr : n->out[0];
      if (op == "Gather") {
        const int k = GetSingleArg<int>(d, "Child", 0);
        const long w = out->width();
        if (k < 0 || k > 1 || w % H) no("Gather of child " + std::to_string(k) + " with width " + std::to_string(w));
        if (s.SI && s.SI != w / H) no("Gather widths differ");
        s.SI = (int)(w / H);
        s.K = std::max(s.K, k + 1);
        std::vector<int> b;
        for (int m = 0; m < s.SI; m++) b.push_back(dag.make(N_CS, -1, -1, k, m));
        val[out] = b;
      } else if (op == "Pull") {
        const long w = out->width();
        if (w == 1) {  // an id, to be looked up
          raw_x.insert(out);
        } else if (w % H == 0 && w / H <= 8 && !s.XD) {  // a row of the vertex input, used as it is
          s.XD = (int)(w / H);
          std::vector<int> b;
          for (int i = 0; i < s.XD; i++) b.push_back(dag.make(N_XD, -1, -1, i));
          val[out] = b;
        } else {
          no("Pull of a vertex input that is neither one id nor a few H-wide blocks");
        }
      } else if (op == "EmbeddingLookup") {
        if (!raw_x.count(n->in[0])) no("EmbeddingLookup of something other than the pulled id");
        long count;
        Resolved r = resolve_external(n->in[1]);
        const Edge *table = n->in[1];
        if (!r.ok || r.offset != 0 || table->shape.size() != 2) no("the embedding table is not a whole 2-D Variable");
        external(table, &count, true);
        s.V = table->shape[0];
        s.E = table->shape[1];
        emb_x.insert(out);
      } else if (alias_op(op)) {
        const Edge *in = n->in[0];
        if (raw_x.count(in)) raw_x.insert(out);
        else if (emb_x.count(in)) emb_x.insert(out);
        else if (val.count(in)) val[out] = val[in];
        // (an alias of an external edge is resolved where it is used)
      } else if (op == "MatMul") {
        const Edge *A = n->in[0], *B = n->in[1];
        if (!is_external(B) || B->shape.size() != 2) no("MatMul whose right operand is not a 2-D view of a Variable");
        const long rows = B->shape[0], cols = B->shape[1];
        if (cols % H) no("MatMul output width is not a multiple of H");
        long count;
        CellParamRef ref = external(B, &count);
        if (count != rows * cols) no("MatMul right operand view has the wrong size");
        std::vector<int> b;
        if (emb_x.count(A)) {
          if (have_xw) no("more than one product with the vertex input");
          if (rows != s.E) no("x * W: W has " + std::to_string(rows) + " rows, the embedding " + std::to_string(s.E));
          have_xw = true;
          s.W = ref;
          s.NX = (int)(cols / H);
          for (int i = 0; i < s.NX; i++) b.push_back(dag.make(N_XW, -1, -1, i));
        } else {
          const std::vector<int> ab = blocks(A);
          if ((long)ab.size() * H != rows) no("MatMul operand widths do not agree");
          for (long o = 0; o < cols / H; o++) {
            RawProduct p;
            for (size_t a = 0; a < ab.size(); a++) p.terms.push_back({ab[a], (long)a * H});
            p.B = ref;
            p.ldb = (int)cols;
            p.col = o * H;
            raw.push_back(p);
            b.push_back(dag.make(N_HU, -1, -1, (int)raw.size() - 1));
          }
        }
        val[out] = b;
      } else if (op == "Slice") {
        const std::vector<int> &in = blocks(n->in[0]);
        const long w = (long)in.size() * H;
        const long stride = d.find_attr("Split") ? w / GetSingleArg<int>(d, "Split") : GetSingleArg<int>(d, "Stride");
        const long off = d.find_attr("Split") ? stride * GetSingleArg<int>(d, "Index") : GetSingleArg<int>(d, "Offset");
        if (off % H || stride % H || off + stride > w) no("Slice that does not cut at multiples of H");
        val[out] = std::vector<int>(in.begin() + off / H, in.begin() + (off + stride) / H);
      } else if (op == "Concat") {
        std::vector<int> b;
        for (const Edge *e : n->in) {
          const std::vector<int> &in = blocks(e);
          b.insert(b.end(), in.begin(), in.end());
        }
        val[out] = b;
      } else if (op == "Add" || op == "Sub" || op == "Mul") {
        const std::vector<int> x = blocks(n->in[0]), y = blocks(n->in[1]);
        if (x.size() != y.size()) no(op + " of operands of different widths");
        const int kind = op == "Add" ? N_ADD : op == "Sub" ? N_SUB : N_MUL;
        const float scale = op == "Mul" ? GetSingleArg<float>(d, "Scale", 1.f) : 1.f;
        std::vector<int> b;
        for (size_t i = 0; i < x.size(); i++) b.push_back(dag.make(kind, x[i], y[i], 0, 0, scale));
        val[out] = b;
      } else if (op == "Sigmoid" || op == "Tanh" || op == "Relu" || op == "Neg") {
        const std::vector<int> x = blocks(n->in[0]);
        const int kind = op == "Sigmoid" ? N_SIGM : op == "Tanh" ? N_TANH : op == "Relu" ? N_RELU : N_NEG;
        std::vector<int> b;
        for (int v : x) b.push_back(dag.make(kind, v));
        val[out] = b;
      } else if (op == "Scatter") {
        st = blocks(n->in[0]);
        s.S = (int)st.size();
        if (s.SI && s.S != s.SI) no("the scattered message is not as wide as the gathered ones");
      } else if (op == "Push") {
        const std::vector<int> &b = blocks(n->in[0]);
        if (b.size() != 1) no("the pushed value is not H wide");
        ret = b[0];
      } else {
        no("operator " + op + " inside F");
      }
    }
    if (st.empty() || ret < 0) no("F has no Scatter or no Push");
    if (s.K < 1) no("F gathers no child");
    if (!raw_x.empty() && !have_xw) no("the vertex input's id is pulled but not looked up and multiplied");
    if (raw.empty()) no("F multiplies no child state");
    if (raw.size() > 32 || s.NX > 16 || s.biases.size() > 32) no("too many products or operands");
  }
};

// ---------------------------------------------------------------- the backward part
struct Derived {
  std::vector<int> dcols;                 // node of every block of a vertex's gradient row
  std::vector<std::vector<int>> dcs;      // [k][m]: node of the elementwise gradient into child k's block m, or -1
  std::vector<int> saved;                 // forward nodes the backward part reads, in sv order
  bool reads_cs = false;
  int ds_mask = 0;
};

Derived derive(Body &r) {
  Dag &dag = r.dag;
  CellSpec &s = r.spec;
  const int nfwd = (int)dag.n.size();
  std::vector<std::vector<int>> adj(nfwd);
  for (int m = 0; m < s.S; m++) adj[r.st[m]].push_back(dag.make(N_DST, -1, -1, m));
  if (r.ret >= 0) adj[r.ret].push_back(dag.make(N_DRET));
  std::vector<int> grad(nfwd, -1);
  for (int id = nfwd - 1; id >= 0; id--) {
    if (adj[id].empty()) continue;
    int gsum = adj[id][0];
    for (size_t i = 1; i < adj[id].size(); i++) gsum = dag.make(N_ADD, gsum, adj[id][i]);
    grad[id] = gsum;
    const ENode q = dag.n[id];
    switch (q.kind) {
      case N_ADD: adj[q.a].push_back(gsum); adj[q.b].push_back(gsum); break;
      case N_SUB: adj[q.a].push_back(gsum); adj[q.b].push_back(dag.make(N_NEG, gsum)); break;
      case N_MUL:
        adj[q.a].push_back(dag.make(N_MUL, gsum, q.b, 0, 0, q.scale));
        adj[q.b].push_back(dag.make(N_MUL, gsum, q.a, 0, 0, q.scale));
        break;
      case N_NEG: adj[q.a].push_back(dag.make(N_NEG, gsum)); break;
      case N_SIGM: adj[q.a].push_back(dag.make(N_DSIGM, gsum, id)); break;
      case N_TANH: adj[q.a].push_back(dag.make(N_DTANH, gsum, id)); break;
      case N_RELU: adj[q.a].push_back(dag.make(N_DRELU, gsum, id)); break;
      default: break;  // inputs
    }
  }
  Derived d;
  const int zero = dag.make(N_ZERO);
  auto input_grad = [&](int kind, int i0, int i1) {
    for (int id = 0; id < nfwd; id++)
      if (dag.n[id].kind == kind && dag.n[id].i0 == i0 && dag.n[id].i1 == i1) return grad[id];
    return -1;
  };
  auto column_of = [&](int node) {
    if (node < 0) node = zero;
    return node;
  };
  // the blocks of d(x * W) first and in order: the weight gradient of W is one product over them
  for (int i = 0; i < s.NX; i++) d.dcols.push_back(column_of(input_grad(N_XW, i, 0)));
  auto shared_column = [&](int node) {
    node = column_of(node);
    for (size_t q = 0; q < d.dcols.size(); q++)
      if (d.dcols[q] == node) return (int)q;
    d.dcols.push_back(node);
    return (int)d.dcols.size() - 1;
  };
  for (size_t p = 0; p < s.products.size(); p++) s.products[p].dcol = shared_column(input_grad(N_HU, (int)p, 0));
  for (size_t i = 0; i < s.biases.size(); i++) s.biases[i].dcol = shared_column(input_grad(N_BIAS, (int)i, 0));
  s.ND = (int)d.dcols.size();
  d.dcs.assign(s.K, std::vector<int>(s.SI, -1));
  for (int k = 0; k < s.K; k++)
    for (int m = 0; m < s.SI; m++) {
      d.dcs[k][m] = input_grad(N_CS, k, m);
      if (d.dcs[k][m] >= 0) d.ds_mask |= 1 << m;
    }
  // forward values the backward part reads: children's states come from the pool, the rest is saved
  std::set<int> seen;
  std::vector<int> todo = d.dcols;
  for (auto &row : d.dcs)
    for (int v : row)
      if (v >= 0) todo.push_back(v);
  std::set<int> saved;
  while (!todo.empty()) {
    const int id = todo.back();
    todo.pop_back();
    if (!seen.insert(id).second) continue;
    const ENode &q = dag.n[id];
    if (id < nfwd) {
      if (q.kind == N_CS) d.reads_cs = true;
      else saved.insert(id);
      continue;
    }
    if (q.a >= 0) todo.push_back(q.a);
    if (q.b >= 0) todo.push_back(q.b);
  }
  d.saved.assign(saved.begin(), saved.end());
  s.NSV = (int)d.saved.size();
  return d;
}

// ---------------------------------------------------------------- writing the source
struct Writer {
  const Body &r;
  const Derived &dv;
  const Dag &dag;
  const CellSpec &s;
  bool device;
  std::ostringstream o;

  Writer(const Body &rd, const Derived &d, bool dev) : r(rd), dv(d), dag(rd.dag), s(rd.spec), device(dev) {}

  std::string name(int id, bool backward, int nfwd) const {
    const ENode &q = dag.n[id];
    switch (q.kind) {
      case N_XW: if (!backward) return "in.xw[" + std::to_string(q.i0) + "]"; break;
      case N_HU: if (!backward) return "in.hu[" + std::to_string(q.i0) + "]"; break;
      case N_BIAS: if (!backward) return "in.bias[" + std::to_string(q.i0) + "]"; break;
      case N_XD: if (!backward) return "in.xd[" + std::to_string(q.i0) + "]"; break;
      case N_CS: return "in.cs[" + std::to_string(q.i0) + "][" + std::to_string(q.i1) + "]";
      case N_DST: return "in.dst[" + std::to_string(q.i0) + "]";
      case N_DRET: return "in.dret";
      case N_ZERO: return "0.f";
      default: break;
    }
    if (backward && id < nfwd) {
      auto it = std::find(dv.saved.begin(), dv.saved.end(), id);
      return "in.sv[" + std::to_string(it - dv.saved.begin()) + "]";
    }
    return "v" + std::to_string(id);
  }

  std::string expr(int id, bool backward, int nfwd) const {
    const ENode &q = dag.n[id];
    auto A = [&] { return name(q.a, backward, nfwd); };
    auto B = [&] { return name(q.b, backward, nfwd); };
    switch (q.kind) {
      case N_ADD: return A() + " + " + B();
      case N_SUB: return A() + " - " + B();
      case N_MUL: return A() + " * " + B() + (q.scale != 1.f ? " * " + literal(q.scale) : "");
      case N_NEG: return "-" + A();
      case N_SIGM: return "cell_sigm(" + A() + ")";
      case N_TANH: return "cell_tanh(" + A() + ")";
      case N_RELU: return "(" + A() + " > 0.f ? " + A() + " : 0.f)";
      case N_DSIGM: return A() + " * (" + B() + " * (1.f - " + B() + "))";
      case N_DTANH: return A() + " * (1.f - " + B() + " * " + B() + ")";
      case N_DRELU: return "(" + B() + " > 0.f ? " + A() + " : 0.f)";
      default: return name(id, backward, nfwd);
    }
  }

  static bool computed(int kind) { return kind >= N_ADD; }

  // statements for the nodes `roots` depend on, in evaluation order
  void body(const std::vector<int> &roots, bool backward, int nfwd) {
    std::set<int> need;
    std::vector<int> todo = roots;
    while (!todo.empty()) {
      const int id = todo.back();
      todo.pop_back();
      if (id < 0 || !need.insert(id).second) continue;
      if (backward && id < nfwd) continue;
      const ENode &q = dag.n[id];
      if (q.a >= 0) todo.push_back(q.a);
      if (q.b >= 0) todo.push_back(q.b);
    }
    for (int id : need) {
      if (backward && id < nfwd) continue;
      if (!computed(dag.n[id].kind)) continue;
      o << "  const float v" << id << " = " << expr(id, backward, nfwd) << ";\n";
    }
  }

  void elementwise(int nfwd) {
    const char *dev = device ? "static __device__ inline " : "static inline ";
    o << "struct FwdIn { float xw[" << std::max(1, s.NX) << "], hu[" << s.products.size() << "], bias[" << std::max<size_t>(1, s.biases.size())
      << "], cs[" << s.K << "][" << s.SI << "], xd[" << std::max(1, s.XD) << "]; };\n";
    o << "struct FwdOut { float st[" << s.S << "], ret, sv[" << std::max(1, s.NSV) << "]; };\n";
    o << "struct BwdIn { float dst[" << s.S << "], dret, sv[" << std::max(1, s.NSV) << "], cs[" << s.K << "][" << s.SI << "]; };\n";
    o << "struct BwdOut { float d[" << s.ND << "], dcs[" << s.K << "][" << s.SI << "]; };\n";
    if (device) {
      // exp through v_exp_f32 and the reciprocal through v_rcp_f32 (1 ulp each); saturation comes out
      // right without special cases
      o << "static __device__ inline float cell_exp(float x) { return __builtin_amdgcn_exp2f(x * 1.4426950408889634f); }\n"
           "static __device__ inline float cell_sigm(float x) { return __builtin_amdgcn_rcpf(1.f + cell_exp(-x)); }\n"
           "static __device__ inline float cell_tanh(float x) { return 1.f - 2.f * __builtin_amdgcn_rcpf(1.f + cell_exp(2.f * x)); }\n";
    } else {
      o << "static inline float cell_sigm(float x) { return 1.f / (1.f + exp(-x)); }\n"
           "static inline float cell_tanh(float x) { return tanh(x); }\n";
    }
    o << dev << "void cell_forward(const FwdIn &in, FwdOut &out) {\n";
    std::vector<int> roots = r.st;
    if (r.ret >= 0) roots.push_back(r.ret);
    roots.insert(roots.end(), dv.saved.begin(), dv.saved.end());
    body(roots, false, nfwd);
    for (int m = 0; m < s.S; m++) o << "  out.st[" << m << "] = " << name(r.st[m], false, nfwd) << ";\n";
    o << "  out.ret = " << (r.ret >= 0 ? name(r.ret, false, nfwd) : std::string("0.f")) << ";\n";
    for (size_t t = 0; t < dv.saved.size(); t++) o << "  out.sv[" << t << "] = " << name(dv.saved[t], false, nfwd) << ";\n";
    o << "}\n";
    o << dev << "void cell_backward(const BwdIn &in, BwdOut &out) {\n";
    roots = dv.dcols;
    for (auto &row : dv.dcs)
      for (int v : row)
        if (v >= 0) roots.push_back(v);
    body(roots, true, nfwd);
    for (size_t q = 0; q < dv.dcols.size(); q++) o << "  out.d[" << q << "] = " << name(dv.dcols[q], true, nfwd) << ";\n";
    for (int k = 0; k < s.K; k++)
      for (int m = 0; m < s.SI; m++)
        o << "  out.dcs[" << k << "][" << m << "] = " << (dv.dcs[k][m] >= 0 ? name(dv.dcs[k][m], true, nfwd) : std::string("0.f")) << ";\n";
    o << "}\n";
  }

  std::string param_ptr(const CellParamRef &ref, bool grad = false) const {
    return "(a.p[" + std::to_string(ref.param + (grad ? CA_MAX_PARAMS : 0)) + "] + " + std::to_string(ref.offset) + "L)";
  }

  void kernels() {
    const int H = s.H, NT = s.terms(), NP = (int)s.products.size(), NA = (int)s.asrc.size();
    o << "#define CELL_H " << H << "\n#define CELL_K " << s.K << "\n#define CELL_S " << s.S << "\n#define CELL_MW " << s.S * H
      << "\n#define CELL_SI " << s.SI << "\n#define CELL_MWI " << s.SI * H << "\n#define CELL_HAS_RET " << (s.has_ret ? 1 : 0)
      << "\n#define CELL_NX " << s.NX << "\n#define CELL_XD " << s.XD << "\n#define CELL_NP " << NP << "\n#define CELL_NA " << NA << "\n#define CELL_NT " << NT
      << "\n#define CELL_ND " << s.ND << "\n#define CELL_NSV " << s.NSV << "\n#define CELL_KS " << s.waves << "\n#define CELL_DS_MASK "
      << dv.ds_mask << "\n#define CELL_BWD_CS " << (dv.reads_cs ? 1 : 0) << "\n";
    o << "typedef float f4 __attribute__((ext_vector_type(4)));\n";
    o << "struct CellArgs {\n  float *pool;\n  const int *child, *pair, *kids, *t2j, *rows;\n  const float *xw;\n"
         "  float *sv, *asrc, *go, *d, *ds, *bt, *colsum, *dpool;\n  const float *x;\n  float *pool_in, *dpool_in;\n"
         "  float *ft_sv, *ft_d, *ft_ds;\n  const float *ft_pool_in;\n  const int *ft_child, *ft_kids;\n  long off, n;\n  float *p["
      << 2 * CA_MAX_PARAMS << "];\n};\n";
    o << "static __device__ inline f4 ld4(const float *p) { return *reinterpret_cast<const f4 *>(p); }\n";
  }

  void product_loops() {
    const int H = s.H, NP = (int)s.products.size(), NA = (int)s.asrc.size();
    // biases and the saved left operands
    o << "static __device__ inline void cell_load_bias(const CellArgs &a, int j, FwdIn &in) {\n";
    for (size_t i = 0; i < s.biases.size(); i++) o << "  in.bias[" << i << "] = " << param_ptr(s.biases[i].ref) << "[j];\n";
    o << "}\n";
    o << "static __device__ inline void cell_store_asrc(float *dst, const FwdIn &in) {\n";
    for (int q = 0; q < NA; q++) {
      o << "  dst[" << (long)q * H << "] = ";
      bool first = true;
      for (int k = 0; k < s.K; k++)
        if (s.asrc[q].mask >> k & 1) {
          o << (first ? "" : " + ") << "in.cs[" << k << "][" << s.asrc[q].block << "]";
          first = false;
        }
      o << ";\n";
    }
    o << "}\n";
    o << "static __device__ inline void cell_add_products(float (&dst)[CELL_SI], const float (&s)[CELL_NA], int k) {\n";
    for (int k = 0; k < s.K; k++) {
      o << "  if (k == " << k << ") {\n";
      for (int q = 0; q < NA; q++)
        if (s.asrc[q].mask >> k & 1) o << "    dst[" << s.asrc[q].block << "] += s[" << q << "];\n";
      o << "  }\n";
    }
    o << "}\n";
    // The weight blocks the terms read, each once (a block may serve several terms).  The round
    // kernels read them from two tile-major copies that cell_pack writes before the forward rounds
    // (for k-group g of 16 k and column tile t of 16 columns, 256 floats hold B[16g + 4s + c][16t + x]
    // at [s][x][c]: a lane's four k are one 16-byte load and a wavefront's fragment one contiguous
    // kilobyte): the blocks as they are for the forward products, transposed for the backward ones.
    struct Blk {
      int param, ldb;
      long at;
    };
    std::vector<Blk> blks;
    std::vector<int> term_blk;
    for (const CellProduct &p : s.products)
      for (const CellTerm &tm : p.terms) {
        const Blk b{p.B.param, p.ldb, p.B.offset + tm.brow * p.ldb + p.col};
        size_t q = 0;
        while (q < blks.size() && !(blks[q].param == b.param && blks[q].ldb == b.ldb && blks[q].at == b.at)) q++;
        if (q == blks.size()) blks.push_back(b);
        term_blk.push_back((int)q);
      }
    const int NBK = (int)blks.size();
    o << "#define CELL_NBK " << NBK << "\n";
    o << "static __device__ inline const float *cell_block(const CellArgs &a, int q) {\n  switch (q) {\n";
    for (int q = 0; q < NBK; q++) o << "    case " << q << ": return a.p[" << blks[q].param << "] + " << blks[q].at << "L;\n";
    o << "  }\n  return nullptr;\n}\n";
    o << "static __device__ inline int cell_block_ld(int q) {\n  switch (q) {\n";
    for (int q = 0; q < NBK; q++) o << "    case " << q << ": return " << blks[q].ldb << ";\n";
    o << "  }\n  return 0;\n}\n";
    // which (child, block) rows the left operands read
    std::set<std::pair<int, int>> raw;
    for (const CellASrc &a : s.asrc)
      for (int k = 0; k < s.K; k++)
        if (a.mask >> k & 1) raw.insert({k, a.block});
    const long kstep = (long)(H / 16) * 256;  // floats between the tiles of consecutive k-groups
    o << "struct FFrag { f4 a[" << NA << "], b[" << NBK << "]; };\n";
    o << "static __device__ inline void cell_ffetch(FFrag &f, const float *const (&crow)[CELL_K], const bool (&has)[CELL_K], "
         "const float *bpk, int kk) {\n  const f4 z = {0.f, 0.f, 0.f, 0.f};\n";
    // (a missing child reads row 0 of the pool and is masked afterwards: the loads are unconditional)
    for (auto &kb : raw)
      o << "  f4 r" << kb.first << "_" << kb.second << " = ld4(crow[" << kb.first << "] + " << (long)kb.second * H << " + kk);\n"
        << "  r" << kb.first << "_" << kb.second << " = has[" << kb.first << "] ? r" << kb.first << "_" << kb.second << " : z;\n";
    for (int q = 0; q < NA; q++) {
      std::string e;
      for (int k = 0; k < s.K; k++)
        if (s.asrc[q].mask >> k & 1) {
          const std::string v = "r" + std::to_string(k) + "_" + std::to_string(s.asrc[q].block);
          e = e.empty() ? v : e + " + " + v;
        }
      o << "  f.a[" << q << "] = " << e << ";\n";
    }
    for (int q = 0; q < NBK; q++) o << "  f.b[" << q << "] = ld4(bpk + " << (long)q * H * H << "L + (long)(kk >> 4) * " << kstep << ");\n";
    o << "}\n";
    o << "static __device__ inline void cell_fmma(const FFrag &f, f4 (&acc)[CELL_NP]) {\n#pragma unroll\n  for (int c = 0; c < 4; c++) {\n";
    int t = 0;
    for (int p = 0; p < NP; p++)
      for (const CellTerm &tm : s.products[p].terms) {
        o << "    acc[" << p << "] = __builtin_amdgcn_mfma_f32_16x16x4f32(f.a[" << tm.asrc << "][c], f.b[" << term_blk[t] << "][c], acc[" << p
          << "], 0, 0, 0);\n";
        t++;
      }
    o << "  }\n}\n";
    // backward: the left operands are blocks of the rows' own gradient rows
    std::vector<int> dcols;
    for (const CellProduct &p : s.products)
      if (std::find(dcols.begin(), dcols.end(), p.dcol) == dcols.end()) dcols.push_back(p.dcol);
    o << "struct BFrag { f4 a[" << dcols.size() << "], b[" << NBK << "]; };\n";
    o << "static __device__ inline void cell_bfetch(BFrag &f, const float *drow, const float *btk, int kk) {\n";
    for (size_t q = 0; q < dcols.size(); q++) o << "  f.a[" << q << "] = ld4(drow + " << (long)dcols[q] * H << " + kk);\n";
    for (int q = 0; q < NBK; q++) o << "  f.b[" << q << "] = ld4(btk + " << (long)q * H * H << "L + (long)(kk >> 4) * " << kstep << ");\n";
    o << "}\n";
    o << "static __device__ inline void cell_bmma(const BFrag &f, f4 (&acc)[CELL_NA]) {\n#pragma unroll\n  for (int c = 0; c < 4; c++) {\n";
    t = 0;
    for (int p = 0; p < NP; p++) {
      const int ai = (int)(std::find(dcols.begin(), dcols.end(), s.products[p].dcol) - dcols.begin());
      for (const CellTerm &tm : s.products[p].terms) {
        o << "    acc[" << tm.asrc << "] = __builtin_amdgcn_mfma_f32_16x16x4f32(f.a[" << ai << "][c], f.b[" << term_blk[t] << "][c], acc[" << tm.asrc
          << "], 0, 0, 0);\n";
        t++;
      }
    }
    o << "  }\n}\n";
    // the bias gradients out of the column sums of the gradient rows
    o << "extern \"C\" __global__ void cell_bias(CellArgs a) {\n  const int j = blockIdx.x * 256 + threadIdx.x;\n  if (j >= CELL_H) return;\n";
    for (const CellBias &b : s.biases) o << "  " << param_ptr(b.ref, true) << "[j] " << (b.add ? "+=" : "=") << " a.colsum[" << (long)b.dcol * H << " + j];\n";
    o << "}\n";
  }
};

// ---------------------------------------------------------------- stages
// The stage of a value is the number of products on the longest way to it from the inputs.  A
// function whose products are all of the first stage (left operands: plain sums of the children's
// state blocks) is one cell.  Otherwise F is cut into a chain of cells, one per stage: cell s holds
// the products of stage s and the elementwise values of that stage; what later stages read of it --
// their products' left operands first of all -- becomes the blocks of a row it writes per vertex,
// which the next cell gathers as the state of its one child, the vertex itself.
struct Chain {
  Reader reader;
  std::vector<Body> cells;
  std::vector<Derived> derived;
  std::vector<int> nfwd;

  explicit Chain(const Graph &g) : reader(g) {
    reader.read();
    const Dag &full = reader.dag;
    const int n = (int)full.n.size();
    // stages
    std::vector<int> stage(n, 0);
    int L = 0;
    for (int id = 0; id < n; id++) {
      const ENode &q = full.n[id];
      if (q.kind == N_HU) {
        int st = 1;
        for (const RawTerm &t : reader.raw[q.i0].terms) {
          int mask, block;
          if (!reader.child_sum(t.node, &mask, &block)) st = std::max(st, 1 + std::max(1, stage[t.node]));
        }
        stage[id] = st;
        L = std::max(L, st);
      } else if (q.kind >= N_ADD) {
        stage[id] = std::max(q.a >= 0 ? stage[q.a] : 0, q.b >= 0 ? stage[q.b] : 0);
      }
    }
    if (L > 4) no("more than four stages of products");
    bool first_stage = false;
    for (int id = 0; id < n; id++) first_stage |= full.n[id].kind == N_HU && stage[id] == 1;
    if (!first_stage) no("no product takes a sum of the children's state blocks as its left operand");
    auto carried = [&](int id) { const int k = full.n[id].kind; return k != N_XW && k != N_BIAS && k != N_XD; };
    // what each cell writes for the later ones: T[s] = blocks of the row cell s writes (s < L), found
    // from the last cell backwards
    std::vector<std::vector<int>> T(L + 1);
    for (int sidx = L; sidx >= 2; sidx--) {
      std::vector<int> &need = T[sidx - 1];
      auto want = [&](int id) {
        if (stage[id] < sidx && carried(id) && std::find(need.begin(), need.end(), id) == need.end()) need.push_back(id);
      };
      // left operands of this stage's products first: the next cell's products read them
      for (int id = 0; id < n; id++)
        if (full.n[id].kind == N_HU && stage[id] == sidx)
          for (const RawTerm &t : reader.raw[full.n[id].i0].terms) want(t.node);
      std::vector<int> roots = sidx == L ? reader.st : T[sidx];
      if (sidx == L && reader.ret >= 0) roots.push_back(reader.ret);
      std::set<int> seen;
      while (!roots.empty()) {
        const int id = roots.back();
        roots.pop_back();
        if (!seen.insert(id).second) continue;
        if (stage[id] < sidx) {
          want(id);
          continue;
        }
        const ENode &q = full.n[id];
        if (q.kind >= N_ADD) {
          if (q.a >= 0) roots.push_back(q.a);
          if (q.b >= 0) roots.push_back(q.b);
        }
      }
      if (need.size() > 12) no("a stage hands more than twelve blocks on to the next");
    }
    // the cells
    for (int sidx = 1; sidx <= L; sidx++) {
      Body c;
      CellSpec &cs = c.spec;
      const CellSpec &rs = reader.spec;
      cs.H = rs.H;
      cs.E = rs.E;
      cs.V = rs.V;
      cs.NX = rs.NX;
      cs.XD = rs.XD;
      cs.W = rs.W;
      cs.params = rs.params;
      cs.K = sidx == 1 ? rs.K : 1;
      cs.SI = sidx == 1 ? rs.SI : (int)T[sidx - 1].size();
      cs.S = sidx == L ? rs.S : (int)T[sidx].size();
      cs.has_ret = sidx == L;
      std::map<int, int> memo, local_bias, local_product;
      std::map<std::pair<int, int>, int> asrc_of;
      auto a_source = [&](int mask, int block) {
        auto key = std::make_pair(mask, block);
        if (!asrc_of.count(key)) {
          asrc_of[key] = (int)cs.asrc.size();
          cs.asrc.push_back({mask, block});
        }
        return asrc_of[key];
      };
      std::function<int(int)> conv = [&](int old) -> int {
        auto it = memo.find(old);
        if (it != memo.end()) return it->second;
        const ENode q = full.n[old];
        int id;
        if (q.kind == N_XW || q.kind == N_XD) {
          id = c.dag.make(q.kind, -1, -1, q.i0);
        } else if (q.kind == N_BIAS) {
          if (!local_bias.count(q.i0)) {
            local_bias[q.i0] = (int)cs.biases.size();
            cs.biases.push_back(rs.biases[q.i0]);
          }
          id = c.dag.make(N_BIAS, -1, -1, local_bias[q.i0]);
        } else if (sidx >= 2 && stage[old] < sidx) {  // written by the cell before: a block of this vertex's own row
          const auto &row = T[sidx - 1];
          id = c.dag.make(N_CS, -1, -1, 0, (int)(std::find(row.begin(), row.end(), old) - row.begin()));
        } else if (q.kind == N_CS) {
          id = c.dag.make(N_CS, -1, -1, q.i0, q.i1);
        } else if (q.kind == N_HU) {
          if (!local_product.count(q.i0)) {
            const RawProduct &rp = reader.raw[q.i0];
            CellProduct p;
            p.B = rp.B;
            p.ldb = rp.ldb;
            p.col = rp.col;
            for (const RawTerm &t : rp.terms) {
              int mask = 1, block = 0;
              if (sidx == 1) {
                if (!reader.child_sum(t.node, &mask, &block)) no("internal: a first-stage product with another left operand");
              } else {
                const auto &row = T[sidx - 1];
                block = (int)(std::find(row.begin(), row.end(), t.node) - row.begin());
              }
              p.terms.push_back({a_source(mask, block), t.brow});
            }
            local_product[q.i0] = (int)cs.products.size();
            cs.products.push_back(p);
          }
          id = c.dag.make(N_HU, -1, -1, local_product[q.i0]);
        } else {
          const int a = q.a >= 0 ? conv(q.a) : -1, b = q.b >= 0 ? conv(q.b) : -1;
          id = c.dag.make(q.kind, a, b, q.i0, q.i1, q.scale);
        }
        return memo[old] = id;
      };
      // (the products in their order of declaration, so that adjacent blocks of one MatMul stay adjacent)
      for (int id = 0; id < n; id++)
        if (full.n[id].kind == N_HU && stage[id] == sidx) conv(id);
      for (int id : (sidx == L ? reader.st : T[sidx])) c.st.push_back(conv(id));
      c.ret = sidx == L && reader.ret >= 0 ? conv(reader.ret) : -1;
      if (cs.products.empty()) no("internal: a stage without products");
      if (cs.products.size() > 16 || cs.asrc.size() > 8) no("too many products or operands in one stage");
      cs.xw_lo = L == 1 ? 0 : cs.NX;
      cs.xw_hi = L == 1 ? cs.NX : 0;
      for (const ENode &q : c.dag.n)
        if (q.kind == N_XW) {
          cs.xw_lo = std::min(cs.xw_lo, q.i0);
          cs.xw_hi = std::max(cs.xw_hi, q.i0 + 1);
        }
      for (CellBias &b : cs.biases)
        for (const Body &before : cells)
          for (const CellBias &e : before.spec.biases) b.add |= e.ref.param == b.ref.param && e.ref.offset == b.ref.offset;
      cells.push_back(std::move(c));
    }
    for (Body &c : cells) {
      nfwd.push_back((int)c.dag.n.size());
      derived.push_back(derive(c));
    }
  }
};

// the source of one cell's kernels; `ft`: the cell whose rows this one gathers, when it is another
// one (a chain), with what was derived for it
void write_cell(Body &c, const Derived &d, int nfwd, const Body *ft, const Derived *ftd, int ft_nfwd) {
  CellSpec &s = c.spec;
  const int H = s.H;
  s.waves = H % 128 == 0 ? 4 : H % 64 == 0 ? 2 : 1;
  // the partial tiles of a workgroup must fit in LDS
  const size_t per_wave = std::max(s.products.size(), s.asrc.size()) * 1024;
  if (s.waves * per_wave > 60 * 1024) no("too many accumulators for one workgroup");
  Writer w(c, d, true);
  w.kernels();
  w.elementwise(nfwd);
  if (ft) {
    const CellSpec &f = ft->spec;
    if (f.S != s.SI) no("internal: a cell gathers other rows than the cell before it writes");
    w.o << "#define FT_K " << f.K << "\n#define FT_S " << f.S << "\n#define FT_SI " << f.SI << "\n#define FT_NSV " << f.NSV << "\n#define FT_ND " << f.ND
        << "\n#define FT_DS_MASK " << ftd->ds_mask << "\n#define FT_BWD_CS " << (ftd->reads_cs ? 1 : 0) << "\n#define FT_HAS_RET " << (f.has_ret ? 1 : 0)
        << "\nnamespace ft {\n";
    Writer other(*ft, *ftd, true);
    other.elementwise(ft_nfwd);
    w.o << other.o.str() << "}  // namespace ft\n";
  } else {
    w.o << "#define FT_K CELL_K\n#define FT_S CELL_S\n#define FT_SI CELL_SI\n#define FT_NSV CELL_NSV\n#define FT_ND CELL_ND\n"
           "#define FT_DS_MASK CELL_DS_MASK\n#define FT_BWD_CS CELL_BWD_CS\n#define FT_HAS_RET CELL_HAS_RET\n"
           "namespace ft {\ntypedef ::BwdIn BwdIn;\ntypedef ::BwdOut BwdOut;\n"
           "static __device__ inline void cell_backward(const BwdIn &in, BwdOut &out) { ::cell_backward(in, out); }\n}  // namespace ft\n";
  }
  w.product_loops();
  w.o << kTemplate;
  s.source = w.o.str();
}

}  // namespace

Resolved resolve_external(const Edge *e) {
  Resolved r;
  r.count = e->width();
  long off = 0;
  const Edge *cur = e;
  while (cur && cur->src) {
    const OpDef &d = cur->src->def;
    const std::string &op = d.name();
    if (op == "Variable") {
      r.var = cur->name;
      r.offset = off;
      r.ok = true;
      return r;
    }
    if (op == "Mirror" || op == "Reshape" || op == "Flatten" || op == "Expand_dims") {
      cur = cur->src->in[0];
    } else if (op == "Slice") {
      const Edge *in = cur->src->in[0];
      long stride = d.find_attr("Split") ? in->width() / GetSingleArg<int>(d, "Split") : GetSingleArg<int>(d, "Stride");
      off += d.find_attr("Split") ? stride * GetSingleArg<int>(d, "Index") : GetSingleArg<int>(d, "Offset");
      cur = in;
    } else {
      return r;
    }
  }
  return r;
}

std::unique_ptr<CellMatch> match_cell(const Graph &g, std::string *why) {
  try {
    Chain b(g);
    std::shared_ptr<CellSpec> head, tail;
    const size_t L = b.cells.size();
    for (size_t i = 0; i < L; i++) {
      const size_t p = (i + L - 1) % L;  // whose rows cell i gathers
      write_cell(b.cells[i], b.derived[i], b.nfwd[i], L > 1 ? &b.cells[p] : nullptr, L > 1 ? &b.derived[p] : nullptr, b.nfwd[p]);
      auto spec = std::make_shared<CellSpec>(b.cells[i].spec);
      if (tail) tail->next = spec;
      else head = spec;
      tail = spec;
    }
    auto m = std::make_unique<CellMatch>();
    m->spec = head;
    m->roles = b.reader.roles;
    m->slots = b.reader.slots;
    return m;
  } catch (const Fail &f) {
    if (why) *why = f.why;
    return nullptr;
  }
}

std::string cell_host_source(const Graph &g, int stage) {
  try {
    Chain b(g);
    if (stage < 0 || stage >= (int)b.cells.size()) return "// no such stage\n";
    Writer w(b.cells[stage], b.derived[stage], false);
    w.o << "#include <math.h>\n";
    w.elementwise(b.nfwd[stage]);
    const CellSpec &s = b.cells[stage].spec;
    w.o << "// stages=" << b.cells.size() << "\n";
    w.o << "// H=" << s.H << " K=" << s.K << " S=" << s.S << " SI=" << s.SI << " NX=" << s.NX << " XD=" << s.XD << " NP=" << s.products.size()
        << " NB=" << s.biases.size() << " ND=" << s.ND << " NSV=" << s.NSV << "\n";
    for (size_t p = 0; p < s.products.size(); p++) w.o << "// product " << p << " dcol " << s.products[p].dcol << "\n";
    for (size_t i = 0; i < s.biases.size(); i++) w.o << "// bias " << i << " dcol " << s.biases[i].dcol << "\n";
    return w.o.str();
  } catch (const Fail &f) {
    return "// not a cell: " + f.why + "\n";
  }
}

}  // namespace mid
}  // namespace cavs
