#include "graph.h"

#include <algorithm>
#include <sstream>
#include <stdexcept>

#include "cavs/util/op_def_builder.h"

namespace cavs {
namespace mid {

void graph_error(const std::string &msg) { throw std::runtime_error(msg); }

Edge *Scope::find(const std::string &n, bool upward) const {
  auto it = edges.find(n);
  if (it != edges.end()) return it->second.get();
  return (upward && parent) ? parent->find(n, true) : nullptr;
}

Edge *Scope::add_edge(const std::string &n, const std::vector<int> &shape) {
  if (edges.count(n)) graph_error("edge '" + n + "' is defined twice in scope " + name);
  auto e = std::make_unique<Edge>();
  e->name = n;
  e->shape = shape;
  e->scope = this;
  Edge *p = e.get();
  edges[n] = std::move(e);
  return p;
}

static Graph *g_graph = nullptr;
Graph &global_graph() {
  if (!g_graph) g_graph = new Graph();
  return *g_graph;
}
Graph *swap_global_graph(Graph *g) {
  Graph *old = g_graph;
  g_graph = g;
  return old;
}
void reset_global_graph() {
  delete g_graph;
  g_graph = nullptr;
}

// ------------------------------------------------------------------ shape inference
static long count_of(const std::vector<int> &s) {
  long c = 1;
  for (int d : s) c *= (d > 0 ? d : 1);
  return c;
}
static bool has_dyn(const std::vector<int> &s) {
  for (int d : s) if (d < 0) return true;
  return false;
}

// Follows the ShapeInference methods of cavs/backend/op_decl_*.cc for the operators on the path.
std::vector<std::vector<int>> infer_shapes(const OpDef &def, const std::vector<const Edge *> &in) {
  const std::string &op = def.name();
  auto need = [&](size_t n) {
    if (in.size() != n) graph_error(op + " expects " + std::to_string(n) + " inputs: " + def.DebugString());
  };
  auto declared = [&]() {
    if (def.shape_size() < 1) graph_error(op + " needs a declared shape: " + def.DebugString());
    return def.shape(0).dims;
  };
  if (op == "Variable" || op == "Placeholder" || op == "ConstOp" || op == "Gather" || op == "Pull" ||
      op == "GraphOutput")
    return {declared()};
  if (op == "Add" || op == "Sub" || op == "Mul" || op == "Equal") {  // op_decl_elementwise.h: the larger operand
    need(2);
    const Edge *big = count_of(in[0]->shape) >= count_of(in[1]->shape) && !has_dyn(in[1]->shape) ? in[0] : in[1];
    if (has_dyn(in[0]->shape)) big = in[0];
    return {big->shape};
  }
  if (op == "Sigmoid" || op == "Tanh" || op == "Relu" || op == "Abs" || op == "Square" || op == "Mirror" ||
      op == "Scatter" || op == "Push" || op == "Neg" || op == "Assign") {
    need(1);
    return {in[0]->shape};
  }
  if (op == "Reduce_sum" || op == "Reduce_mean") {
    need(1);
    return {{1}};
  }
  if (op == "Reshape") {  // op_decl_reshape.cc: the declared shape, element count preserved
    need(1);
    std::vector<int> s = declared();
    if (!has_dyn(s) && !has_dyn(in[0]->shape) && count_of(s) != count_of(in[0]->shape))
      graph_error("Reshape changes the element count: " + def.DebugString());
    return {s};
  }
  if (op == "Flatten") {
    need(1);
    const auto &s = in[0]->shape;
    int rest = 1;
    for (size_t i = 1; i < s.size(); i++) rest *= s[i];
    return {{s[0], rest}};
  }
  if (op == "Expand_dims") {
    need(1);
    std::vector<int> s = in[0]->shape;
    int axis = GetSingleArg<int>(def, "Axis", 0);
    if (axis < 0 || axis > (int)s.size()) graph_error("Expand_dims axis out of range");
    s.insert(s.begin() + axis, 1);
    return {s};
  }
  if (op == "Slice") {  // op_decl_slice_join.cc:46-63: a 1-D block of the flattened input
    need(1);
    long dims = count_of(in[0]->shape);
    int stride;
    if (def.find_attr("Split")) {
      int split = GetSingleArg<int>(def, "Split");
      if (split <= 0 || dims % split) graph_error("Slice cannot split " + std::to_string(dims) + " by " + std::to_string(split));
      stride = (int)(dims / split);
    } else {
      stride = GetSingleArg<int>(def, "Stride");
      int offset = GetSingleArg<int>(def, "Offset");
      if (offset < 0 || stride <= 0 || offset + stride > dims) graph_error("Slice out of range: " + def.DebugString());
    }
    return {{stride}};
  }
  if (op == "Concat") {  // op_decl_slice_join.cc:98-122, axis 0
    if (in.empty()) graph_error("Concat of nothing");
    std::vector<int> s = in[0]->shape;
    int sum = 0;
    for (auto *e : in) {
      if (e->shape.size() != s.size()) graph_error("Concat ranks differ");
      sum += e->shape[0];
    }
    s[0] = sum;
    return {s};
  }
  if (op == "MatMul") {  // op_decl_matmul.cc: [m,k] x [k,n], with the Transpose attribute used by gradients
    need(2);
    std::vector<int> a = in[0]->shape, b = in[1]->shape;
    if (a.size() == 1) a.insert(a.begin(), 1);
    if (a.size() != 2 || b.size() != 2) graph_error("MatMul needs matrices: " + def.DebugString());
    if (a[1] != b[0]) graph_error("MatMul inner dimensions differ: " + def.DebugString());
    return {{a[0], b[1]}};
  }
  if (op == "EmbeddingLookup") {  // op_decl_embedding_lookup.cc: input dims + embedding width
    need(2);
    if (in[1]->shape.size() != 2) graph_error("EmbeddingLookup needs a [vocabulary, width] table");
    std::vector<int> s = in[0]->shape;
    s.push_back(in[1]->shape[1]);
    return {s};
  }
  if (op == "FullyConnected") {  // op_decl_fullyconnected.cc: X[N,K] W[Out,K] B[1,Out]
    need(3);
    const auto &x = in[0]->shape, &w = in[1]->shape, &b = in[2]->shape;
    if (x.size() != 2 || w.size() != 2 || b.size() != 2 || x[1] != w[1] || b[0] != 1 || b[1] != w[0])
      graph_error("FullyConnected shapes do not agree: " + def.DebugString());
    return {{x[0], w[0]}};
  }
  if (op == "SoftmaxEntropyLoss") {
    need(2);
    if (in[0]->shape.size() != 2) graph_error("SoftmaxEntropyLoss needs [N, classes] logits");
    return {{in[0]->shape[0], 1}};
  }
  graph_error("operator '" + op + "' is outside the F-over-G path and is not implemented");
}

// ------------------------------------------------------------------ graph construction
static Node *add_node(Scope *s, const OpDef &def) {
  auto n = std::make_unique<Node>();
  n->def = def;
  n->scope = s;
  std::vector<const Edge *> ins;
  for (auto &name : def.input()) {
    Edge *e = s->find(name);
    if (!e) graph_error("input '" + name + "' of " + def.name() + " is not defined");
    n->in.push_back(e);
    ins.push_back(e);
    e->dst.push_back(n.get());
  }
  auto shapes = infer_shapes(def, ins);
  for (int i = 0; i < def.output_size(); i++) {
    Edge *e = s->add_edge(def.output(i), shapes[std::min<size_t>(i, shapes.size() - 1)]);
    e->src = n.get();
    n->out.push_back(e);
  }
  n->def.clear_shape();
  for (auto *e : n->out) n->def.add_shape()->dims = e->shape;
  Node *p = n.get();
  s->nodes.push_back(std::move(n));
  return p;
}

std::vector<int> Graph::add_op(const OpDef &def) {
  if (def.output_size() < 1) graph_error("an operator needs an output name");
  Node *n = add_node(&main, def);
  if (def.name() == "GraphOutput") {
    if (!func) graph_error("GraphOutput without a vertex function");
    graph_output = def.output(0);
    // every external edge the function reads becomes an extra input of GraphOutput
    // (cavs/midend/scope.cc:65-89), which is how gradients reach the weights
    for (auto &name : func_inputs) {
      Edge *e = main.find(name);
      n->in.push_back(e);
      n->def.add_input(name);
      e->dst.push_back(n);
    }
  }
  version++;
  return n->out[0]->shape;
}

// cavs/midend/graph_util.cc:296-332: the function body gets its own scope; an edge is
// dynamic iff Gather/Pull produced it or an op with a dynamic input did.
std::vector<int> Graph::add_function(const FunctionDef &fdef) {
  if (func) graph_error("only one vertex function per program is supported");
  func = std::make_unique<Scope>();
  func->name = fdef.name();
  func->parent = &main;
  std::vector<int> ret;
  std::set<std::string> ext;
  for (const OpDef &d : fdef.ops()) {
    Node *n = add_node(func.get(), d);
    bool dyn = d.name() == "Gather" || d.name() == "Pull";
    for (Edge *e : n->in) {
      dyn |= e->dynamic;
      if (e->scope != func.get() && ext.insert(e->name).second) func_inputs.push_back(e->name);
    }
    for (Edge *e : n->out) e->dynamic = dyn;
    if (d.name() == "Push") ret = n->out[0]->shape;
  }
  if (ret.empty()) graph_error("the vertex function has no Push");
  func_ret_shape = ret;
  version++;
  return ret;
}

void Graph::add_control_dependency(const OpDef &def) {
  // ControlDependency(a, b): a's producer runs after b is available
  if (def.input_size() != 2) graph_error("ControlDependency takes two inputs");
  Edge *a = main.find(def.input(0));
  if (!a || !a->src) graph_error("ControlDependency on an unknown symbol");
  a->src->after.push_back(def.input(1));
  version++;
}

// ------------------------------------------------------------------ autograd
namespace {

struct GradBuilder {
  Scope *scope;
  std::set<std::string> trainable;       // edges a gradient must reach
  std::set<std::string> written;         // gradient edges that already have a producer
  std::vector<OpDef> out;

  static std::string G(const std::string &n) { return GetGradientName(n); }

  // Adds one gradient op; each output accumulates iff an earlier op already wrote it
  // (the reference only accumulates through Mirror/Slice, cavs/midend/edge.cc:27-38).
  void emit(OpDefBuilder &b, const std::vector<std::string> &outputs) {
    std::vector<int> acc;
    for (auto &o : outputs) {
      b.Output(o);
      acc.push_back(written.count(o) ? 1 : 0);
      written.insert(o);
    }
    b.AttrList("Acc", acc);
    out.push_back(b.Finalize());
  }

  bool wants(const Edge *e) const { return trainable.count(e->name) != 0; }

  // MakeGradient of one forward node, given that G(output) exists.
  void node_grad(const Node *n) {
    const OpDef &d = n->def;
    const std::string &op = d.name();
    auto in = [&](int i) { return n->in[i]->name; };
    const std::string y = n->out.empty() ? "" : n->out[0]->name;
    const std::string dy = G(y);
    if (op == "Add" || op == "Sub") {
      // op_decl_elementwise_arithmetic.cc:28-66: each operand receives dy (column-summed when
      // the operand is a row broadcast over the slab); Sub negates the second
      for (int i = 0; i < 2; i++) {
        if (!wants(n->in[i])) continue;
        OpDefBuilder b(i == 1 && op == "Sub" ? "Neg" : "Assign");
        b.Input(dy).Device(d);
        emit(b, {G(in(i))});
      }
    } else if (op == "Mul") {  // :68-109: da = dy*b, db = dy*a
      for (int i = 0; i < 2; i++) {
        if (!wants(n->in[i])) continue;
        OpDefBuilder b("Mul");
        b.Input(dy).Input(in(1 - i)).Device(d);
        emit(b, {G(in(i))});
      }
    } else if (op == "MatMul") {  // op_decl_matmul.cc:18-69
      if (wants(n->in[0])) {
        OpDefBuilder b("MatMul");
        b.Input(dy).Input(in(1)).AttrList("Transpose", std::vector<int>{0, 1}).Device(d);
        emit(b, {G(in(0))});
      }
      if (wants(n->in[1])) {
        OpDefBuilder b("MatMul");
        b.Input(in(0)).Input(dy).AttrList("Transpose", std::vector<int>{1, 0}).Device(d);
        emit(b, {G(in(1))});
      }
    } else if (op == "Sigmoid" || op == "Tanh" || op == "Relu") {  // op_decl_elementwise_activation.cc: (dy, y, x)
      if (wants(n->in[0])) {
        OpDefBuilder b(GetGradientName(op));
        b.Input(dy).Input(y).Input(in(0)).Device(d);
        emit(b, {G(in(0))});
      }
    } else if (op == "Square") {
      if (wants(n->in[0])) {
        OpDefBuilder b("Mul");
        b.Input(dy).Input(in(0)).AttrSingle("Scale", 2.f).Device(d);
        emit(b, {G(in(0))});
      }
    } else if (op == "Slice") {  // op_decl_slice_join.cc:32-43
      if (wants(n->in[0])) {
        if (!written.count(G(in(0)))) {  // the block is added into a zeroed buffer
          OpDefBuilder z("Fill");
          z.Input(in(0)).AttrSingle("Value", 0.f).Device(d);
          emit(z, {G(in(0))});
        }
        OpDefBuilder b("PartialAccumulate");
        b.Input(dy).Input(in(0)).Attr(d).Device(d);
        emit(b, {G(in(0))});
      }
    } else if (op == "Concat") {  // :79-95
      std::vector<std::string> outs, ins;
      bool any = false;
      for (auto *e : n->in) {
        ins.push_back(e->name);
        outs.push_back(G(e->name));
        any |= wants(e);
      }
      if (any) {
        OpDefBuilder b("SliceAll");
        b.Input(dy).Input(ins).Device(d);
        emit(b, outs);
      }
    } else if (op == "Mirror") {  // :173-182
      if (wants(n->in[0])) {
        OpDefBuilder b("Accumulate");
        b.Input(dy).Device(d);
        emit(b, {G(in(0))});
      }
    } else if (op == "Reshape" || op == "Flatten" || op == "Expand_dims") {  // op_decl_reshape.cc:14-25
      if (wants(n->in[0])) {
        OpDefBuilder b("ReshapeLike");
        b.Input(dy).Input(in(0)).Device(d);
        emit(b, {G(in(0))});
      }
    } else if (op == "EmbeddingLookup") {  // op_decl_embedding_lookup.cc: only the table gets a gradient
      if (wants(n->in[1])) {
        OpDefBuilder b(GetGradientName(op));
        b.Input(dy).Input(in(0)).Device(d);
        emit(b, {G(in(1))});
      }
    } else if (op == "Gather") {  // op_decl_graphop.cc:25-141: Gather <-> Scatter, Pull <-> Push
      OpDefBuilder b("Scatter");
      b.Input(dy).AttrSingle("Child", GetSingleArg<int>(d, "Child", 0)).AttrSingle("Backward", true).Device(d);
      emit(b, {});
    } else if (op == "Scatter") {
      OpDefBuilder b("Gather");
      b.AttrSingle("Child", 0).AttrSingle("Backward", true).Shape(n->in[0]->shape).Device(d);
      emit(b, {G(in(0))});
    } else if (op == "Push") {
      OpDefBuilder b("Pull");
      b.AttrSingle("Backward", true).Shape(n->in[0]->shape).Device(d);
      emit(b, {G(in(0))});
    } else if (op == "Pull") {
      // its gradient (a Push of d vertex-input) is never consumed: the vertex placeholder is not trainable
    } else if (op == "FullyConnected") {  // op_decl_fullyconnected.cc: (dY, X, W, B) -> (dW, dB, dX)
      OpDefBuilder b(GetGradientName(op));
      b.Input(dy).Input(in(0)).Input(in(1)).Input(in(2)).Device(d);
      emit(b, {G(in(1)), G(in(2)), G(in(0))});
    } else if (op == "SoftmaxEntropyLoss") {  // ignores dy, scales by 1/N (op_impl_softmax_entropy_logits_loss.cu:212-250)
      OpDefBuilder b(GetGradientName(op));
      b.Input(in(0)).Input(in(1)).Device(d);
      emit(b, {G(in(0))});
    } else if (op == "Reduce_sum" || op == "Reduce_mean") {  // op_decl_reduction.cc:19-28: broadcast of dy
      OpDefBuilder b("Fill");
      b.Input(in(0)).Input(dy).AttrSingle("Mean", op == "Reduce_mean").Device(d);
      emit(b, {G(in(0))});
    } else if (op == "Abs") {
      graph_error("Abs has no gradient on this path");
    } else if (op == "GraphOutput") {
      // (dGraphOutput, forward inputs...) -> gradients of the external edges F reads
      std::vector<std::string> outs;
      for (size_t i = 2; i < n->in.size(); i++) outs.push_back(G(n->in[i]->name));
      OpDefBuilder b(GetGradientName(op));
      b.Input(dy).Input(d.input()).Device(d);
      emit(b, outs);
    } else if (op == "Variable" || op == "Placeholder" || op == "ConstOp") {
    } else {
      graph_error("no gradient rule for operator '" + op + "'");
    }
  }
};

// edges of `s` (and of F's external inputs) from which a trainable variable is reachable backwards
std::set<std::string> reaches_variable(const Scope &s, const std::set<std::string> &vars,
                                       const std::set<std::string> &extra = {}) {
  std::set<std::string> r(vars);
  r.insert(extra.begin(), extra.end());
  for (auto &n : s.nodes) {
    bool any = false;
    for (Edge *e : n->in) any |= r.count(e->name) != 0;
    if (n->def.name() == "Pull" || n->def.name() == "Gather") any = n->def.name() == "Gather";
    if (any)
      for (Edge *e : n->out) r.insert(e->name);
  }
  return r;
}

}  // namespace

// cavs/midend/graph_util.cc:262-294 (AddOptimizerOp), :87-152 (GenGradient), :334-458
// (ComputeGradientForFunction).
void Graph::add_optimizer(const OpDef &def) {
  if (opt.present) graph_error("only one optimizer per program is supported");
  if (def.input_size() != 1) graph_error("Optimizer takes the loss as its only input");
  Edge *loss = main.find(def.input(0));
  if (!loss) graph_error("Optimizer on an unknown symbol");
  opt.present = true;
  opt.output = def.output(0);
  opt.loss = loss->name;
  opt.lr = GetSingleArg<float>(def, "Learning_rate", 1.f);
  opt.clip = GetSingleArg<float>(def, "Clip", 0.f);
  opt.iters = GetSingleArg<int>(def, "Iters", 1);
  opt.vars = GetListArgS(def, "Vars");
  if (opt.vars.empty())  // all Variables (cavs/frontend/c_api.cc:119-141)
    for (auto &n : main.nodes)
      if (n->def.name() == "Variable") opt.vars.push_back(n->out[0]->name);
  std::set<std::string> vars(opt.vars.begin(), opt.vars.end());

  // ---- main scope: nodes on a path variable -> loss, reverse topological order
  std::set<std::string> fwd = reaches_variable(main, vars);
  std::set<const Node *> back;  // nodes from which the loss is reachable
  {
    std::vector<const Node *> stack = {loss->src};
    while (!stack.empty()) {
      const Node *n = stack.back();
      stack.pop_back();
      if (!n || !back.insert(n).second) continue;
      for (Edge *e : n->in) stack.push_back(e->src);
    }
  }
  GradBuilder gb;
  gb.scope = &main;
  gb.trainable = fwd;
  {
    OpDefBuilder seed("ConstOp");  // d loss = 1 (graph_util.cc:117-126)
    seed.AttrSingle("init", 1.f).Shape(loss->shape).Input(loss->name);
    gb.emit(seed, {GetGradientName(loss->name)});
  }
  for (auto it = main.nodes.rbegin(); it != main.nodes.rend(); ++it) {
    const Node *n = it->get();
    if (!back.count(n) || n->out.empty() || !fwd.count(n->out[0]->name)) continue;
    if (!gb.written.count(GetGradientName(n->out[0]->name))) continue;
    if (n->def.name() == "GraphOutput") {
      // ---- backward vertex function
      std::set<std::string> ext;
      for (size_t i = 2; i < n->in.size(); i++)
        if (fwd.count(n->in[i]->name)) ext.insert(n->in[i]->name);
      std::set<std::string> ffwd = reaches_variable(*func, {}, ext);
      GradBuilder fb;
      fb.scope = func.get();
      fb.trainable = ffwd;
      // terminals: the gradients of Push and Scatter inputs come from Pull / Gather
      for (auto fit = func->nodes.rbegin(); fit != func->nodes.rend(); ++fit) {
        const Node *fn = fit->get();
        const std::string &fop = fn->def.name();
        bool terminal = fop == "Push" || fop == "Scatter";
        if (!terminal) {
          if (fn->out.empty() || !ffwd.count(fn->out[0]->name)) continue;
          if (!fb.written.count(GetGradientName(fn->out[0]->name))) continue;
        } else if (!ffwd.count(fn->in[0]->name)) {
          continue;
        }
        fb.node_grad(fn);
      }
      // BatchingWeightUpdater (cavs/midend/batch_weight_updater.h:12-84): ops that only
      // produce gradients of non-dynamic edges run once, after the loop, over all rows
      func_backward.clear();
      func_deferred.clear();
      std::set<std::string> deferred_out;
      for (const OpDef &g : fb.out) {
        bool all_static = g.output_size() > 0;
        for (auto &o : g.output()) {
          Edge *fe = func->find(GetOriginName(o));
          if (!fe) graph_error("gradient of unknown edge " + o);
          all_static &= !fe->dynamic;
        }
        if (all_static) {
          func_deferred.push_back(g);
          for (auto &o : g.output()) deferred_out.insert(o);
        } else {
          for (auto &i : g.input())
            if (deferred_out.count(i)) graph_error("a per-round gradient op depends on a deferred one: " + g.DebugString());
          func_backward.push_back(g);
        }
      }
      // the external gradients F produced count as written in the main scope
      std::vector<std::string> produced;
      for (size_t i = 2; i < n->in.size(); i++)
        if (fb.written.count(GetGradientName(n->in[i]->name))) produced.push_back(n->in[i]->name);
      OpDefBuilder b("GraphOutput_grad");
      b.Input(GetGradientName(n->out[0]->name)).Input(n->def.input()).Device(n->def);
      std::vector<std::string> outs;
      for (auto &p : produced) outs.push_back(GetGradientName(p));
      gb.emit(b, outs);
      continue;
    }
    gb.node_grad(n);
  }
  opt.backward = gb.out;
  for (auto &v : opt.vars)
    if (!gb.written.count(GetGradientName(v))) {
      // a variable the loss does not depend on keeps a zero gradient
      OpDefBuilder z("Fill");
      z.Input(v).AttrSingle("Value", 0.f);
      gb.emit(z, {GetGradientName(v)});
      opt.backward.push_back(gb.out.back());
    }
  version++;
}

std::string Graph::dump() const {
  std::ostringstream o;
  o << "main:\n";
  for (auto &n : main.nodes) o << "  " << n->def.DebugString() << "\n";
  if (func) {
    o << "function " << func->name << ":\n";
    for (auto &n : func->nodes) o << "  " << n->def.DebugString() << (n->out.size() && n->out[0]->dynamic ? "  [dynamic]" : "") << "\n";
    o << "function " << func->name << "_grad (per round):\n";
    for (auto &d : func_backward) o << "  " << d.DebugString() << "\n";
    o << "function " << func->name << "_grad (deferred, all rows):\n";
    for (auto &d : func_deferred) o << "  " << d.DebugString() << "\n";
  }
  if (opt.present) {
    o << "backward (main):\n";
    for (auto &d : opt.backward) o << "  " << d.DebugString() << "\n";
  }
  return o.str();
}

}  // namespace mid
}  // namespace cavs
