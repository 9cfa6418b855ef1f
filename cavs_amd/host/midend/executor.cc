#include "executor.h"

#include <algorithm>
#include <cstdio>
#include <cmath>
#include <cstring>

#include "fusion.h"
#include "lowering.h"

namespace cavs {
namespace mid {

namespace {
// splitmix64: deterministic filler streams (the reference default-constructs a
// std::default_random_engine per filler, cavs/backend/functor_filler.h:92-97, so every
// Uniform variable starts with the same stream; here each variable gets its own)
struct Rng {
  uint64_t s;
  uint64_t next() {
    s += 0x9E3779B97F4A7C15ull;
    uint64_t z = s;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
  }
  float uniform() { return (float)(next() >> 40) / (float)(1 << 24); }
};

long numel(const std::vector<int> &s) {
  long c = 1;
  for (int d : s) c *= (d > 0 ? d : 1);
  return c;
}
}  // namespace

Executor::Executor(int opt, const std::string &name) : opt_(opt), name_(name) {
  check(cavs_init(0));
  check(cavs_stream_create(&stream_));
}

Executor::~Executor() {
  cavs_stream_sync(stream_);
  engine_.reset();
  if (copy_stream_) {
    cavs_stream_sync(copy_stream_);
    cavs_stream_destroy(copy_stream_);
  }
  for (void *e : {feeds_up_ev_, run_done_ev_[0], run_done_ev_[1]})
    if (e) cavs_event_destroy(e);
  for (auto &kv : fused_handles_)
    if (kv.second) cavs_fused_release(kv.second);
  tensors_.clear();
  cavs_stream_destroy(stream_);
}

const Edge *Executor::edge(const std::string &name) const {
  Graph &g = global_graph();
  const Edge *e = g.func ? g.func->find(name) : g.main.find(name);
  if (!e && IsGradientName(name)) e = edge(GetOriginName(name));  // a gradient has its origin's geometry
  return e;
}

Tensor *Executor::find_tensor(const std::string &name) {
  auto it = tensors_.find(name);
  return it == tensors_.end() ? nullptr : it->second.get();
}

Tensor &Executor::tensor(const std::string &name) {
  Tensor *t = find_tensor(name);
  if (!t) fail(CAVS_EINVAL, "tensor '" + name + "' has not been computed");
  return *t;
}

float *Executor::workspace(size_t bytes) {
  if (ws_.capacity() * 4 < bytes) {
    check(cavs_stream_sync(stream_));
    ws_.reserve(std::max<size_t>(bytes / 4 + 1, (size_t)4 << 20));
  }
  return ws_.get();
}

void Executor::set_variable(const std::string &name, const float *data, size_t n) {
  const Edge *e = global_graph().main.find(name);
  if (!e || !e->src || e->src->def.name() != "Variable") fail(CAVS_EINVAL, "'" + name + "' is not a Variable");
  if ((size_t)numel(e->shape) != n)
    fail(CAVS_EINVAL, "Variable '" + name + "' has " + std::to_string(numel(e->shape)) + " elements, got " + std::to_string(n));
  pending_vars_[name].assign(data, data + n);
  Tensor *t = find_tensor(name);
  if (t) {
    check(cavs_memcpy_h2d(t->base, data, n * 4, stream_));
    check(cavs_stream_sync(stream_));
  }
}

void Executor::init_variables() {
  Graph &g = global_graph();
  uint64_t index = 0;
  for (auto &n : g.main.nodes) {
    if (n->def.name() != "Variable") continue;
    const std::string &name = n->out[0]->name;
    index++;
    if (find_tensor(name)) continue;
    auto t = std::make_unique<Tensor>();
    t->width = numel(n->out[0]->shape);
    t->own.reserve(t->width);
    t->base = t->own.get();
    std::vector<float> host(t->width);
    auto pv = pending_vars_.find(name);
    if (pv != pending_vars_.end()) {
      host = pv->second;
    } else {
      const std::string &label = n->def.label();
      Rng rng{0x5EEDull * 1315423911ull + index * 0x9E3779B97F4A7C15ull};
      if (label == "ConstantFiller") {
        std::fill(host.begin(), host.end(), GetSingleArg<float>(n->def, "const_value", 0.f));
      } else if (label == "Uniform") {
        float lo = GetSingleArg<float>(n->def, "minval", -1.f), hi = GetSingleArg<float>(n->def, "maxval", 1.f);
        for (auto &v : host) v = lo + (hi - lo) * rng.uniform();
      } else if (label == "Normal") {
        for (auto &v : host) {
          float u1 = std::max(rng.uniform(), 1e-7f), u2 = rng.uniform();
          v = std::sqrt(-2.f * std::log(u1)) * std::cos(6.2831853f * u2);
        }
      } else if (label == "Xavier") {
        float fan = (float)std::max<long>(1, t->width / std::max(1, n->out[0]->shape[0]));
        float a = std::sqrt(3.f / fan);
        for (auto &v : host) v = -a + 2 * a * rng.uniform();
      } else {
        fail(CAVS_EUNSUPPORTED, "filler '" + label + "' is not implemented");
      }
    }
    check(cavs_memcpy_h2d(t->base, host.data(), host.size() * 4, stream_));
    check(cavs_stream_sync(stream_));
    tensors_[name] = std::move(t);
  }
}

void Executor::compile() {
  Graph &g = global_graph();
  if (compiled_version_ == g.version) return;
  compiled_version_ = g.version;
  nch_ = 0;
  pool_w_ = ret_w_ = arg_w_ = 0;
  lowered_ = false;
  lowering_.reset();
  if (engine_) {  // (made for the program as it was)
    check(cavs_stream_sync(stream_));
    engine_.reset();
  }
  if (g.func) {
    for (auto &n : g.func->nodes) {
      const std::string &op = n->def.name();
      if (op == "Gather") {
        int c = GetSingleArg<int>(n->def, "Child", 0);
        if (c < 0 || c > 1) fail(CAVS_EUNSUPPORTED, "Gather child index must be 0 or 1");
        nch_ = std::max(nch_, c + 1);
        long w = n->out[0]->width();
        if (pool_w_ && pool_w_ != w) fail(CAVS_EINVAL, "all Gather/Scatter messages must have one width");
        pool_w_ = w;
      } else if (op == "Scatter") {
        long w = n->in[0]->width();
        if (pool_w_ && pool_w_ != w) fail(CAVS_EINVAL, "all Gather/Scatter messages must have one width");
        pool_w_ = w;
      } else if (op == "Push") {
        ret_w_ = n->in[0]->width();
      } else if (op == "Pull") {
        arg_w_ = n->out[0]->width();
      }
    }
    if (lowering_mode_ > 0 && (opt_ & OPT_BATCHING)) {
      lowering_ = match_vertex_function(g, lowering_mode_ == 1 ? 1 : 2);
      if (lowering_ && lowering_->cell) {
        // the generated kernels must compile (the module stays cached for the engine); if they do
        // not, F runs operator by operator like any function that is not of the shape
        for (std::shared_ptr<const CellSpec> c = lowering_->cell; c; c = c->next) {
          void *module = nullptr;
          if (cavs_cell_compile(c->source.c_str(), &module) != CAVS_OK) {
            std::fprintf(stderr, "cavs: the round kernels generated for the vertex function did not compile (%s); running it operator by operator\n",
                         cavs_last_error());
            lowering_.reset();
            break;
          }
          cavs_cell_release(module);
        }
      }
      lowered_ = lowering_ != nullptr;
    }
  }
  // programs as executed; with OPT_FUSION connected elementwise operators become generated kernels
  func_fwd_.clear();
  func_bwd_ = g.func_backward;
  func_def_ = g.func_deferred;
  main_all_.clear();
  main_cache_.clear();
  fused_groups_ = 0;
  for (auto &n : g.main.nodes) main_all_.push_back(n->def);
  if (g.func)
    for (auto &n : g.func->nodes) func_fwd_.push_back(n->def);
  round_zero_.clear();
  if ((opt_ & OPT_FUSION) && g.func && !lowered_) {
    std::vector<OpDef> fwd = fused(func_fwd_, {&func_bwd_, &func_def_, &main_all_, &g.opt.backward}, {});
    // the per-round backward program, with the deferred ops that fit riding along as reducing outputs
    FusionEnv env = graph_env(g);
    for (auto *o : {&func_fwd_, &main_all_, &g.opt.backward})
      for (auto &d : *o)
        for (int k = 0; k < operands_read(d); k++) env.live.insert(d.input(k));
    for (auto &v : g.opt.vars) env.live.insert(GetGradientName(v));
    BackwardFusion bf = fuse_function_backward(func_bwd_, func_def_, env);
    fused_groups_ += bf.groups;
    round_zero_ = bf.zero_before_loop;
    std::vector<OpDef> &kept_bwd = bf.per_round, &new_def = bf.deferred;
    func_fwd_.swap(fwd);
    func_bwd_.swap(kept_bwd);
    func_def_.swap(new_def);
  }
}

std::vector<OpDef> Executor::fused(const std::vector<OpDef> &prog, const std::vector<const std::vector<OpDef> *> &others,
                                   const std::vector<std::string> &extra_live) {
  Graph &g = global_graph();
  FusionEnv env = graph_env(g);
  for (auto *o : others)
    for (auto &d : *o)
      for (int k = 0; k < operands_read(d); k++) env.live.insert(d.input(k));
  for (auto &v : g.opt.vars) env.live.insert(GetGradientName(v));
  for (auto &x : extra_live) env.live.insert(x);
  int made = 0;
  std::vector<OpDef> out = fuse_program(prog, env, &made);
  fused_groups_ += made;
  return out;
}

// FusedKernel: the generated kernel reads x[idx % x_count], so per-round slabs and
// broadcast rows go in with their own element counts (cavs/backend/op_impl_fusedkernel.cu)
void Executor::exec_fused(const OpDef &d, const RoundCtx &c) {
  const std::string kname = GetSingleArg<std::string>(d, "KernelName", "");
  void *&h = fused_handles_[kname];
  if (!h) check(cavs_fused_compile(kname.c_str(), GetSingleArg<std::string>(d, "KernelSource", "").c_str(), &h));
  std::vector<float *> outs;
  std::vector<const float *> ins;
  std::vector<int> oc, ic;
  // the element range is that of the widest argument (cavs/backend/op_impl_fused_kernel.cu:44-58);
  // outputs narrower than it are added to with atomicAdd
  long cnt, w, n_elements = 0;
  for (auto &x : d.input()) {
    ins.push_back(view(x, c, &cnt, &w));
    ic.push_back((int)cnt);
    n_elements = std::max(n_elements, cnt);
  }
  const std::vector<std::string> zero_first = GetListArgS(d, "ZeroEnforced");
  for (int i = 0; i < d.output_size(); i++) {
    const std::string &name = d.output(i);
    const Edge *e = edge(name);
    if (!e) fail(CAVS_EINVAL, "no edge for fused output '" + name + "'");
    auto &slot = tensors_[name];
    if (!slot) slot = std::make_unique<Tensor>();
    Tensor &t = *slot;
    t.width = e->width();
    t.per_vertex = e->per_vertex();
    if (t.per_vertex) t.rows = N_;
    if (t.own.capacity() < t.count()) {
      check(cavs_stream_sync(stream_));
      t.own.reserve(t.count() + t.count() / 4);
    }
    t.base = t.own.get();
    outs.push_back(view(name, c, &cnt, &w));
    oc.push_back((int)cnt);
    n_elements = std::max(n_elements, cnt);
    // a reduced output this kernel is the first writer of starts from zero: here, or -- inside the
    // backward round loop, where every round adds to it -- once before the loop
    if (!c.in_round_loop && std::find(zero_first.begin(), zero_first.end(), name) != zero_first.end())
      check(cavs_zero(outs.back(), (size_t)cnt * 4, stream_));
  }
  if (n_elements == 0) return;
  check(cavs_fused_launch(h, outs.data(), (int)outs.size(), ins.data(), (int)ins.size(), oc.data(), ic.data(),
                          (int)n_elements, stream_));
}

// Pointer, element count and row width of an edge as seen by an op running in `c`.
float *Executor::view(const std::string &name, const RoundCtx &c, long *count, long *width) {
  Tensor &t = tensor(name);
  *width = t.width;
  if (!t.per_vertex) {
    *count = t.width;
    return t.base;
  }
  const Edge *e = edge(name);
  if (c.in_function && e && e->dynamic) {
    *count = c.n * t.width;
    return t.base + c.off * t.width;
  }
  *count = t.rows * t.width;
  return t.base;
}

void Executor::forward_needed(const std::vector<std::string> &targets, std::vector<const Node *> *order) {
  Graph &g = global_graph();
  std::set<const Node *> need;
  std::vector<const Node *> stack;
  for (auto &t : targets) {
    const Edge *e = g.main.find(t);
    if (!e) fail(CAVS_EINVAL, "unknown symbol '" + t + "'");
    stack.push_back(e->src);
  }
  while (!stack.empty()) {
    const Node *n = stack.back();
    stack.pop_back();
    if (!n || !need.insert(n).second) continue;
    for (Edge *e : n->in) stack.push_back(e->src);
    for (auto &a : n->after) {
      const Edge *e = g.main.find(a);
      if (e) stack.push_back(e->src);
    }
  }
  for (auto &n : g.main.nodes)
    if (need.count(n.get())) order->push_back(n.get());
}

// ------------------------------------------------------------------ one operator
namespace {
struct Shape2 {
  long rows, cols;
};
}  // namespace

void Executor::exec(const OpDef &d, const RoundCtx &c) {
  const std::string &op = d.name();
  auto acc = [&](int i) {
    auto *a = d.find_attr("Acc");
    return a && i < (int)a->value_.list_i.size() && a->value_.list_i[i] != 0;
  };
  // output tensor i with the geometry of its edge; per-vertex edges hold N_ rows
  auto out_tensor = [&](int i) -> Tensor & {
    const std::string &name = d.output(i);
    const Edge *e = edge(name);
    if (!e) fail(CAVS_EINVAL, "no edge for output '" + name + "' of " + op);
    auto &slot = tensors_[name];
    if (!slot) slot = std::make_unique<Tensor>();
    Tensor &t = *slot;
    t.width = e->width();
    t.per_vertex = e->per_vertex();
    if (t.per_vertex) t.rows = N_;
    return t;
  };
  auto alloc = [&](Tensor &t) {
    size_t need = t.count();
    if (t.own.capacity() < need) {
      check(cavs_stream_sync(stream_));
      t.own.reserve(need + need / 4);
    }
    t.base = t.own.get();
  };
  auto out_view = [&](int i, long *count, long *width) -> float * {
    Tensor &t = out_tensor(i);
    alloc(t);
    return view(d.output(i), c, count, width);
  };
  auto alias = [&](const std::string &src, long offset) {
    Tensor &s = tensor(src);
    Tensor &t = out_tensor(0);
    t.base = s.base + offset;
  };
  // stored 2-D geometry of an operand of MatMul
  auto mat = [&](const std::string &name, long count, long width) -> Shape2 {
    const Edge *e = edge(name);
    if (e && e->per_vertex()) return {count / width, width};
    if (e && e->shape.size() == 2) return {e->shape[0], e->shape[1]};
    return {1, count};
  };

  long n0, w0, n1, w1, no, wo;
  if (op == "Variable" || op == "Placeholder" || op == "ControlDependency") return;
  if (op == "FusedKernel") return exec_fused(d, c);
  if (op == "Mirror" || op == "Reshape" || op == "Flatten" || op == "Expand_dims") {
    alias(d.input(0), 0);  // ShareMemory: no copy (cavs/backend/op_impl_reshape.cc)
    return;
  }
  if (op == "Add" || op == "Sub" || op == "Mul" || op == "Equal") {
    const float *a = view(d.input(0), c, &n0, &w0), *b = view(d.input(1), c, &n1, &w1);
    float *o = out_view(0, &no, &wo);
    int code = op == "Add" ? CAVS_EW_ADD : op == "Sub" ? CAVS_EW_SUB : op == "Mul" ? CAVS_EW_MUL : CAVS_EW_EQUAL;
    if (no != std::max(n0, n1))  // only reachable as the gradient of a broadcast operand of Mul
      fail(CAVS_EUNSUPPORTED, op + ": reducing a product onto a broadcast operand is not implemented");
    check(cavs_ew_binary(code, o, a, n0, b, n1, no, acc(0), stream_));
    float scale = GetSingleArg<float>(d, "Scale", 1.f);
    if (scale != 1.f) {
      if (acc(0)) fail(CAVS_EUNSUPPORTED, "scaled product cannot accumulate");
      check(cavs_scale(o, o, scale, no, stream_));
    }
    return;
  }
  if (op == "Sigmoid" || op == "Tanh" || op == "Relu" || op == "Abs" || op == "Square") {
    const float *a = view(d.input(0), c, &n0, &w0);
    float *o = out_view(0, &no, &wo);
    int code = op == "Sigmoid" ? CAVS_EW_SIGMOID : op == "Tanh" ? CAVS_EW_TANH : op == "Relu" ? CAVS_EW_RELU
               : op == "Abs" ? CAVS_EW_ABS : CAVS_EW_SQUARE;
    check(cavs_ew_unary(code, o, a, n0, 0, stream_));
    return;
  }
  if (op == "Sigmoid_grad" || op == "Tanh_grad" || op == "Relu_grad") {  // (dy, y, x) -> dx
    const float *dy = view(d.input(0), c, &n0, &w0), *y = view(d.input(1), c, &n1, &w1);
    float *o = out_view(0, &no, &wo);
    int code = op == "Sigmoid_grad" ? CAVS_EW_SIGMOID_GRAD : op == "Tanh_grad" ? CAVS_EW_TANH_GRAD : CAVS_EW_RELU_GRAD;
    check(cavs_ew_binary(code, o, dy, n0, y, n1, no, acc(0), stream_));
    return;
  }
  if (op == "Assign" || op == "Neg" || op == "Accumulate" || op == "ReshapeLike") {
    const float *a = view(d.input(0), c, &n0, &w0);
    float *o = out_view(0, &no, &wo);
    if (no == n0) {
      check(cavs_ew_unary(op == "Neg" ? CAVS_EW_NEG : CAVS_EW_ASSIGN, o, a, n0, acc(0), stream_));
    } else if (no < n0 && n0 % no == 0) {
      // the operand was broadcast over the rows of the slab: its gradient is the column sum
      // (UnaryBroadcastingKernel, cavs/backend/op_impl_elementwise.cuh:24-34)
      if (op == "Neg") fail(CAVS_EUNSUPPORTED, "negated broadcast gradient is not implemented");
      check(cavs_colsum(o, a, (int)no, (int)(n0 / no), (int)no, acc(0), stream_));
    } else {
      fail(CAVS_EINVAL, op + ": cannot map " + std::to_string(n0) + " elements onto " + std::to_string(no));
    }
    return;
  }
  if (op == "Fill") {
    float *o = out_view(0, &no, &wo);
    if (d.input_size() == 2) {  // gradient of a reduction: broadcast of dy (op_decl_reduction.cc:19-28)
      const float *dy = view(d.input(1), c, &n1, &w1);
      if (acc(0)) fail(CAVS_EUNSUPPORTED, "Fill cannot accumulate");
      check(cavs_fill(o, 0.f, no, stream_));
      check(cavs_ew_binary(CAVS_EW_ADD, o, o, no, dy, 1, no, 0, stream_));
    } else {
      check(cavs_fill(o, GetSingleArg<float>(d, "Value", 0.f), no, stream_));
    }
    return;
  }
  if (op == "ConstOp") {
    float *o = out_view(0, &no, &wo);
    check(cavs_fill(o, GetSingleArg<float>(d, "init", 0.f), no, stream_));
    return;
  }
  if (op == "Slice" || op == "PartialAccumulate") {
    // forward: out = in[:, offset : offset+stride]; gradient: dIn[:, offset : ...] += dOut
    const std::string &wide_name = op == "Slice" ? d.input(0) : d.output(0);
    const Edge *we = edge(wide_name);
    long wide_w = we->width();
    long stride, offset;
    if (d.find_attr("Split")) {
      stride = wide_w / GetSingleArg<int>(d, "Split");
      offset = stride * GetSingleArg<int>(d, "Index");
    } else {
      offset = GetSingleArg<int>(d, "Offset");
      stride = GetSingleArg<int>(d, "Stride");
    }
    if (op == "Slice") {
      if (!we->per_vertex()) {  // contiguous block of a static tensor: a view
        alias(d.input(0), offset);
        return;
      }
      const float *a = view(d.input(0), c, &n0, &w0);
      float *o = out_view(0, &no, &wo);
      check(cavs_copy_rows(o, (int)stride, a + offset, (int)wide_w, (int)(n0 / wide_w), (int)stride, stream_));
    } else {
      const float *dy = view(d.input(0), c, &n0, &w0);
      float *o = out_view(0, &no, &wo);
      check(cavs_add_rows(o + offset, (int)wide_w, dy, (int)stride, (int)(no / wide_w), (int)stride, stream_));
    }
    return;
  }
  if (op == "Concat" || op == "SliceAll") {
    // Concat: out[:, block_i] = in_i ; SliceAll (its gradient): dIn_i = dOut[:, block_i]
    if (op == "Concat") {
      float *o = out_view(0, &no, &wo);
      long col = 0;
      for (int i = 0; i < d.input_size(); i++) {
        const float *a = view(d.input(i), c, &n0, &w0);
        check(cavs_copy_rows(o + col, (int)wo, a, (int)w0, (int)(n0 / w0), (int)w0, stream_));
        col += w0;
      }
    } else {
      const float *dy = view(d.input(0), c, &n0, &w0);
      long col = 0;
      for (int i = 0; i < d.output_size(); i++) {
        float *o = out_view(i, &no, &wo);
        if (acc(i))
          check(cavs_add_rows(o, (int)wo, dy + col, (int)w0, (int)(no / wo), (int)wo, stream_));
        else
          check(cavs_copy_rows(o, (int)wo, dy + col, (int)w0, (int)(no / wo), (int)wo, stream_));
        col += wo;
      }
    }
    return;
  }
  if (op == "MatMul") {
    const float *a = view(d.input(0), c, &n0, &w0), *b = view(d.input(1), c, &n1, &w1);
    float *o = out_view(0, &no, &wo);
    Shape2 sa = mat(d.input(0), n0, w0), sb = mat(d.input(1), n1, w1);
    int tA = 0, tB = 0;
    if (auto *t = d.find_attr("Transpose")) {
      tA = (int)t->value_.list_i[0];
      tB = (int)t->value_.list_i[1];
    }
    long M = tA ? sa.cols : sa.rows, K = tA ? sa.rows : sa.cols;
    long Kb = tB ? sb.cols : sb.rows, Nn = tB ? sb.rows : sb.cols;
    if (K != Kb || M * Nn != no)
      fail(CAVS_EINVAL, "MatMul shapes do not agree: " + d.DebugString());
    float *ws = workspace(cavs_sgemm_splitk_workspace((int)M, (int)Nn, (int)K));
    check(cavs_sgemm_splitk(tA, tB, (int)M, (int)Nn, (int)K, 1.f, a, (int)sa.cols, b, (int)sb.cols, acc(0) ? 1.f : 0.f, o,
                            (int)Nn, ws, ws_.capacity() * 4, stream_));
    return;
  }
  if (op == "EmbeddingLookup") {
    const float *ids = view(d.input(0), c, &n0, &w0), *table = view(d.input(1), c, &n1, &w1);
    float *o = out_view(0, &no, &wo);
    int E = edge(d.input(1))->shape[1];
    check(cavs_embed_fwd(o, E, ids, table, (int)n0, E, stream_));
    return;
  }
  if (op == "EmbeddingLookup_grad") {  // (dy, ids) -> dTable
    const float *dy = view(d.input(0), c, &n0, &w0), *ids = view(d.input(1), c, &n1, &w1);
    float *o = out_view(0, &no, &wo);
    int E = edge(d.output(0))->shape[1];
    if (!acc(0)) check(cavs_zero(o, (size_t)no * 4, stream_));
    check(cavs_embed_bwd(o, ids, dy, E, (int)n1, E, stream_));
    return;
  }
  if (op == "FullyConnected") {  // X[N,K] W[Out,K] B[1,Out]
    const float *x = view(d.input(0), c, &n0, &w0), *w = view(d.input(1), c, &n1, &w1);
    long nb, wb;
    const float *b = view(d.input(2), c, &nb, &wb);
    float *o = out_view(0, &no, &wo);
    int K = (int)w0, Nrow = (int)(n0 / w0), Out = (int)(n1 / K);
    float *ws = workspace(cavs_sgemm_splitk_workspace(Nrow, Out, K));
    check(cavs_sgemm_splitk(0, 1, Nrow, Out, K, 1.f, x, K, w, K, 0.f, o, Out, ws, ws_.capacity() * 4, stream_));
    check(cavs_bias_add_rows(o, o, b, Nrow, Out, stream_));
    return;
  }
  if (op == "FullyConnected_grad") {  // (dY, X, W, B) -> (dW, dB, dX)
    const float *dy = view(d.input(0), c, &n0, &w0), *x = view(d.input(1), c, &n1, &w1);
    long nw, ww;
    const float *w = view(d.input(2), c, &nw, &ww);
    int Out = (int)w0, Nrow = (int)(n0 / w0), K = (int)w1;
    long cnt, wd;
    float *dW = out_view(0, &cnt, &wd);
    float *ws = workspace(cavs_sgemm_splitk_workspace(Out, K, Nrow));
    check(cavs_sgemm_splitk(1, 0, Out, K, Nrow, 1.f, dy, Out, x, K, acc(0) ? 1.f : 0.f, dW, K, ws, ws_.capacity() * 4, stream_));
    float *dB = out_view(1, &cnt, &wd);
    check(cavs_colsum(dB, dy, Out, Nrow, Out, acc(1), stream_));
    float *dX = out_view(2, &cnt, &wd);
    ws = workspace(cavs_sgemm_splitk_workspace(Nrow, K, Out));
    check(cavs_sgemm_splitk(0, 0, Nrow, K, Out, 1.f, dy, Out, w, K, acc(2) ? 1.f : 0.f, dX, K, ws, ws_.capacity() * 4, stream_));
    return;
  }
  if (op == "SoftmaxEntropyLoss" || op == "SoftmaxEntropyLoss_grad") {
    const float *x = view(d.input(0), c, &n0, &w0), *lab = view(d.input(1), c, &n1, &w1);
    float *o = out_view(0, &no, &wo);
    int C = (int)w0, Nrow = (int)(n0 / w0);
    if (op == "SoftmaxEntropyLoss") {
      check(cavs_softmax_xent(o, nullptr, x, lab, Nrow, C, stream_));
    } else {
      if (acc(0)) fail(CAVS_EUNSUPPORTED, "SoftmaxEntropyLoss_grad cannot accumulate");
      check(cavs_softmax_xent(nullptr, o, x, lab, Nrow, C, stream_));
    }
    return;
  }
  if (op == "Reduce_sum" || op == "Reduce_mean") {
    // sum of absolute values (cublasSasum), cavs/backend/op_impl_blas1_cublas.cc:62-77
    const float *a = view(d.input(0), c, &n0, &w0);
    float *o = out_view(0, &no, &wo);
    float *tmp = workspace((size_t)n0 * 4 + 64);
    check(cavs_ew_unary(CAVS_EW_ABS, tmp, a, n0, 0, stream_));
    check(cavs_colsum(o, tmp, 1, (int)n0, 1, 0, stream_));
    if (op == "Reduce_mean") check(cavs_scale(o, o, 1.f / (float)n0, 1, stream_));
    return;
  }
  // ---- graph ops (cavs/backend/op_impl_graphop.cu) ----
  const bool backward = GetSingleArg<bool>(d, "Backward", false);
  if (op == "Gather") {
    float *o = out_view(0, &no, &wo);
    int child = GetSingleArg<int>(d, "Child", 0);
    if (!backward)
      check(cavs_gather_rows(o, (int)wo, pool_.get(), (int)pool_w_, d_child_[child] + c.off, (int)c.n, (int)wo, stream_));
    else  // gradient of Scatter: rows of the gradient pool through the recorded scatter list
      check(cavs_gather_rows(o, (int)wo, dpool_.get(), (int)pool_w_, d_pair_ + c.off, (int)c.n, (int)wo, stream_));
    return;
  }
  if (op == "Scatter") {
    const float *a = view(d.input(0), c, &n0, &w0);
    if (!backward) {
      check(cavs_scatter_rows(pool_.get(), (int)pool_w_, d_pair_ + c.off, a, (int)w0, (int)c.n, (int)w0, stream_));
    } else {  // gradient of Gather(child): rows to the children's gradient-pool rows
      int child = GetSingleArg<int>(d, "Child", 0);
      check(cavs_scatter_rows(dpool_.get(), (int)pool_w_, d_child_[child] + c.off, a, (int)w0, (int)c.n, (int)w0, stream_));
    }
    return;
  }
  if (op == "Pull") {
    float *o = out_view(0, &no, &wo);
    const float *src = backward ? dgo_ : func_arg_;
    if (!src) fail(CAVS_EINVAL, "Pull without a bound function argument");
    check(cavs_gather_rows(o, (int)wo, src, (int)wo, d_t2j_ + c.off, (int)c.n, (int)wo, stream_));
    return;
  }
  if (op == "Push") {
    if (backward) return;  // d vertex-input: never consumed
    const float *a = view(d.input(0), c, &n0, &w0);
    check(cavs_copy_rows(ret_.at(c.off * ret_w_), (int)ret_w_, a, (int)w0, (int)c.n, (int)w0, stream_));
    return;
  }
  fail(CAVS_EUNSUPPORTED, "operator '" + op + "' has no implementation on this path");
}

// ------------------------------------------------------------------ the vertex function
// One upload per step: t2j, the scatter/gather-back pairing list and one list per child.
void Executor::upload_lists() {
  const Schedule &s = sched_;
  const long N = N_;
  const size_t total = (size_t)N * 4;
  check(cavs_stream_sync(stream_));  // the staging buffer may still be in flight
  idx_host_.reserve(total);
  if (idx_dev_.capacity() < total) idx_dev_.reserve(total + total / 4);
  int *t2j = idx_host_.get(), *pair = t2j + N, *ch0 = pair + N, *ch1 = ch0 + N;
  std::memcpy(t2j, s.tids_to_jobids.data(), sizeof(int) * N);
  std::fill(pair, pair + 3 * N, -1);
  for (const Round &r : s.rounds) {
    const int m = r.scatter_end - r.scatter_begin;
    for (int b = 0; b < m; b++) {
      int tid = s.scatter_ids[r.scatter_begin + b];
      if (pairing_ == CAVS_PAIR_REFERENCE) pair[r.offset + b] = tid; else pair[tid] = tid;
    }
    int *ch[2] = {ch0, ch1};
    for (int cidx = 0; cidx < 2; cidx++) {
      const int len = r.gather_end[cidx] - r.gather_begin[cidx];
      if (len == 0) continue;
      if (len != r.n) fail(CAVS_EUNSUPPORTED, "a round mixes vertices with and without child " + std::to_string(cidx));
      for (int b = 0; b < len; b++) ch[cidx][r.offset + b] = s.gather_ids[cidx][r.gather_begin[cidx] + b];
    }
  }
  check(cavs_memcpy_h2d(idx_dev_.get(), idx_host_.get(), total * sizeof(int), stream_));
  d_t2j_ = idx_dev_.get();
  d_pair_ = d_t2j_ + N;
  d_child_[0] = d_pair_ + N;
  d_child_[1] = d_child_[0] + N;
}

// GraphStatement::Run, cavs/midend/statement.cc:43-85
void Executor::run_graph_output(const OpDef &d) {
  // the graph placeholder stays on the host (graph_scheduler.cc:15)
  Tensor &gt = tensor(d.input(0));
  const Edge *ge = edge(d.input(0));
  if (ge->shape.size() != 2) fail(CAVS_EINVAL, "the graph placeholder must be [batch, max vertices]");
  const int32_t *graph = reinterpret_cast<const int32_t *>(gt.base);
  auto &slot = tensors_[d.output(0)];
  if (!slot) slot = std::make_unique<Tensor>();
  Tensor &go = *slot;
  go.width = ret_w_;
  go.per_vertex = true;
  // the vertex placeholder may be left unfed when F never Pulls (apps/paper/tree-fc-cavs.cc:104)
  Tensor *arg = find_tensor(d.input(1));
  func_arg_ = arg ? arg->base : nullptr;
  if (lowered_) {  // the engine schedules, runs the fused rounds and owns GraphOutput
    lowered_forward(graph, ge->shape[0], ge->shape[1], nullptr);
    return;
  }
  std::string err = build_schedule(graph, ge->shape[0], ge->shape[1], (opt_ & OPT_BATCHING) != 0, &sched_);
  if (!err.empty()) fail(CAVS_EINVAL, "graph feed rejected: " + err);
  if (sched_.executed != sched_.N)
    fail(CAVS_EUNSUPPORTED, "the batch holds a single-vertex sample, which the reference never executes");
  N_ = sched_.N;
  go.rows = N_;
  if (go.own.capacity() < go.count()) {
    check(cavs_stream_sync(stream_));
    go.own.reserve(go.count() + go.count() / 4);
  }
  go.base = go.own.get();
  size_t need_pool = (size_t)N_ * pool_w_, need_ret = (size_t)N_ * ret_w_;
  if (pool_.capacity() < need_pool || ret_.capacity() < need_ret) {
    check(cavs_stream_sync(stream_));
    pool_.reserve(need_pool + need_pool / 4);
    dpool_.reserve(need_pool + need_pool / 4);
    ret_.reserve(need_ret + need_ret / 4);
  }
  upload_lists();
  for (const Round &r : sched_.rounds) {
    RoundCtx c{r.offset, r.n, true};
    for (const OpDef &fd : func_fwd_) exec(fd, c);
  }
  // FunctionPopRet: GraphOutput[tids_to_jobids[t]] = ret[t]
  check(cavs_scatter_rows(go.base, (int)ret_w_, d_t2j_, ret_.get(), (int)ret_w_, (int)N_, (int)ret_w_, stream_));
}

// GraphGradStatement::Run, cavs/midend/statement.cc:87-123
void Executor::run_graph_output_grad(const OpDef &d) {
  dgo_ = tensor(d.input(0)).base;
  if (lowered_) {
    lowered_backward(d);
    return;
  }
  // outputs the per-round generated kernels add every round's rows onto
  for (auto &name : round_zero_) {
    const Edge *e = edge(name);
    if (!e) fail(CAVS_EINVAL, "no edge for reduced output '" + name + "'");
    auto &slot = tensors_[name];
    if (!slot) slot = std::make_unique<Tensor>();
    Tensor &t = *slot;
    t.width = e->width();
    t.per_vertex = false;
    if (t.own.capacity() < t.count()) {
      check(cavs_stream_sync(stream_));
      t.own.reserve(t.count());
    }
    if (!t.base) t.base = t.own.get();
    check(cavs_zero(t.base, t.count() * 4, stream_));
  }
  for (int k : sched_.bwd_rounds) {
    const Round &r = sched_.rounds[k];
    RoundCtx c{r.offset, r.n, true, true};
    for (const OpDef &gd : func_bwd_) exec(gd, c);
  }
  RoundCtx all{0, N_, true};
  for (const OpDef &gd : func_def_) exec(gd, all);
}

// ------------------------------------------------------------------ Session::Run
void Executor::run(const std::vector<std::string> &outputs, std::vector<HostTensor *> *results,
                   const std::vector<std::pair<std::string, const HostTensor *>> &feeds) {
  Graph &g = global_graph();
  compile();
  init_variables();
  // feeds: the graph placeholder stays on the host, everything else goes to the device
  const int parity = run_parity_;
  run_parity_ ^= 1;
  if (run_busy_[parity]) {  // the Run before last read this set of feed buffers
    check(cavs_event_sync(run_done_ev_[parity]));
    run_busy_[parity] = false;
  }
  bool uploads = false;
  for (auto &f : feeds) {
    const Edge *e = g.main.find(f.first);
    if (!e || !e->src || e->src->def.name() != "Placeholder") fail(CAVS_EINVAL, "'" + f.first + "' is not a Placeholder");
    auto &slot = tensors_[f.first];
    if (!slot) slot = std::make_unique<Tensor>();
    Tensor &t = *slot;
    t.width = numel(e->shape);
    if (f.second->data.size() != (size_t)t.width * 4) fail(CAVS_EINVAL, "feed '" + f.first + "' has the wrong size");
    if (e->src->def.device() == CPU) {
      t.base = reinterpret_cast<float *>(const_cast<char *>(f.second->data.data()));
    } else {
      if (!copy_stream_) {
        check(cavs_stream_create(&copy_stream_));
        check(cavs_event_create(&feeds_up_ev_));
        check(cavs_event_create(&run_done_ev_[0]));
        check(cavs_event_create(&run_done_ev_[1]));
      }
      FeedStage &st = feed_stages_[f.first];
      const size_t bytes = (size_t)t.width * 4;
      // A placeholder the Run before this one did not feed still points at this set's buffer, and
      // that Run's kernels may be reading it: wait for them too (the usual case, a placeholder fed
      // by every Run, alternates between the sets and needs no such wait).
      if (t.base && t.base == st.dev[parity].get() && run_busy_[parity ^ 1]) {
        check(cavs_event_sync(run_done_ev_[parity ^ 1]));
        run_busy_[parity ^ 1] = false;
      }
      st.slot[parity].reserve(bytes);
      st.dev[parity].reserve(t.width);
      t.base = st.dev[parity].get();
      std::memcpy(st.slot[parity].get(), f.second->data.data(), bytes);
      check(cavs_memcpy_h2d(t.base, st.slot[parity].get(), bytes, copy_stream_));
      uploads = true;
    }
  }
  if (uploads) {
    // a few microseconds of waiting, while the compute stream is still busy with the previous Run
    check(cavs_event_record(feeds_up_ev_, copy_stream_));
    check(cavs_event_sync(feeds_up_ev_));
  }
  struct MarkRunDone {  // once everything this Run enqueues is in the stream, whichever way it leaves
    Executor *e;
    int parity;
    bool on;
    ~MarkRunDone() {
      if (on && cavs_event_record(e->run_done_ev_[parity], e->stream_) == CAVS_OK) e->run_busy_[parity] = true;
    }
  } mark_done{this, parity, copy_stream_ != nullptr};  // every Run, so that a later one can tell when this one's reads are over
  bool train = false;
  std::vector<std::string> targets;
  for (auto &o : outputs) {
    if (g.opt.present && o == g.opt.output) {
      train = true;
      targets.push_back(g.opt.loss);
    } else {
      targets.push_back(o);
    }
  }
  std::vector<const Node *> order;
  forward_needed(targets, &order);
  RoundCtx mainctx{0, 0, false};
  std::string key = train ? "T" : "F";
  for (auto &t : targets) key += "|" + t;
  auto it = main_cache_.find(key);
  if (it == main_cache_.end()) {
    MainProgram mp;
    for (const Node *n : order) mp.fwd.push_back(n->def);
    if (train) mp.bwd = g.opt.backward;
    if (opt_ & OPT_FUSION) {
      std::vector<OpDef> none, fwd, bwd;
      fwd = fused(mp.fwd, {&func_fwd_, &func_bwd_, &func_def_, train ? &g.opt.backward : &none}, targets);
      if (train) bwd = fused(mp.bwd, {&func_fwd_, &func_bwd_, &func_def_}, targets);
      mp.fwd.swap(fwd);
      mp.bwd.swap(bwd);
    }
    if (train && lowered_) {
      plan_gradient_binds(&mp);
      plan_fused_head(&mp);
    }
    it = main_cache_.emplace(key, std::move(mp)).first;
  }
  binds_ = &it->second.binds;
  const HeadFuse &head = it->second.head;
  // The optimizer's scope -- the replayed forward ops, the gradients and the update -- runs
  // `iters` times per Run (ScopedNode(s_, name, iters), cavs/midend/graph_util.cc:266-283;
  // BasicBlock::Run, cavs/midend/statement.h:66-75).
  const int passes = train ? std::max(1, g.opt.iters) : 1;
  // Launches that can ride in others when the lowered vertex function's backward pass follows in
  // this Run: the sum of the head's gradient partials (into the launch that opens that pass) and,
  // when nothing between that pass and the update reads them (no clipping, every later gradient op
  // planned away), the engine's pending bias gradients (into the launch that applies the updates).
  head_defer_ = defer_bias_ = false;
  if (train && lowered_) {
    int at = -1;
    const std::vector<char> &skip = it->second.skip_bwd;
    for (size_t i = 0; i < it->second.bwd.size(); i++)
      if (it->second.bwd[i].name() == "GraphOutput_grad") at = (int)i;
    if (at >= 0 && head.fc >= 0 && head.fc_grad >= 0 && head.fc_grad < at) head_defer_ = true;
    if (at >= 0 && g.opt.clip <= 0.f) {
      defer_bias_ = true;
      for (size_t i = at + 1; i < it->second.bwd.size(); i++)
        if (!(i < skip.size() && skip[i])) defer_bias_ = false;
    }
  }
  for (int pass = 0; pass < passes; pass++) {
  bool head_fused = false;
  for (size_t i = 0; i < it->second.fwd.size(); i++) {
    const OpDef &d = it->second.fwd[i];
    if ((int)i == head.fc) head_fused = run_fused_head(it->second);
    if (head_fused && ((int)i == head.fc || (int)i == head.loss)) continue;
    if (d.name() == "GraphOutput") run_graph_output(d); else exec(d, mainctx);
  }
  if (train) {
    const std::vector<char> &skip = it->second.skip_bwd;
    for (size_t i = 0; i < it->second.bwd.size(); i++) {
      const OpDef &d = it->second.bwd[i];
      if (i < skip.size() && skip[i]) continue;
      if (head_fused && ((int)i == head.loss_grad || (int)i == head.fc_grad || (int)i == head.seed)) continue;
      if (d.name() == "GraphOutput_grad") run_graph_output_grad(d); else exec(d, mainctx);
    }
    // SGD: w -= lr * g (cavs/backend/op_impl_sgd.cu); clipping is not on the measured path
    if (g.opt.clip > 0.f) {  // Clip precedes SGD (cavs/midend/graph_util.cc, op_impl_clip.cu)
      std::vector<float *> gp;
      std::vector<size_t> gn;
      for (auto &v : g.opt.vars) {
        Tensor &gr = tensor(GetGradientName(v));
        gp.push_back(gr.base);
        gn.push_back(gr.count());
      }
      const size_t bytes = cavs_clip_grads_workspace((int)gp.size());
      check(cavs_clip_grads((int)gp.size(), gp.data(), gn.data(), g.opt.clip, workspace(bytes), bytes, stream_));
    }
    // every variable's update in one launch (they touch disjoint tensors)
    std::vector<cavs_task> updates;
    std::vector<const float *> by_bias_job;
    // (the lowered F's launches over the rounds near the roots can give up: no update runs then)
    const int *guard = engine_ ? engine_->update_guard() : nullptr;
    const cavs_task guard_task{CAVS_TASK_GUARD, 0.f, 0, 0, 0, const_cast<int *>(guard), nullptr, nullptr, nullptr};
    if (guard) updates.push_back(guard_task);
    if (engine_ && defer_bias_) engine_->update_bias_jobs(g.opt.lr, &updates, &by_bias_job);
    for (auto &v : g.opt.vars) {
      Tensor &w = tensor(v), &gr = tensor(GetGradientName(v));
      if (std::find(by_bias_job.begin(), by_bias_job.end(), w.base) != by_bias_job.end()) continue;  // gradient and update by that job
      if (updates.size() + 2 > 12) {
        check(cavs_run_tasks((int)updates.size(), updates.data(), stream_));
        updates.clear();
        if (guard) updates.push_back(guard_task);
      }
      // the lowered F reads its recurrent weights from a packed copy that the update keeps current
      if (engine_ && engine_->update_jobs(w.base, gr.base, g.opt.lr, &updates)) continue;
      updates.push_back({CAVS_TASK_SGD, g.opt.lr, (long long)w.count(), 0, 0, w.base, gr.base, nullptr, nullptr});
    }
    check(cavs_run_tasks((int)updates.size(), updates.data(), stream_));
  }
  }  // passes
  results->assign(outputs.size(), nullptr);
  // A Run that asks for the optimizer only (the training loop of the reference's apps) has
  // nothing to hand back: it returns with the step still in flight, and the host prepares the
  // next batch meanwhile.  Whatever reads a value afterwards waits for the stream first.
  bool reads = false;
  for (auto &o : outputs)
    if (!(g.opt.present && o == g.opt.output)) reads = true;
  if (!reads) {
    dirty_ = true;
    return;
  }
  check(cavs_stream_sync(stream_));
  dirty_ = false;
  for (size_t i = 0; i < outputs.size(); i++) {
    if (g.opt.present && outputs[i] == g.opt.output) continue;
    Tensor &t = tensor(outputs[i]);
    auto *h = new HostTensor;
    h->name = outputs[i];
    h->data.resize(t.count() * 4);
    check(cavs_memcpy_d2h(h->data.data(), t.base, h->data.size(), stream_));
    (*results)[i] = h;
  }
  check(cavs_stream_sync(stream_));
  if (engine_) engine_->tail_check();
}

long Executor::read_tensor(const std::string &name, float *out, size_t cap) {
  Tensor *t = find_tensor(name);
  if (!t || !t->base) return 0;
  const Edge *e = edge(name);
  if (e && e->src && e->src->def.name() == "Placeholder" && e->src->def.device() == CPU) return 0;
  size_t n = t->count();
  if (!out || cap < n) return -(long)n;
  check(cavs_memcpy_d2h(out, t->base, n * 4, stream_));
  check(cavs_stream_sync(stream_));
  if (engine_) engine_->tail_check();
  return (long)n;
}

}  // namespace mid
}  // namespace cavs
