#include "lowering.h"

#include <algorithm>

#include <functional>
#include <set>
#include <sstream>

#include "cavs/frontend/cxx/graphsupport.h"
#include "cavs/frontend/cxx/sym.h"
#include "cell_gen.h"
#include "executor.h"

namespace cavs {
namespace mid {

namespace {

// Canonical text of the vertex function: the expressions feeding Scatter and Push, with
// aliasing ops made transparent, shared sub-expressions numbered in traversal order and
// external edges replaced by positional placeholders.
struct Canon {
  const Scope *func;
  std::map<std::string, int> memo;
  std::vector<const Edge *> ext;
  std::map<std::string, int> ext_id;

  static std::string shape_str(const Edge *e) {
    std::string s = "[";
    for (size_t i = 0; i < e->shape.size(); i++) s += (i ? "," : "") + std::to_string(e->shape[i]);
    return s + "]";
  }

  std::string expr(const Edge *e) {
    if (e->scope != func) {
      Resolved r = resolve_external(e);
      std::string key = r.ok ? r.var + "@" + std::to_string(r.offset) + "+" + std::to_string(r.count) : e->name;
      if (!ext_id.count(key)) {
        ext_id[key] = (int)ext.size();
        ext.push_back(e);
      }
      return "$" + std::to_string(ext_id[key]);
    }
    auto it = memo.find(e->name);
    if (it != memo.end()) return "#" + std::to_string(it->second);
    const Node *n = e->src;
    const OpDef &d = n->def;
    const std::string &op = d.name();
    if (op == "Mirror" || op == "Reshape" || op == "Flatten" || op == "Expand_dims") return expr(n->in[0]);
    std::string s;
    if (op == "Gather") {
      s = "Gather{" + std::to_string(GetSingleArg<int>(d, "Child", 0)) + "," + std::to_string(e->width()) + "}";
    } else if (op == "Pull") {
      s = "Pull{" + std::to_string(e->width()) + "}";
    } else if (op == "Slice") {
      long w = n->in[0]->width();
      long stride = d.find_attr("Split") ? w / GetSingleArg<int>(d, "Split") : GetSingleArg<int>(d, "Stride");
      long off = d.find_attr("Split") ? stride * GetSingleArg<int>(d, "Index") : GetSingleArg<int>(d, "Offset");
      s = "Slice{" + std::to_string(off) + "," + std::to_string(stride) + "}(" + expr(n->in[0]) + ")";
    } else if (op == "MatMul") {
      s = "MatMul(" + expr(n->in[0]) + "," + expr(n->in[1]) + ":" + shape_str(n->in[1]) + ")";
    } else {
      s = op + "(";
      for (size_t i = 0; i < n->in.size(); i++) s += (i ? "," : "") + expr(n->in[i]);
      s += ")";
    }
    int id = (int)memo.size();
    memo[e->name] = id;
    return "#" + std::to_string(id) + "=" + s;
  }

  std::string function() {
    std::string out;
    for (auto &n : func->nodes) {
      if (n->def.name() == "Scatter") out += "Scatter:" + expr(n->in[0]) + ";";
      if (n->def.name() == "Push") out += "Push:" + expr(n->in[0]) + ";";
    }
    return out;
  }
};

// ---- the recognised vertex functions, declared through the front end itself ----
struct TemplateDims {
  int V, E, H;
};

class TreeLstmT : public GraphSupport {
 public:
  TreeLstmT(const Sym &g, const Sym &v, TemplateDims d) : GraphSupport(g, v), E(d.E), H(d.H) {
    emb = Sym::Variable(DT_FLOAT, {d.V, E});
    W = Sym::Variable(DT_FLOAT, {4 * E * H});
    U = Sym::Variable(DT_FLOAT, {4 * H * H});
    B = Sym::Variable(DT_FLOAT, {4 * H});
    b_i = B.Slice(0, H); b_f = B.Slice(H, H); b_u = B.Slice(2 * H, H); b_o = B.Slice(3 * H, H);
    U_iou = U.Slice(0, 3 * H * H).Reshape({H, 3 * H});
    U_f = U.Slice(3 * H * H, H * H).Reshape({H, H});
  }
  void Node() override {
    Sym left = Gather(0, {2 * H}), right = Gather(1, {2 * H});
    Sym h_l, c_l, h_r, c_r;
    std::tie(h_l, c_l) = left.Split2();
    std::tie(h_r, c_r) = right.Split2();
    Sym h_lr = h_l + h_r;
    Sym x = Pull(0, {1}).EmbeddingLookup(emb);
    Sym xW = Sym::MatMul(x, W.Reshape({E, 4 * H}));
    Sym xW_i, xW_o, xW_u, xW_f;
    std::tie(xW_i, xW_o, xW_u, xW_f) = xW.Split4();
    Sym hU = Sym::MatMul(h_lr, U_iou);
    Sym hU_i, hU_o, hU_u;
    std::tie(hU_i, hU_o, hU_u) = hU.Split3();
    Sym hU_fl = Sym::MatMul(h_l, U_f), hU_fr = Sym::MatMul(h_r, U_f);
    Sym i = (xW_i + hU_i + b_i).Sigmoid();
    Sym o = (xW_o + hU_o + b_o).Sigmoid();
    Sym u = (xW_u + hU_u + b_u).Tanh();
    Sym f_l = (xW_f + hU_fl + b_f).Sigmoid();
    Sym f_r = (xW_f + hU_fr + b_f).Sigmoid();
    Sym c = i * u + f_l * c_l + f_r * c_r;
    Sym h = o * Sym::Tanh(c);
    Scatter(Sym::Concat({h, c}));
    Push(h);
  }
  Sym emb, W, U, B, b_i, b_f, b_u, b_o, U_iou, U_f;
  int E, H;
};

class SeqLstmT : public GraphSupport {
 public:
  SeqLstmT(const Sym &g, const Sym &v, TemplateDims d) : GraphSupport(g, v), H(d.H) {
    emb = Sym::Variable(DT_FLOAT, {d.V, H});
    Wv = Sym::Variable(DT_FLOAT, {8 * H * H});
    Bv = Sym::Variable(DT_FLOAT, {4 * H});
    Ux = Wv.Slice(0, 4 * H * H); Wh = Wv.Slice(4 * H * H, 4 * H * H);
    bi = Bv.Slice(0, H); bf = Bv.Slice(H, H); bu = Bv.Slice(2 * H, H); bo = Bv.Slice(3 * H, H);
  }
  void Node() override {
    Sym child = Gather(0, {2 * H});
    Sym ch, cc;
    std::tie(ch, cc) = child.Split2();
    Sym x = Pull(0, {1}).EmbeddingLookup(emb);
    Sym tmp = Sym::MatMul(x, Ux.Reshape({H, 4 * H})) + Sym::MatMul(ch.Expand_dims(0), Wh.Reshape({H, 4 * H}));
    Sym i, f, u, o;
    std::tie(i, f, u, o) = tmp.Split4();
    i = (i + bi).Sigmoid(); f = (f + bf).Sigmoid(); u = (u + bu).Tanh(); o = (o + bo).Sigmoid();
    Sym c = i * u + f * cc;
    Sym h = o * Sym::Tanh(c);
    Scatter(Sym::Concat({h, c}));
    Push(h);
  }
  Sym emb, Wv, Bv, Ux, Wh, bi, bf, bu, bo;
  int H;
};

class TreeFcT : public GraphSupport {
 public:
  TreeFcT(const Sym &g, const Sym &v, TemplateDims d, int variant) : GraphSupport(g, v), H(d.H), variant_(variant) {
    W = Sym::Variable(DT_FLOAT, {2 * H, H});
    if (variant_) Bv = Sym::Variable(DT_FLOAT, {H});
  }
  void Node() override {
    Sym left = Gather(0, {H}), right = Gather(1, {H});
    Sym fc = Sym::MatMul(Sym::Concat({left, right}).Reshape({1, 2 * H}), W);
    Sym res = variant_ ? (fc + Bv + Pull(0, {H})).Tanh() : fc.Relu();
    Scatter(res);
    Push(res);
  }
  Sym W, Bv;
  int H, variant_;
};

struct Template {
  std::string canon;
  std::vector<std::string> roles;  // role of the i-th external placeholder
};

// Declares a template in a scratch graph and canonicalises it.
Template make_template(int model, TemplateDims d, int variant) {
  Template t;
  Graph scratch;
  Graph *user = swap_global_graph(&scratch);
  try {
    Sym g = Sym::Placeholder(DT_FLOAT, {2, 4}, "CPU");
    Sym v = Sym::Placeholder(DT_FLOAT, {2, 4});
    std::map<std::string, std::string> role_of;  // "var@offset" -> role
    std::unique_ptr<GraphSupport> gs;
    auto key = [](const Sym &var, long off) { return var.output(0) + "@" + std::to_string(off); };
    const long H = d.H;
    if (model == CAVS_MODEL_TREELSTM) {
      auto *m = new TreeLstmT(g, v, d);
      gs.reset(m);
      role_of[key(m->emb, 0)] = "Emb";
      role_of[key(m->W, 0)] = "W";
      role_of[key(m->U, 0)] = "U_iou";
      role_of[key(m->U, 3 * H * H)] = "U_f";
      role_of[key(m->B, 0)] = "b_i"; role_of[key(m->B, H)] = "b_f";
      role_of[key(m->B, 2 * H)] = "b_u"; role_of[key(m->B, 3 * H)] = "b_o";
    } else if (model == CAVS_MODEL_LSTM) {
      auto *m = new SeqLstmT(g, v, d);
      gs.reset(m);
      role_of[key(m->emb, 0)] = "Emb";
      role_of[key(m->Wv, 0)] = "Ux"; role_of[key(m->Wv, 4 * H * H)] = "Wh";
      role_of[key(m->Bv, 0)] = "b_i"; role_of[key(m->Bv, H)] = "b_f";
      role_of[key(m->Bv, 2 * H)] = "b_u"; role_of[key(m->Bv, 3 * H)] = "b_o";
    } else {
      auto *m = new TreeFcT(g, v, d, variant);
      gs.reset(m);
      role_of[key(m->W, 0)] = "W";
      if (variant) role_of[key(m->Bv, 0)] = "Bv";
    }
    gs->Output();
    Canon c;
    c.func = scratch.func.get();
    t.canon = c.function();
    for (const Edge *e : c.ext) {
      Resolved r = resolve_external(e);
      t.roles.push_back(role_of[r.var + "@" + std::to_string(r.offset)]);
    }
  } catch (...) {
    swap_global_graph(user);
    throw;
  }
  swap_global_graph(user);
  return t;
}

struct RoleSlot {
  const char *param;  // engine parameter
  long offset;        // element offset inside it (in units given by the lambdas below)
};

}  // namespace

namespace {
std::unique_ptr<Lowering> match_template(const Graph &g);
}

std::unique_ptr<Lowering> match_vertex_function(const Graph &g, int mode) {
  if (!g.func) return nullptr;
  if (mode == 1) {
    auto lw = match_template(g);
    if (lw) return lw;
  }
  std::unique_ptr<CellMatch> m = match_cell(g);
  if (!m) return nullptr;
  auto lw = std::make_unique<Lowering>();
  lw->model = CAVS_MODEL_CELL;
  lw->H = m->spec->H;
  lw->E = m->spec->E;
  lw->V = m->spec->V;
  lw->use_x = m->spec->NX > 0 || m->spec->XD > 0;
  lw->roles = m->roles;
  lw->cell = m->spec;
  lw->cell_slots = m->slots;
  return lw;
}

namespace {
std::unique_ptr<Lowering> match_template(const Graph &g) {
  if (!g.func) return nullptr;
  // cheap signature first: graph ops and the embedding table decide which template to try
  int gathers = 0, pulls = 0;
  long pool_w = 0, ret_w = 0, pull_w = 0;
  const Edge *table = nullptr;
  for (auto &n : g.func->nodes) {
    const std::string &op = n->def.name();
    if (op == "Gather") { gathers++; pool_w = n->out[0]->width(); }
    if (op == "Pull") { pulls++; pull_w = n->out[0]->width(); }
    if (op == "Push") ret_w = n->in[0]->width();
    if (op == "EmbeddingLookup") table = n->in[1];
  }
  int model, variant = 0;
  TemplateDims d{0, 0, (int)ret_w};
  if (table) {
    if (table->shape.size() != 2 || pool_w != 2 * ret_w) return nullptr;
    d.V = table->shape[0];
    d.E = table->shape[1];
    model = gathers == 2 ? CAVS_MODEL_TREELSTM : CAVS_MODEL_LSTM;
    if (model == CAVS_MODEL_LSTM && d.E != d.H) return nullptr;
  } else {
    if (gathers != 2 || pool_w != ret_w) return nullptr;
    model = CAVS_MODEL_TREEFC;
    variant = pulls ? 1 : 0;
    if (variant && pull_w != ret_w) return nullptr;
  }
  Template t = make_template(model, d, variant);
  Canon c;
  c.func = g.func.get();
  if (c.function() != t.canon || c.ext.size() != t.roles.size()) return nullptr;
  auto lw = std::make_unique<Lowering>();
  lw->model = model;
  lw->H = d.H;
  lw->E = d.E;
  lw->V = d.V;
  lw->act = variant;
  lw->use_bias = variant;
  lw->use_x = variant;
  std::map<std::string, Resolved> where;
  for (size_t i = 0; i < c.ext.size(); i++) {
    Resolved r = resolve_external(c.ext[i]);
    if (!r.ok) return nullptr;  // an external input that is not a view of a Variable
    lw->roles[t.roles[i]] = c.ext[i]->name;
    where[t.roles[i]] = r;
  }
  // the fused kernels read U_iou|U_f, the two LSTM weight blocks and the four bias blocks
  // as one contiguous array each: the user's views must be laid out that way
  const long H = d.H;
  auto follows = [&](const char *a, const char *b, long gap) {
    return where[a].var == where[b].var && where[b].offset == where[a].offset + gap;
  };
  if (model != CAVS_MODEL_TREEFC &&
      !(follows("b_i", "b_f", H) && follows("b_f", "b_u", H) && follows("b_u", "b_o", H)))
    return nullptr;
  if (model == CAVS_MODEL_TREELSTM && !follows("U_iou", "U_f", 3 * H * H)) return nullptr;
  if (model == CAVS_MODEL_LSTM && !follows("Ux", "Wh", 4 * H * H)) return nullptr;
  return lw;
}

}  // namespace

// ------------------------------------------------------------------ running the lowered F
namespace {
struct Slot {
  const char *param;
  long offset, count;
};
std::map<std::string, Slot> role_slots(const Lowering &lw) {
  const long H = lw.H, E = lw.E, V = lw.V;
  std::map<std::string, Slot> m;
  if (lw.model == CAVS_MODEL_CELL) {
    for (auto &kv : lw.cell_slots) m[kv.first] = {kv.second.param.c_str(), kv.second.offset, kv.second.count};
    return m;
  }
  if (lw.model == CAVS_MODEL_TREELSTM) {
    m["Emb"] = {"Emb", 0, V * E};
    m["W"] = {"W", 0, 4 * E * H};
    m["U_iou"] = {"U", 0, 3 * H * H};
    m["U_f"] = {"U", 3 * H * H, H * H};
  } else if (lw.model == CAVS_MODEL_LSTM) {
    m["Emb"] = {"Emb", 0, V * H};
    m["Ux"] = {"W", 0, 4 * H * H};
    m["Wh"] = {"W", 4 * H * H, 4 * H * H};
  } else {
    m["W"] = {"W", 0, 2 * H * H};
    if (lw.use_bias) m["Bv"] = {"Bv", 0, H};
  }
  if (lw.model != CAVS_MODEL_TREEFC) {
    m["b_i"] = {"Bv", 0, H};
    m["b_f"] = {"Bv", H, H};
    m["b_u"] = {"Bv", 2 * H, H};
    m["b_o"] = {"Bv", 3 * H, H};
  }
  return m;
}
}  // namespace

int Executor::fused_path_kind() const { return !lowered_ ? 0 : lowering_->model == CAVS_MODEL_CELL ? 2 : 1; }

void Executor::lowered_forward(const int32_t *graph, int B, int maxlen, float *) {
  const Lowering &lw = *lowering_;
  if (!engine_) {
    cavs_session_config cfg{};
    cfg.model = lw.model;
    cfg.loss = CAVS_LOSS_SUM_ABS;  // the loss head stays in the main scope
    cfg.opt = opt_;
    cfg.V = lw.V;
    cfg.E = lw.E;
    cfg.H = lw.H;
    cfg.act = lw.act;
    cfg.use_bias = lw.use_bias;
    cfg.use_x = lw.use_x;
    cfg.split_backward_rounds = lowering_mode_ == 3;
    engine_ = std::make_unique<Engine>(cfg, stream_, lw.cell);
  }
  engine_->set_pairing(pairing_);
  // parameters live in the user's Variable tensors; the engine reads them in place
  std::set<std::string> bound;
  for (auto &kv : role_slots(lw)) {
    const Slot &s = kv.second;
    if (!bound.insert(s.param).second) continue;  // every view of an array leads to its base address
    Tensor &t = tensor(lw.roles.at(kv.first));
    engine_->bind_param(s.param, t.base - s.offset, nullptr);
  }
  engine_->forward_only(graph, B, maxlen, func_arg_, nullptr);
  N_ = engine_->total_length();
  Tensor &go = tensor(global_graph().graph_output);
  go.base = engine_->graph_out_ptr();
  go.rows = N_;
}

// See GradBind.  A PartialAccumulate qualifies when what it adds is an output of the lowered F
// that is written, not accumulated (possibly through ReshapeLike views); a Variable qualifies
// when its gradient is written by one zero Fill and qualifying PartialAccumulates only, whose
// blocks tile it and line up with the engine's layout of whole parameters.
void Executor::plan_gradient_binds(MainProgram *mp) const {
  const Lowering &lw = *lowering_;
  const std::vector<OpDef> &ops = mp->bwd;
  mp->skip_bwd.assign(ops.size(), 0);
  mp->binds.clear();
  int gi = -1;
  for (size_t i = 0; i < ops.size(); i++)
    if (ops[i].name() == "GraphOutput_grad") gi = (int)i;
  if (gi < 0) return;
  const OpDef &go = ops[gi];
  auto slots = role_slots(lw);
  std::map<std::string, std::string> role_of_edge;
  for (auto &kv : lw.roles) role_of_edge[kv.second] = kv.first;
  std::map<std::string, std::string> role_of_grad;  // written (not accumulated) outputs of the lowered F
  auto *accs = go.find_attr("Acc");
  for (int i = 0; i < go.output_size(); i++) {
    const bool acc = accs && i < (int)accs->value_.list_i.size() && accs->value_.list_i[i] != 0;
    auto rit = role_of_edge.find(GetOriginName(go.output(i)));
    if (!acc && rit != role_of_edge.end()) role_of_grad[go.output(i)] = rit->second;
  }
  std::map<std::string, int> producer;
  std::map<std::string, std::vector<int>> writers;
  for (size_t i = 0; i < ops.size(); i++)
    for (int k = 0; k < ops[i].output_size(); k++) {
      producer[ops[i].output(k)] = (int)i;
      writers[ops[i].output(k)].push_back((int)i);
    }
  struct Block {
    int op;
    std::string role;
    long offset, stride;
    std::vector<int> views;  // the ReshapeLike operators between the lowered F's output and the block
  };
  std::map<std::string, std::vector<Block>> blocks;  // by destination
  std::map<std::string, bool> bad;
  for (size_t i = gi + 1; i < ops.size(); i++) {
    const OpDef &d = ops[i];
    if (d.name() != "PartialAccumulate") continue;
    const std::string &dst = d.output(0);
    const Edge *we = edge(dst);
    if (!we || we->per_vertex()) { bad[dst] = true; continue; }
    long stride, offset;
    if (d.find_attr("Split")) {
      stride = we->width() / GetSingleArg<int>(d, "Split");
      offset = stride * GetSingleArg<int>(d, "Index");
    } else {
      offset = GetSingleArg<int>(d, "Offset");
      stride = GetSingleArg<int>(d, "Stride");
    }
    std::string src = d.input(0);
    std::vector<int> views;
    for (int hops = 0; hops < 8 && !role_of_grad.count(src); hops++) {
      auto pit = producer.find(src);
      if (pit == producer.end() || pit->second <= gi || ops[pit->second].name() != "ReshapeLike") break;
      views.push_back(pit->second);
      src = ops[pit->second].input(0);
    }
    auto rit = role_of_grad.find(src);
    if (rit == role_of_grad.end()) { bad[dst] = true; continue; }
    blocks[dst].push_back({(int)i, rit->second, offset, stride, views});
  }
  for (auto &kv : blocks) {
    const std::string &dst = kv.first;
    std::vector<Block> &bl = kv.second;
    if (bad[dst]) continue;
    const Edge *we = edge(dst);
    // writers: one Fill with zero, then the blocks
    int fill = -1;
    bool ok = true;
    for (int w : writers[dst]) {
      const OpDef &d = ops[w];
      if (d.name() == "Fill" && d.input_size() == 1 && GetSingleArg<float>(d, "Value", 0.f) == 0.f && fill < 0) fill = w;
      else if (d.name() != "PartialAccumulate") ok = false;
    }
    if (!ok || fill < 0 || fill > bl.front().op) continue;
    // the blocks tile the Variable
    std::sort(bl.begin(), bl.end(), [](const Block &a, const Block &b) { return a.offset < b.offset; });
    long at = 0;
    for (const Block &b : bl) {
      if (b.offset != at) ok = false;
      at += b.stride;
    }
    if (!ok || at != we->width()) continue;
    // and are whole engine parameters in the engine's layout
    std::map<std::string, long> base;    // param -> offset of its gradient inside dst
    std::map<std::string, long> covered; // param -> elements covered
    for (const Block &b : bl) {
      const Slot &s = slots.at(b.role);
      if (b.stride != s.count) ok = false;
      const long off = b.offset - s.offset;
      if (base.count(s.param) && base[s.param] != off) ok = false;
      base[s.param] = off;
      covered[s.param] += s.count;
    }
    for (auto &pv : covered) {
      long total = 0;
      for (auto &sv : slots)
        if (pv.first == sv.second.param) total += sv.second.count;
      if (total != pv.second) ok = false;  // a slice of the parameter goes somewhere else
    }
    if (!ok) continue;
    mp->skip_bwd[fill] = 1;
    for (const Block &b : bl) {
      mp->skip_bwd[b.op] = 1;
      // a copy whose only readers are skipped is dead too (nearest to the block first)
      for (int v : b.views) {
        bool read = false;
        for (size_t i = 0; i < ops.size(); i++) {
          if (mp->skip_bwd[i]) continue;
          for (int k = 0; k < ops[i].input_size(); k++) read |= ops[i].input(k) == ops[v].output(0);
        }
        if (read) break;
        mp->skip_bwd[v] = 1;
      }
    }
    for (auto &pv : base) mp->binds.push_back({pv.first, dst, pv.second});
  }
}

// See HeadFuse.
void Executor::plan_fused_head(MainProgram *mp) const {
  HeadFuse h;
  const std::vector<OpDef> &fwd = mp->fwd, &bwd = mp->bwd;
  auto no_acc = [](const OpDef &d) {
    auto *a = d.find_attr("Acc");
    if (a)
      for (int v : a->value_.list_i)
        if (v) return false;
    return true;
  };
  for (size_t i = 0; i < fwd.size() && h.loss < 0; i++) {
    if (fwd[i].name() != "SoftmaxEntropyLoss") continue;
    for (size_t k = 0; k < i; k++)
      if (fwd[k].name() == "FullyConnected" && fwd[k].output(0) == fwd[i].input(0)) {
        h.fc = (int)k;
        h.loss = (int)i;
      }
  }
  if (h.loss < 0) return;
  const OpDef &fc = fwd[h.fc], &loss = fwd[h.loss];
  // the labels must exist when the FullyConnected operator runs
  for (size_t k = h.fc; k < fwd.size(); k++)
    for (int o = 0; o < fwd[k].output_size(); o++)
      if (fwd[k].output(o) == loss.input(1)) return;
  for (size_t i = 0; i < bwd.size(); i++) {
    const OpDef &d = bwd[i];
    if (d.name() == "SoftmaxEntropyLoss_grad" && d.input(0) == fc.output(0) && d.input(1) == loss.input(1)) h.loss_grad = (int)i;
  }
  if (h.loss_grad < 0) return;
  const std::string &dy = bwd[h.loss_grad].output(0);
  for (size_t i = 0; i < bwd.size(); i++) {
    const OpDef &d = bwd[i];
    bool reads = false;
    for (int k = 0; k < d.input_size(); k++) reads |= d.input(k) == dy;
    if (!reads) continue;
    if (d.name() != "FullyConnected_grad" || h.fc_grad >= 0 || d.input(0) != dy || d.input(1) != fc.input(0) ||
        d.input(2) != fc.input(1))
      return;  // someone else wants d logits
    h.fc_grad = (int)i;
  }
  if (h.fc_grad < 0 || !no_acc(bwd[h.fc_grad]) || !no_acc(bwd[h.loss_grad])) return;
  for (size_t i = 0; i < bwd.size(); i++) {  // the seed of d loss: SoftmaxEntropyLoss_grad does not read it
    if (bwd[i].name() != "ConstOp" || bwd[i].output(0) != GetGradientName(loss.output(0))) continue;
    bool read = false;
    for (auto &d : bwd)
      for (int k = 0; k < d.input_size(); k++) read |= d.input(k) == bwd[i].output(0);
    if (!read) h.seed = (int)i;
  }
  mp->head = h;
}

float *Executor::output_storage(const std::string &name, long *count) {
  const Edge *e = edge(name);
  if (!e) fail(CAVS_EINVAL, "no edge for '" + name + "'");
  auto &slot = tensors_[name];
  if (!slot) slot = std::make_unique<Tensor>();
  Tensor &t = *slot;
  t.width = e->width();
  t.per_vertex = e->per_vertex();
  if (t.per_vertex) t.rows = N_;
  const size_t need = t.count();
  if (t.own.capacity() < need) {
    check(cavs_stream_sync(stream_));
    t.own.reserve(need + need / 4);
  }
  t.base = t.own.get();
  if (count) *count = (long)need;
  return t.base;
}

// Returns false (and does nothing) when the shape of this batch is not one the fused entry point takes.
bool Executor::run_fused_head(const MainProgram &mp) {
  const HeadFuse &h = mp.head;
  if (h.fc < 0) return false;
  const OpDef &fc = mp.fwd[h.fc], &loss = mp.fwd[h.loss], &fg = mp.bwd[h.fc_grad];
  RoundCtx c{0, 0, false};
  long n0, w0, n1, w1, nb, wb, nl, wl;
  const float *x = view(fc.input(0), c, &n0, &w0), *w = view(fc.input(1), c, &n1, &w1);
  const float *b = view(fc.input(2), c, &nb, &wb), *lab = view(loss.input(1), c, &nl, &wl);
  const int K = (int)w0, Nrow = (int)(n0 / w0), C = (int)(n1 / K);
  const size_t bytes = cavs_fc_softmax_xent_workspace(Nrow, K, C);
  if (bytes == 0 || nb != C || nl != Nrow) return false;
  long cnt;
  float *logits = output_storage(fc.output(0), &cnt);
  float *lo = output_storage(loss.output(0), &cnt);
  if (cnt != Nrow) return false;
  float *dW = output_storage(fg.output(0), &cnt);
  float *dB = output_storage(fg.output(1), &cnt);
  float *dX = output_storage(fg.output(2), &cnt);
  // The weight and bias gradients come out as partial sums.  With the engine's backward pass
  // following in this Run, adding them up is a job of the launch that opens that pass (one launch
  // less); the partials then live in a buffer of their own until it has run.
  if (engine_ && head_defer_) {
    if (head_parts_.capacity() * 4 < bytes) {
      check(cavs_stream_sync(stream_));
      head_parts_.reserve(bytes / 4 + 1);
    }
    check(cavs_fc_softmax_xent(x, w, b, lab, lo, logits, dX, nullptr, nullptr, head_parts_.get(), head_parts_.capacity() * 4, Nrow, K,
                               C, stream_));
    engine_->queue_prologue_task({CAVS_TASK_SUM_PARTS, 0.f, cavs_fc_softmax_xent_parts(Nrow), (long long)C * K + C, (long long)C * K,
                                  head_parts_.get(), dW, dB, nullptr});
    return true;
  }
  float *ws = workspace(bytes);
  check(cavs_fc_softmax_xent(x, w, b, lab, lo, logits, dX, dW, dB, ws, ws_.capacity() * 4, Nrow, K, C, stream_));
  return true;
}

void Executor::lowered_backward(const OpDef &d) {
  const Lowering &lw = *lowering_;
  if (binds_) {
    for (const GradBind &b : *binds_) {
      const Edge *e = edge(b.dst);
      auto &slot = tensors_[b.dst];
      if (!slot) slot = std::make_unique<Tensor>();
      Tensor &t = *slot;
      t.width = e->width();
      t.per_vertex = false;
      if (t.own.capacity() < (size_t)t.width) {
        check(cavs_stream_sync(stream_));
        t.own.reserve(t.width);
      }
      t.base = t.own.get();
      engine_->bind_param_grad(b.param, t.base + b.offset);
    }
  }
  engine_->backward_only(dgo_, !defer_bias_);
  // hand the gradients of the external edges to the main-scope backward program
  auto slots = role_slots(lw);
  std::map<std::string, std::string> role_of_edge;
  for (auto &kv : lw.roles) role_of_edge[kv.second] = kv.first;
  auto *accs = d.find_attr("Acc");
  for (int i = 0; i < d.output_size(); i++) {
    const std::string &gname = d.output(i);
    auto rit = role_of_edge.find(GetOriginName(gname));
    if (rit == role_of_edge.end()) fail(CAVS_EINVAL, "no lowered gradient for " + gname);
    const Slot &s = slots.at(rit->second);
    const Edge *e = edge(gname);
    auto &slot = tensors_[gname];
    if (!slot) slot = std::make_unique<Tensor>();
    Tensor &t = *slot;
    t.width = e->width();
    t.per_vertex = false;
    bool acc = accs && i < (int)accs->value_.list_i.size() && accs->value_.list_i[i] != 0;
    float *src = const_cast<float *>(engine_->grad_ptr(s.param)) + s.offset;
    if (!acc) {
      // a view of the engine's gradient array: it stays valid until the next backward pass, and
      // whoever consumes it in the main scope reads it in this Run
      t.base = src;
      continue;
    }
    if (t.own.capacity() < (size_t)t.width) {
      check(cavs_stream_sync(stream_));
      t.own.reserve(t.width);
    }
    t.base = t.own.get();  // zeroed at the start of the pass like every accumulating output
    check(cavs_ew_unary(CAVS_EW_ASSIGN, t.base, src, (size_t)s.count, 1, stream_));
  }
}

}  // namespace mid
}  // namespace cavs
