// The three vertex functions of the reference's benchmark applications, written against
// the front end exactly as a user would (apps/paper/tree-lstm-cavs.cc:106-184,
// seq-lstm-cavs.cc:43-95, tree-fc-cavs.cc:21-40), plus an extern "C" harness so that the
// tests and the benchmark can drive them from Python.  Every tensor that is consumed
// more than once inside F goes through Mirror(), which is what makes the reference's own
// gradient rules accumulate instead of overwrite.
#include <cstring>
#include <memory>
#include <string>
#include <vector>

#include "cavs/frontend/cxx/graphsupport.h"
#include "cavs/frontend/cxx/session.h"
#include "cavs/frontend/cxx/sym.h"

using std::tie;
using std::vector;

namespace {

struct Dims {
  int B, maxlen, V, E, H, C;
};

class TreeLSTM : public GraphSupport {
 public:
  TreeLSTM(const Sym &graph_ph, const Sym &vertex_ph, const Dims &d) : GraphSupport(graph_ph, vertex_ph), E(d.E), H(d.H) {
    embedding = Sym::Variable(DT_FLOAT, {d.V, E}, Sym::Uniform(-0.1f, 0.1f));
    W = Sym::Variable(DT_FLOAT, {4 * E * H}, Sym::Uniform(-0.1f, 0.1f));
    U = Sym::Variable(DT_FLOAT, {4 * H * H}, Sym::Uniform(-0.1f, 0.1f));
    B = Sym::Variable(DT_FLOAT, {4 * H}, Sym::Zeros());
    b_i = B.Slice(0, H);
    b_f = B.Slice(H, H);
    b_u = B.Slice(2 * H, H);
    b_o = B.Slice(3 * H, H);
    U_iou = U.Slice(0, 3 * H * H).Reshape({H, 3 * H});
    U_f = U.Slice(3 * H * H, H * H).Reshape({H, H});
  }
  void Node() override {
    Sym left = Gather(0, {2 * H});
    Sym right = Gather(1, {2 * H});
    Sym h_l, c_l, h_r, c_r;
    tie(h_l, c_l) = left.Split2();
    tie(h_r, c_r) = right.Split2();
    Sym h_lr = h_l.Mirror() + h_r.Mirror();

    Sym x = Pull(0, {1});
    x = x.EmbeddingLookup(embedding.Mirror());
    Sym xW = Sym::MatMul(x, W.Reshape({E, 4 * H}).Mirror()).Reshape({H * 4});
    Sym xW_i, xW_o, xW_u, xW_f;
    tie(xW_i, xW_o, xW_u, xW_f) = xW.Split4();

    Sym hU_iou = Sym::MatMul(h_lr.Reshape({1, H}), U_iou.Mirror()).Reshape({H * 3});
    Sym hU_i, hU_o, hU_u;
    tie(hU_i, hU_o, hU_u) = hU_iou.Split3();
    Sym hU_fl = Sym::MatMul(h_l.Mirror().Reshape({1, H}), U_f.Mirror()).Reshape({H});
    Sym hU_fr = Sym::MatMul(h_r.Mirror().Reshape({1, H}), U_f.Mirror()).Reshape({H});

    Sym i = (xW_i + hU_i + b_i.Mirror()).Sigmoid();
    Sym o = (xW_o + hU_o + b_o.Mirror()).Sigmoid();
    Sym u = (xW_u + hU_u + b_u.Mirror()).Tanh();
    Sym f_l = (xW_f.Mirror() + hU_fl + b_f.Mirror()).Sigmoid();
    Sym f_r = (xW_f.Mirror() + hU_fr + b_f.Mirror()).Sigmoid();

    Sym c = i * u + f_l * c_l + f_r * c_r;
    Sym h = o * Sym::Tanh(c.Mirror());
    Scatter(Sym::Concat({h.Mirror(), c.Mirror()}));
    Push(h.Mirror());
  }
  Sym embedding, W, U, B;

 private:
  int E, H;
  Sym b_i, b_f, b_u, b_o, U_iou, U_f;
};

// A binary Tree-LSTM whose forget gates have a recurrent matrix per child (f_l = sigmoid(x W_f +
// h_l U_fl + b_f), f_r likewise with U_fr), with the gates' biases in the order of their columns:
// not one of the reference's applications -- a vertex function a user might write, which the
// hand-written round kernels do not cover.  U holds [U_iou (H x 3H) | U_fl (H x H) | U_fr (H x H)].
class TreeLSTM2 : public GraphSupport {
 public:
  TreeLSTM2(const Sym &graph_ph, const Sym &vertex_ph, const Dims &d) : GraphSupport(graph_ph, vertex_ph), E(d.E), H(d.H) {
    embedding = Sym::Variable(DT_FLOAT, {d.V, E}, Sym::Uniform(-0.1f, 0.1f));
    W = Sym::Variable(DT_FLOAT, {4 * E * H}, Sym::Uniform(-0.1f, 0.1f));
    U = Sym::Variable(DT_FLOAT, {5 * H * H}, Sym::Uniform(-0.1f, 0.1f));
    B = Sym::Variable(DT_FLOAT, {4 * H}, Sym::Zeros());
    b_iou = B.Slice(0, 3 * H);
    b_f = B.Slice(3 * H, H);
    U_iou = U.Slice(0, 3 * H * H).Reshape({H, 3 * H});
    U_fl = U.Slice(3 * H * H, H * H).Reshape({H, H});
    U_fr = U.Slice(4 * H * H, H * H).Reshape({H, H});
  }
  void Node() override {
    Sym left = Gather(0, {2 * H});
    Sym right = Gather(1, {2 * H});
    Sym h_l, c_l, h_r, c_r;
    tie(h_l, c_l) = left.Split2();
    tie(h_r, c_r) = right.Split2();
    Sym h_lr = h_l.Mirror() + h_r.Mirror();
    Sym x = Pull(0, {1});
    x = x.EmbeddingLookup(embedding.Mirror());
    Sym xW = Sym::MatMul(x, W.Reshape({E, 4 * H}).Mirror()).Reshape({H * 4});
    Sym xW_iou = xW.Slice(0, 3 * H);
    Sym xW_f = xW.Slice(3 * H, H);
    Sym iou = xW_iou + Sym::MatMul(h_lr.Reshape({1, H}), U_iou.Mirror()).Reshape({H * 3}) + b_iou.Mirror();
    Sym gi, go, gu;
    tie(gi, go, gu) = iou.Split3();
    Sym i = gi.Sigmoid(), o = go.Sigmoid(), u = gu.Tanh();
    Sym f_l = (xW_f.Mirror() + Sym::MatMul(h_l.Mirror().Reshape({1, H}), U_fl.Mirror()).Reshape({H}) + b_f.Mirror()).Sigmoid();
    Sym f_r = (xW_f.Mirror() + Sym::MatMul(h_r.Mirror().Reshape({1, H}), U_fr.Mirror()).Reshape({H}) + b_f.Mirror()).Sigmoid();
    Sym c = i * u + f_l * c_l + f_r * c_r;
    Sym h = o * Sym::Tanh(c.Mirror());
    Scatter(Sym::Concat({h.Mirror(), c.Mirror()}));
    Push(h.Mirror());
  }
  Sym embedding, W, U, B;

 private:
  int E, H;
  Sym b_iou, b_f, U_iou, U_fl, U_fr;
};

// A gated tree cell with one state block: z = sigmoid(x W_z + (h_l + h_r) U_z + b_z),
// u = tanh(x W_u + h_l U_l + h_r U_r + b_u), h = u * z + (h_l + h_r) - z * (h_l + h_r) scaled by a half.
// The children's states enter both through products and elementwise, and the product of u takes the
// concatenation of the children as its left operand.
class TreeGate : public GraphSupport {
 public:
  TreeGate(const Sym &graph_ph, const Sym &vertex_ph, const Dims &d) : GraphSupport(graph_ph, vertex_ph), E(d.E), H(d.H) {
    embedding = Sym::Variable(DT_FLOAT, {d.V, E}, Sym::Uniform(-0.1f, 0.1f));
    W = Sym::Variable(DT_FLOAT, {2 * E * H}, Sym::Uniform(-0.1f, 0.1f));
    U = Sym::Variable(DT_FLOAT, {3 * H * H}, Sym::Uniform(-0.1f, 0.1f));
    B = Sym::Variable(DT_FLOAT, {2 * H}, Sym::Zeros());
    U_z = U.Slice(0, H * H).Reshape({H, H});
    U_lr = U.Slice(H * H, 2 * H * H).Reshape({2 * H, H});
  }
  void Node() override {
    Sym h_l = Gather(0, {H});
    Sym h_r = Gather(1, {H});
    Sym hs = h_l.Mirror() + h_r.Mirror();
    Sym x = Pull(0, {1});
    x = x.EmbeddingLookup(embedding.Mirror());
    Sym xW = Sym::MatMul(x, W.Reshape({E, 2 * H}).Mirror()).Reshape({H * 2});
    Sym xW_z, xW_u;
    tie(xW_z, xW_u) = xW.Split2();
    Sym b_z, b_u;
    tie(b_z, b_u) = B.Mirror().Split2();
    Sym z = (xW_z + Sym::MatMul(hs.Mirror().Reshape({1, H}), U_z.Mirror()).Reshape({H}) + b_z).Sigmoid();
    Sym lr = Sym::Concat({h_l.Mirror(), h_r.Mirror()});
    Sym u = (xW_u + Sym::MatMul(lr.Reshape({1, 2 * H}), U_lr.Mirror()).Reshape({H}) + b_u).Tanh();
    Sym half = hs.Mirror() * hs.Mirror().Sigmoid();  // a smooth stand-in for a constant factor
    Sym h = u * z.Mirror() + half.Mirror() - z.Mirror() * half.Mirror();
    Scatter(h.Mirror());
    Push(h.Mirror());
  }
  Sym embedding, W, U, B;

 private:
  int E, H;
  Sym U_z, U_lr;
};

class SeqLSTM : public GraphSupport {
 public:
  SeqLSTM(const Sym &graph_ph, const Sym &vertex_ph, const Dims &d) : GraphSupport(graph_ph, vertex_ph), H(d.H) {
    embedding = Sym::Variable(DT_FLOAT, {d.V, H}, Sym::Uniform(-0.1f, 0.1f));
    LSTM_w = Sym::Variable(DT_FLOAT, {8 * H * H}, Sym::Uniform(-0.1f, 0.1f));
    LSTM_b = Sym::Variable(DT_FLOAT, {4 * H}, Sym::Zeros());
    Ux = LSTM_w.Slice(0, 4 * H * H);
    Wh = LSTM_w.Slice(4 * H * H, 4 * H * H);
    bi = LSTM_b.Slice(0, H);
    bf = LSTM_b.Slice(H, H);
    bu = LSTM_b.Slice(2 * H, H);
    bo = LSTM_b.Slice(3 * H, H);
  }
  void Node() override {
    Sym child = Gather(0, {2 * H});
    Sym child_h, child_c;
    tie(child_h, child_c) = child.Split2();
    Sym x = Pull(0, {1});
    x = x.EmbeddingLookup(embedding);
    Sym tmp = Sym::MatMul(x, Ux.Mirror().Reshape({H, 4 * H})) +
              Sym::MatMul(child_h.Expand_dims(0), Wh.Mirror().Reshape({H, 4 * H}));
    Sym i, f, u, o;
    tie(i, f, u, o) = tmp.Split4();
    i = (i + bi.Mirror()).Sigmoid();
    f = (f + bf.Mirror()).Sigmoid();
    u = (u + bu.Mirror()).Tanh();
    o = (o + bo.Mirror()).Sigmoid();
    Sym c = i * u + f * child_c;
    Sym h = o * Sym::Tanh(c.Mirror());
    Scatter(Sym::Concat({h.Mirror(), c.Mirror()}));
    Push(h.Mirror());
  }
  Sym embedding, LSTM_w, LSTM_b;

 private:
  int H;
  Sym Ux, Wh, bi, bf, bu, bo;
};

class TreeFC : public GraphSupport {
 public:
  // variant 0: the reference app (relu, no bias, no vertex input); variant 1: tanh + bias + Pull'ed input
  TreeFC(const Sym &graph_ph, const Sym &vertex_ph, const Dims &d, int variant)
      : GraphSupport(graph_ph, vertex_ph), H(d.H), variant_(variant) {
    W = Sym::Variable(DT_FLOAT, {2 * H, H}, Sym::Uniform(-0.1f, 0.1f));
    if (variant_) Bv = Sym::Variable(DT_FLOAT, {H}, Sym::Zeros());
  }
  void Node() override {
    Sym left = Gather(0, {H});
    Sym right = Gather(1, {H});
    Sym fc = Sym::MatMul(Sym::Concat({left, right}).Reshape({1, 2 * H}), W.Mirror()).Reshape({H});
    Sym res;
    if (variant_) {
      Sym x = Pull(0, {H});
      res = (fc + Bv.Mirror() + x).Tanh();
    } else {
      res = fc.Relu();
    }
    Scatter(res.Mirror());
    Push(res.Mirror());
  }
  Sym W, Bv;

 private:
  int H, variant_;
};

// A child-sum Tree-GRU: r = sigmoid(x W_r + hs U_r + b_r), z = sigmoid(x W_z + hs U_z + b_z) with
// hs = h_l + h_r, candidate c = tanh(x W_c + (r * hs) U_c + b_c), h = z * hs + c - z * c.  The left
// operand of the candidate's product depends on another product of the same vertex: a function of
// two stages.
class TreeGRU : public GraphSupport {
 public:
  TreeGRU(const Sym &graph_ph, const Sym &vertex_ph, const Dims &d) : GraphSupport(graph_ph, vertex_ph), E(d.E), H(d.H) {
    embedding = Sym::Variable(DT_FLOAT, {d.V, E}, Sym::Uniform(-0.1f, 0.1f));
    W = Sym::Variable(DT_FLOAT, {3 * E * H}, Sym::Uniform(-0.1f, 0.1f));
    U = Sym::Variable(DT_FLOAT, {3 * H * H}, Sym::Uniform(-0.1f, 0.1f));
    B = Sym::Variable(DT_FLOAT, {3 * H}, Sym::Zeros());
    U_r = U.Slice(0, H * H).Reshape({H, H});
    U_z = U.Slice(H * H, H * H).Reshape({H, H});
    U_c = U.Slice(2 * H * H, H * H).Reshape({H, H});
    b_r = B.Slice(0, H);
    b_z = B.Slice(H, H);
    b_c = B.Slice(2 * H, H);
  }
  void Node() override {
    Sym h_l = Gather(0, {H});
    Sym h_r = Gather(1, {H});
    Sym hs = h_l + h_r;
    Sym x = Pull(0, {1});
    x = x.EmbeddingLookup(embedding.Mirror());
    Sym xW = Sym::MatMul(x, W.Reshape({E, 3 * H}).Mirror()).Reshape({H * 3});
    Sym xW_r, xW_z, xW_c;
    tie(xW_r, xW_z, xW_c) = xW.Split3();
    Sym r = (xW_r + Sym::MatMul(hs.Mirror().Reshape({1, H}), U_r.Mirror()).Reshape({H}) + b_r.Mirror()).Sigmoid();
    Sym z = (xW_z + Sym::MatMul(hs.Mirror().Reshape({1, H}), U_z.Mirror()).Reshape({H}) + b_z.Mirror()).Sigmoid();
    Sym rh = r * hs.Mirror();
    Sym c = (xW_c + Sym::MatMul(rh.Reshape({1, H}), U_c.Mirror()).Reshape({H}) + b_c.Mirror()).Tanh();
    Sym h = z.Mirror() * hs.Mirror() + c.Mirror() - z.Mirror() * c.Mirror();
    Scatter(h.Mirror());
    Push(h.Mirror());
  }
  Sym embedding, W, U, B;

 private:
  int E, H;
  Sym U_r, U_z, U_c, b_r, b_z, b_c;
};

// Three stages of products that share operands across the stages: the first and the third multiply by
// the same weight block and read the same block of x * W, the first and the second add the same bias.
//   a = sigmoid(xW_0 + hs U_1 + b_1),  m = tanh(xW_1 + (a hs) U_2 + b_1),  q = tanh(xW_0 + m U_1 + b_2),
//   h = a q + hs - a hs                                        with hs = h_l + h_r
class TreeDeep : public GraphSupport {
 public:
  TreeDeep(const Sym &graph_ph, const Sym &vertex_ph, const Dims &d) : GraphSupport(graph_ph, vertex_ph), E(d.E), H(d.H) {
    embedding = Sym::Variable(DT_FLOAT, {d.V, E}, Sym::Uniform(-0.1f, 0.1f));
    W = Sym::Variable(DT_FLOAT, {2 * E * H}, Sym::Uniform(-0.1f, 0.1f));
    U = Sym::Variable(DT_FLOAT, {2 * H * H}, Sym::Uniform(-0.1f, 0.1f));
    B = Sym::Variable(DT_FLOAT, {2 * H}, Sym::Zeros());
    U_1 = U.Slice(0, H * H).Reshape({H, H});
    U_2 = U.Slice(H * H, H * H).Reshape({H, H});
    b_1 = B.Slice(0, H);
    b_2 = B.Slice(H, H);
  }
  void Node() override {
    Sym hs = Gather(0, {H}) + Gather(1, {H});
    Sym x = Pull(0, {1});
    x = x.EmbeddingLookup(embedding.Mirror());
    Sym xW = Sym::MatMul(x, W.Reshape({E, 2 * H}).Mirror()).Reshape({H * 2});
    Sym xW_0, xW_1;
    tie(xW_0, xW_1) = xW.Split2();
    Sym a = (xW_0.Mirror() + Sym::MatMul(hs.Mirror().Reshape({1, H}), U_1.Mirror()).Reshape({H}) + b_1.Mirror()).Sigmoid();
    Sym ah = a.Mirror() * hs.Mirror();
    Sym m = (xW_1 + Sym::MatMul(ah.Mirror().Reshape({1, H}), U_2.Mirror()).Reshape({H}) + b_1.Mirror()).Tanh();
    Sym q = (xW_0.Mirror() + Sym::MatMul(m.Reshape({1, H}), U_1.Mirror()).Reshape({H}) + b_2.Mirror()).Tanh();
    Sym h = a.Mirror() * q + hs.Mirror() - ah.Mirror();
    Scatter(h.Mirror());
    Push(h.Mirror());
  }
  Sym embedding, W, U, B;

 private:
  int E, H;
  Sym U_1, U_2, b_1, b_2;
};

// A family of vertex functions of the general one-stage shape, one per seed, for testing the
// lowering onto generated kernels beyond the handful of named cells: one or two children, one or
// two state blocks, three or four gates, each gate with its own recurrent weights applied to the
// first child's h, the last child's h, the sum or the concatenation of the children's h, sigmoid
// or tanh per gate.  Bits 16-17 of the seed add stages of products: the last gate then multiplies
// the first gate times its operand (two stages), and the one before it the last gate times its
// operand (three).  Every tensor that is used more than once goes through Mirror().
class RandomCell : public GraphSupport {
 public:
  RandomCell(const Sym &graph_ph, const Sym &vertex_ph, const Dims &d, unsigned seed)
      : GraphSupport(graph_ph, vertex_ph), E(d.E), H(d.H), K(1 + (seed & 1)), S(1 + ((seed >> 1) & 1)), NG(3 + ((seed >> 2) & 1)),
        deep(std::min(2u, (seed >> 16) & 3)) {
    embedding = Sym::Variable(DT_FLOAT, {d.V, E}, Sym::Uniform(-0.1f, 0.1f));
    W = Sym::Variable(DT_FLOAT, {NG * E * H}, Sym::Uniform(-0.1f, 0.1f));
    int usize = 0;
    for (int g = 0; g < NG; g++) {
      src[g] = (seed >> (3 + 2 * g)) & 3;
      tanh_[g] = (seed >> (11 + g)) & 1;
      rows[g] = (src[g] == 3 && K == 2) ? 2 * H : H;
      usize += rows[g] * H;
    }
    U = Sym::Variable(DT_FLOAT, {usize}, Sym::Uniform(-0.1f, 0.1f));
    B = Sym::Variable(DT_FLOAT, {NG * H}, Sym::Zeros());
    int at = 0;
    for (int g = 0; g < NG; g++) {
      Ug[g] = U.Slice(at, rows[g] * H).Reshape({rows[g], H});
      bg[g] = B.Slice(g * H, H);
      at += rows[g] * H;
    }
  }
  void Node() override {
    Sym h[2], c[2];
    for (int k = 0; k < K; k++) {
      if (S == 2) tie(h[k], c[k]) = Gather(k, {2 * H}).Split2();
      else h[k] = Gather(k, {H});
    }
    Sym x = Pull(0, {1});
    x = x.EmbeddingLookup(embedding.Mirror());
    Sym xW = Sym::MatMul(x, W.Reshape({E, NG * H}).Mirror()).Reshape({NG * H});
    Sym gate[4];
    // the gates in the order of their stages: those over the children's states, then the last one
    // (over the first gate times the states), then the one before it (over the last gate times them)
    int order[4], scaled_by[4], n = 0;
    for (int g = 0; g < NG - deep; g++) order[n] = g, scaled_by[n++] = -1;
    if (deep >= 1) order[n] = NG - 1, scaled_by[n++] = 0;
    if (deep >= 2) order[n] = NG - 2, scaled_by[n++] = NG - 1;
    for (int i = 0; i < NG; i++) {
      const int g = order[i], by = scaled_by[i];
      auto part = [&](int k) { return by < 0 ? h[k].Mirror() : gate[by].Mirror() * h[k].Mirror(); };
      Sym a;
      if (K == 1 || src[g] == 0) a = part(0);
      else if (src[g] == 1) a = part(1);
      else if (src[g] == 2) a = part(0) + part(1);
      else a = Sym::Concat({part(0), part(1)});
      Sym pre = xW.Slice(g * H, H) + Sym::MatMul(a.Reshape({1, rows[g]}), Ug[g].Mirror()).Reshape({H}) + bg[g].Mirror();
      gate[g] = tanh_[g] ? pre.Tanh() : pre.Sigmoid();
    }
    Sym hn;
    if (S == 2) {
      Sym cn = gate[0].Mirror() * gate[1].Mirror() + gate[2].Mirror() * c[0].Mirror();
      if (K == 2) cn = cn + gate[NG - 1].Mirror() * c[1].Mirror();
      hn = gate[1].Mirror() * Sym::Tanh(cn.Mirror());
      if (NG == 4 && K == 1) hn = hn + gate[3].Mirror() * gate[0].Mirror();
      Scatter(Sym::Concat({hn.Mirror(), cn.Mirror()}));
    } else {
      hn = gate[0].Mirror() * gate[1].Mirror() + gate[2].Mirror() * h[0].Mirror();
      if (K == 2) hn = hn - gate[NG - 1].Mirror() * h[1].Mirror();
      else if (NG == 4) hn = hn + gate[3].Mirror();
      Scatter(hn.Mirror());
    }
    Push(hn.Mirror());
  }
  Sym embedding, W, U, B;
  int children() const { return K; }

 private:
  int E, H, K, S, NG, deep;
  int src[4], tanh_[4], rows[4];
  Sym Ug[4], bg[4];
};

struct App {
  Dims d{};
  std::string model;
  std::unique_ptr<GraphSupport> gs;
  Sym graph, vertex, label, mask, weight, bias, graph_output, loss, train, total;
  vector<std::pair<std::string, Sym>> vars;  // oracle name -> Variable
  std::unique_ptr<Session> sess;
};

App *g_app = nullptr;

}  // namespace

extern "C" {

// model: "treelstm" | "lstm" | "treefc" (reference app) | "treefc_x" (tanh + bias + input, sum of
// squares at the roots).  Declares the program and opens a session.  One app per process at a time.
// gradient clipping threshold of the optimizer the next cavs_app_create declares (0: none)
static float g_clip = 0.f;
void cavs_app_set_clip(float clip) { g_clip = clip; }
// passes of the optimizer's scope per Session::Run of the next app (Optimizer(vars, lr, clip, iters))
static int g_iters = 1;
void cavs_app_set_iters(int iters) { g_iters = iters > 0 ? iters : 1; }

int cavs_app_create(const char *model, int B, int maxlen, int V, int E, int H, int C, int opt, float lr) {
  try {
    delete g_app;
    g_app = nullptr;
    C_ResetGraph();
    auto app = std::make_unique<App>();
    app->d = Dims{B, maxlen, V, E, H, C};
    app->model = model;
    const Dims &d = app->d;
    app->graph = Sym::Placeholder(DT_FLOAT, {B, maxlen}, "CPU");
    bool fc = app->model == "treefc" || app->model == "treefc_x";
    app->vertex = Sym::Placeholder(DT_FLOAT, app->model == "treefc_x" ? vector<int>{B * maxlen, H} : vector<int>{B, maxlen});
    if (!fc) {
      app->label = Sym::Placeholder(DT_FLOAT, {B, maxlen});
      app->weight = Sym::Variable(DT_FLOAT, {C, H}, Sym::Uniform(-0.1f, 0.1f));
      app->bias = Sym::Variable(DT_FLOAT, {1, C}, Sym::Zeros());
    }
    if (app->model == "treelstm") {
      auto *m = new TreeLSTM(app->graph, app->vertex, d);
      app->gs.reset(m);
      app->vars = {{"Emb", m->embedding}, {"W", m->W}, {"U", m->U}, {"Bv", m->B}};
    } else if (app->model == "treelstm2") {
      auto *m = new TreeLSTM2(app->graph, app->vertex, d);
      app->gs.reset(m);
      app->vars = {{"Emb", m->embedding}, {"W", m->W}, {"U", m->U}, {"Bv", m->B}};
    } else if (app->model == "treegate") {
      auto *m = new TreeGate(app->graph, app->vertex, d);
      app->gs.reset(m);
      app->vars = {{"Emb", m->embedding}, {"W", m->W}, {"U", m->U}, {"Bv", m->B}};
    } else if (app->model == "treegru") {
      auto *m = new TreeGRU(app->graph, app->vertex, d);
      app->gs.reset(m);
      app->vars = {{"Emb", m->embedding}, {"W", m->W}, {"U", m->U}, {"Bv", m->B}};
    } else if (app->model == "treedeep") {
      auto *m = new TreeDeep(app->graph, app->vertex, d);
      app->gs.reset(m);
      app->vars = {{"Emb", m->embedding}, {"W", m->W}, {"U", m->U}, {"Bv", m->B}};
    } else if (app->model.rfind("cell", 0) == 0) {
      auto *m = new RandomCell(app->graph, app->vertex, d, (unsigned)std::stoul(app->model.substr(4)));
      app->gs.reset(m);
      app->vars = {{"Emb", m->embedding}, {"W", m->W}, {"U", m->U}, {"Bv", m->B}};
    } else if (app->model == "lstm") {
      auto *m = new SeqLSTM(app->graph, app->vertex, d);
      app->gs.reset(m);
      app->vars = {{"Emb", m->embedding}, {"W", m->LSTM_w}, {"Bv", m->LSTM_b}};
    } else if (fc) {
      auto *m = new TreeFC(app->graph, app->vertex, d, app->model == "treefc_x");
      app->gs.reset(m);
      app->vars = {{"W", m->W}};
      if (app->model == "treefc_x") app->vars.push_back({"Bv", m->Bv});
    } else {
      return -1;
    }
    app->graph_output = app->gs->Output();
    if (!fc) {
      app->vars.push_back({"Wfc", app->weight});
      app->vars.push_back({"bfc", app->bias});
      Sym label_reshape = app->label.Reshape({-1, 1});
      label_reshape.ControlDependency(app->graph_output);
      app->loss = app->graph_output.FullyConnected(app->weight, app->bias).SoftmaxEntropyLoss(label_reshape);
      app->total = app->loss.Reduce_mean();
    } else if (app->model == "treefc_x") {
      app->mask = Sym::Placeholder(DT_FLOAT, {B * maxlen, H});
      Sym mask_rows = app->mask.Reshape({-1, H});
      mask_rows.ControlDependency(app->graph_output);
      app->loss = (app->graph_output.Square() * mask_rows).Reduce_sum();
      app->total = app->loss;
    } else {
      app->loss = app->graph_output.Reduce_sum();  // tree-fc-cavs.cc:96
      app->total = app->loss;
    }
    app->train = app->loss.Optimizer({}, lr, g_clip, g_iters);
    if (opt >= 0) app->sess = std::make_unique<Session>(opt);  // opt < 0: declare only (no device needed)
    g_app = app.release();
    return 0;
  } catch (const std::exception &e) {
    std::fprintf(stderr, "cavs_app_create: %s\n", e.what());
    return -2;
  }
}

int cavs_app_set_param(const char *name, const float *data, size_t n) {
  if (!g_app) return -1;
  for (auto &v : g_app->vars)
    if (v.first == name) {
      try {
        g_app->sess->SetVariable(v.second, data, n);
        return 0;
      } catch (const std::exception &e) {
        std::fprintf(stderr, "cavs_app_set_param: %s\n", e.what());
        return -2;
      }
    }
  return -3;
}

void cavs_app_configure(int pairing, int allow_fused) {
  if (!g_app) return;
  g_app->sess->SetPairing(pairing);
  g_app->sess->SetLoweringMode(allow_fused);
}

// One Session::Run of {train, loss, graph_output} (or without train).  graph is the
// [B, maxlen] parent array; x and labels are full placeholder buffers (packed by vertex id).
// Outputs: loss rows (N, or 1 for the Tree-FC losses) and graph_out [N, H]; returns N or < 0.
long cavs_app_step(const int *graph, const float *x, const float *labels, const float *mask, int train,
                   float *loss_out, size_t loss_cap, float *go_out, size_t go_cap) {
  if (!g_app) return -1;
  try {
    App &a = *g_app;
    vector<std::pair<Sym, void *>> feeds = {{a.graph, (void *)graph}};
    bool fc = a.model == "treefc" || a.model == "treefc_x";
    if (!fc || a.model == "treefc_x") feeds.push_back({a.vertex, (void *)x});
    if (!fc) feeds.push_back({a.label, (void *)labels});
    if (a.model == "treefc_x") feeds.push_back({a.mask, (void *)mask});
    vector<Sym> outs;
    if (train) outs.push_back(a.train);
    if (train && !loss_out && !go_out) {  // as the reference apps loop: sess.Run({train}, feeds), nothing read back
      a.sess->Run(outs, feeds);
      return 0;
    }
    outs.push_back(a.loss);
    outs.push_back(a.graph_output);
    a.sess->Run(outs, feeds);
    vector<float> go = a.sess->Read(a.graph_output.output(0));
    vector<float> loss = a.sess->Read(a.loss.output(0));
    if (loss.size() > loss_cap || go.size() > go_cap) return -4;
    std::memcpy(loss_out, loss.data(), loss.size() * 4);
    std::memcpy(go_out, go.data(), go.size() * 4);
    return (long)(go.size() / a.d.H);
  } catch (const std::exception &e) {
    std::fprintf(stderr, "cavs_app_step: %s\n", e.what());
    return -2;
  }
}

// gradient (grad != 0) or current value of a parameter by oracle name
long cavs_app_read_param(const char *name, int grad, float *out, size_t cap) {
  if (!g_app) return -1;
  for (auto &v : g_app->vars)
    if (v.first == name) {
      try {
        vector<float> t = g_app->sess->Read(v.second.output(0) + (grad ? "_grad" : ""));
        if (t.size() > cap) return -(long)t.size();
        std::memcpy(out, t.data(), t.size() * 4);
        return (long)t.size();
      } catch (const std::exception &e) {
        std::fprintf(stderr, "cavs_app_read_param: %s\n", e.what());
        return -2;
      }
    }
  return -3;
}

long cavs_app_read(const char *edge, float *out, size_t cap) {
  if (!g_app) return -1;
  return C_ReadTensor(g_app->sess->handle(), edge, out, cap);
}

// element count of a parameter by oracle name (the cells of the seeded family size theirs by the seed)
long cavs_app_var_size(const char *name) {
  if (!g_app) return -1;
  for (auto &v : g_app->vars)
    if (v.first == name) {
      long n = 1;
      for (int d : v.second.shape(0)) n *= d;
      return n;
    }
  return -3;
}

int cavs_app_uses_fused_path(void) { return g_app ? g_app->sess->FusedPathKind() : 0; }
int cavs_app_generated_kernels(void) { return g_app ? g_app->sess->GeneratedKernels() : 0; }

void cavs_app_destroy(void) {
  delete g_app;
  g_app = nullptr;
  C_ResetGraph();
}

}  // extern "C"
