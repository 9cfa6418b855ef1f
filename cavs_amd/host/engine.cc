#include "engine.h"

#include <algorithm>
#include <chrono>
#include <cstring>

// runs one backend call inside a profiling bracket of the given kernel class
#define CAVS_TIMED(cls, call)   \
  do {                          \
    ProfScope _ps(this, cls);   \
    check(call);                \
  } while (0)

namespace cavs {

namespace {
// polls of a tail launch's bounded wait (a poll is a round trip to the L2 and a short sleep: ~1 us)
constexpr int kTailSpins = 1 << 19;
inline size_t grow(size_t need, size_t have) {
  if (need <= have) return have;
  size_t g = have + have / 4;
  return std::max(need, g);
}
}  // namespace

Engine::Engine(const cavs_session_config &cfg, void *external_stream, std::shared_ptr<const CellSpec> cell) : cfg_(cfg), cell_(std::move(cell)) {
  if (cfg.model < 0 || cfg.model > CAVS_MODEL_CELL) fail(CAVS_EINVAL, "unknown model " + std::to_string(cfg.model));
  if ((cfg.model == CAVS_MODEL_CELL) != (cell_ != nullptr))
    fail(CAVS_EINVAL, "model CAVS_MODEL_CELL is a vertex function lowered by the front end and comes with its description");
  if (cfg.loss < 0 || cfg.loss > 2) fail(CAVS_EINVAL, "unknown loss " + std::to_string(cfg.loss));
  if (cfg.pairing < 0 || cfg.pairing > 1) fail(CAVS_EINVAL, "unknown pairing");
  if (cfg.H <= 0) fail(CAVS_EINVAL, "hidden size must be positive");
  const size_t H = cfg.H;
  E_ = cfg.model == CAVS_MODEL_LSTM ? cfg.H : cfg.E;  // the chain LSTM requires E == H
  ld_e_ = cfg.model == CAVS_MODEL_TREELSTM ? E_ + 4 : E_;
  mw_ = cfg.model == CAVS_MODEL_TREEFC ? cfg.H : 2 * cfg.H;
  nch_ = cfg.model == CAVS_MODEL_LSTM ? 1 : 2;
  if (cell_) {
    if (cell_->H != cfg.H || cell_->K < 1 || cell_->K > 2 || (int)cell_->params.size() > CA_MAX_PARAMS)
      fail(CAVS_EINVAL, "the description of the lowered vertex function does not fit the session");
    E_ = ld_e_ = cell_->E;
    const CellSpec *tail = cell_.get();
    while (tail->next) tail = tail->next.get();
    if (tail->S != cell_->SI) fail(CAVS_EINVAL, "the last cell of the chain does not write what the first one gathers");
    mw_ = tail->S * cfg.H;
    nch_ = cell_->K;
  }
  const bool reads_x = cell_ ? cell_->NX > 0 : cfg.model != CAVS_MODEL_TREEFC;
  if (reads_x && (cfg.V <= 0 || E_ <= 0))
    fail(CAVS_EINVAL, "vocabulary and embedding sizes must be positive");
  if (cfg.loss == CAVS_LOSS_SOFTMAX && cfg.C <= 0) fail(CAVS_EINVAL, "class count must be positive");
  check(cavs_init(cfg.device));
  if (external_stream) {
    stream_ = external_stream;
    own_stream_ = false;
  } else {
    check(cavs_stream_create(&stream_));
  }
  for (auto &e : ev_) check(cavs_event_create(&e));
  switch (cfg.model) {
    case CAVS_MODEL_TREELSTM:
      add_param("Emb", (size_t)cfg.V * E_);
      add_param("W", (size_t)E_ * 4 * H, 4 * 4 * H);  // four more rows (one used): the bias gradient comes out of the same product
      add_param("U", 4 * H * H);
      add_param("Bv", 4 * H);
      break;
    case CAVS_MODEL_LSTM:
      add_param("Emb", (size_t)cfg.V * H);
      add_param("W", 8 * H * H);
      add_param("Bv", 4 * H);
      break;
    case CAVS_MODEL_CELL:
      for (const CellParam &p : cell_->params) add_param(p.name, (size_t)p.size);
      for (std::shared_ptr<const CellSpec> c = cell_; c; c = c->next) {
        cells_.emplace_back();
        cells_.back().spec = c;
        check(cavs_cell_compile(c->source.c_str(), &cells_.back().module));
      }
      break;
    default:
      add_param("W", 2 * H * H);
      if (cfg.use_bias) add_param("Bv", H);
  }
  if (cfg.loss == CAVS_LOSS_SOFTMAX) {
    add_param("Wfc", (size_t)cfg.C * H);
    add_param("bfc", cfg.C);
  }
  tail_setup();
}

// ------------------------------------------------------------------ the rounds near the roots in one launch
// Whether this device runs the workgroups of such a launch all at once on one XCD is asked once,
// with the barrier alone (cavs_tail_probe); a device that does not keeps to one launch per round.
void Engine::tail_setup() {
  tail_ready_ = false;
  if (cfg_.model != CAVS_MODEL_TREELSTM || !(cfg_.opt & CAVS_OPT_BATCHING) || cfg_.tail_rows < 0) return;
  if (!cavs_tail_rounds_ok(1, cfg_.H)) return;
  const size_t words = cavs_tail_sync_bytes() / sizeof(int);
  tail_sync_.reserve(words);
  check(cavs_zero(tail_sync_.get(), words * sizeof(int), stream_));
  check(cavs_tail_probe(reinterpret_cast<unsigned *>(tail_sync_.get()), cfg_.H, kTailSpins, stream_));
  int head[4] = {0, 0, 0, 0};
  check(cavs_memcpy_d2h(head, tail_sync_.get(), sizeof(head), stream_));
  check(cavs_stream_sync(stream_));
  tail_ready_ = head[1] == 0;
  if (!tail_ready_) check(cavs_zero(tail_sync_.get(), words * sizeof(int), stream_));
}

int Engine::tail_limit() const {
  if (!tail_ready_ || fused_rows() <= 0) return 0;
  // a round whose rows are dealt so that some group gets more than this stays a launch of its own
  // (the launches take a group's share of a round in slices of at most 32 rows).  64 takes in every
  // round above the leaves of a batch of 64 parse trees: measured 0.363 ms per step against 0.366
  // with 32, where the first one or two rounds stay launches of their own; 96 and 128: the same.
  return cfg_.tail_rows > 0 ? cfg_.tail_rows : 64;
}

// The rounds inside the tail launches and who runs which row (build_tail_lists): the groups' row
// lists go to `rows_out` (room for N ints), the plan to tail_.
void Engine::build_tail_plan(const int *kid_rows, int *rows_out) {
  tail_ = TailPlan();
  const int lim = tail_limit();
  if (lim <= 0 || nch_ != 2 || !cavs_round_packed_ok(1, cfg_.H) || !cavs_tail_rounds_ok(1, cfg_.H)) return;
  build_tail_lists(*sched_, kid_rows, lim, cavs_tail_max_groups(), cavs_tail_max_rounds(), 32, &tail_, rows_out);
  tail_.vertices = (double)tail_.rows;
  tail_.flops = 2.0 * tail_.rows * cfg_.H * 5.0 * cfg_.H;
}

void Engine::tail_check() {
  if (!tail_pending_) return;
  tail_pending_ = false;
  int words[4] = {0, 0, 0, 0};
  check(cavs_memcpy_d2h(words, tail_sync_.get(), sizeof(words), stream_));
  check(cavs_stream_sync(stream_));
  if (words[1] == 0) return;
  // every launch since the one that gave up left at once, and every parameter update watched the
  // word: the parameters are those of the last good step.  From here on: one launch per round.
  tail_ready_ = false;
  state_epoch_++;
  upk_valid_ = wfct_valid_ = false;
  emb_sparse_valid_ = false;
  check(cavs_zero(tail_sync_.get(), cavs_tail_sync_bytes(), stream_));
  fail(CAVS_EHIP, std::string("a launch over the rounds near the roots gave up (") +
                      (words[1] == CAVS_TAIL_TIMEOUT ? "its workgroups were not all resident within the wait's bound"
                                                     : "its workgroups did not share one XCD") +
                      "): the results of the steps since the last synchronisation are undefined and their parameter updates were "
                      "skipped; the session continues with one launch per round");
}

Engine::~Engine() {
  cavs_stream_sync(stream_);
  for (CellStage &st : cells_) cavs_cell_release(st.module);
  for (auto &e : ev_) cavs_event_destroy(e);
  for (auto &h : hlists_) {
    if (h.free_ev) cavs_event_destroy(h.free_ev);
    if (h.up_ev) cavs_event_destroy(h.up_ev);
  }
  for (auto &e : prof_events_) cavs_event_destroy(e);
  if (sched_stream_) {
    cavs_stream_sync(sched_stream_);
    cavs_stream_destroy(sched_stream_);
  }
  if (aux_stream_) {
    cavs_stream_sync(aux_stream_);
    cavs_stream_destroy(aux_stream_);
    cavs_event_destroy(aux_fork_ev_);
    cavs_event_destroy(aux_join_ev_);
  }
  for (void *e : chunk_done_ev_)
    if (e) cavs_event_destroy(e);
  for (auto &d : dsched_)
    if (d.free_ev) cavs_event_destroy(d.free_ev);
  if (own_stream_) cavs_stream_destroy(stream_);
}

void Engine::add_param(const std::string &name, size_t n, size_t extra_grad) {
  auto p = std::make_unique<Param>();
  p->n = n;
  p->own_w.reserve(n);
  p->own_g.reserve(n + extra_grad);
  p->w = p->own_w.get();
  p->g = p->own_g.get();
  check(cavs_zero(p->w, n * 4, stream_));
  check(cavs_zero(p->g, n * 4, stream_));
  params_[name] = std::move(p);
}

Param &Engine::param(const std::string &name) {
  auto it = params_.find(name);
  if (it == params_.end()) fail(CAVS_EINVAL, "this model has no parameter named '" + name + "'");
  return *it->second;
}

void Engine::bind_param(const std::string &name, float *w, float *g) {
  Param &p = param(name);
  if (!w) fail(CAVS_EINVAL, "bind_param('" + name + "'): null weight pointer");
  if (p.w != w) upk_valid_ = wfct_valid_ = false;
  state_epoch_++;
  p.w = w;
  p.g = g ? g : p.own_g.get();
}

// a classifier wide enough for the transposed copy of its weights to pay (head_forward_backward)
bool Engine::wide_head() const {
  return cfg_.loss == CAVS_LOSS_SOFTMAX && (size_t)cfg_.C * cfg_.H >= ((size_t)1 << 18) &&
         cavs_fc_softmax_xent_workspace(1, cfg_.H, cfg_.C) == 0;
}

bool Engine::update_jobs(float *w, float *g, float lr, std::vector<cavs_task> *out) {
  if (!w || !g) return false;
  if (wide_head() && w == param("Wfc").w && WfcT_.capacity() >= (size_t)cfg_.C * cfg_.H) {
    out->push_back({CAVS_TASK_SGD_TRANSPOSE, lr, cfg_.C, cfg_.H, 0, WfcT_.get(), w, g, nullptr});
    wfct_valid_ = true;
    return true;
  }
  if (Upk_.capacity() == 0) return false;
  const long long H = cfg_.H;
  if (cfg_.model == CAVS_MODEL_TREELSTM && w == param("U").w) {
    out->push_back({CAVS_TASK_SGD_PACK, lr, H, 3 * H, 0, Upk_.get(), w, g, nullptr});
    out->push_back({CAVS_TASK_SGD_PACK, lr, H, H, 0, Upk_.at((size_t)3 * H * H), w + 3 * H * H, g + 3 * H * H, nullptr});
  } else if (cfg_.model == CAVS_MODEL_LSTM && w == param("W").w) {  // [U' | W'], W' with its packed copy
    const long long half = 4 * H * H;
    out->push_back({CAVS_TASK_SGD, lr, half, 0, 0, w, g, nullptr, nullptr});
    out->push_back({CAVS_TASK_SGD_PACK, lr, H, 4 * H, 0, Upk_.get(), w + half, g + half, nullptr});
  } else {
    return false;
  }
  upk_valid_ = true;
  return true;
}

void Engine::set_param(const std::string &name, const float *host, size_t n) {
  Param &p = param(name);
  if (n != p.n || !host)
    fail(CAVS_EINVAL, "parameter '" + name + "' has " + std::to_string(p.n) + " elements, got " + std::to_string(n));
  check(cavs_memcpy_h2d(p.w, host, n * 4, stream_));
  check(cavs_stream_sync(stream_));
  upk_valid_ = wfct_valid_ = false;
  state_epoch_++;
}

void Engine::get_param(const std::string &name, float *host, size_t n, bool grad) {
  Param &p = param(name);
  if (n != p.n || !host)
    fail(CAVS_EINVAL, "parameter '" + name + "' has " + std::to_string(p.n) + " elements, got " + std::to_string(n));
  aux_join();
  check(cavs_memcpy_d2h(host, grad ? p.g : p.w, n * 4, stream_));
  check(cavs_stream_sync(stream_));
}

// ------------------------------------------------------------------ profiling
void *Engine::prof_event() {
  if (prof_used_ == prof_events_.size()) {
    void *e = nullptr;
    check(cavs_event_create(&e));
    prof_events_.push_back(e);
  }
  return prof_events_[prof_used_++];
}

Engine::ProfScope::ProfScope(Engine *eng, int cls) : e(eng), s{cls, nullptr, nullptr}, on(eng->profile_) {
  if (!on) return;
  s.a = e->prof_event();
  s.b = e->prof_event();
  check(cavs_profile_arm(s.a, s.b));
}

Engine::ProfScope::~ProfScope() {
  if (!on) return;
  int launched = 0;
  if (cavs_profile_disarm(&launched) == CAVS_OK && launched) e->spans_.push_back(s);
}

void Engine::profile_enable(bool on) {
  check(cavs_stream_sync(stream_));
  profile_ = on;
  spans_.clear();
  prof_used_ = 0;
}

void Engine::profile_read(int cls, double *total_ms, double *launches) {
  check(cavs_stream_sync(stream_));
  double t = 0, n = 0;
  for (const Span &sp : spans_) {
    if (sp.cls != cls) continue;
    float ms = 0.f;
    check(cavs_event_elapsed_ms(&ms, sp.a, sp.b));
    t += ms;
    n += 1;
  }
  *total_ms = t;
  *launches = n;
}

// ------------------------------------------------------------------ counted wrappers
// All GEMMs go through the workspace-assisted entry point, which picks the kernel by
// shape (full tiles, skinny, or split K through the workspace).
float *Engine::workspace(size_t bytes) {
  if (ws_.capacity() * 4 < bytes) {
    check(cavs_stream_sync(stream_));  // the old workspace may still be in use
    ws_.reserve(std::max<size_t>(bytes / 4 + 1, (size_t)8 << 20));
  }
  return ws_.get();
}

void Engine::gemm(int tA, int tB, int M, int N, int K, const float *A, int lda, const float *B,
                  int ldb, float beta, float *C, int ldc) {
  float *ws = workspace(cavs_sgemm_splitk_workspace(M, N, K));
  ProfScope ps(this, K_GEMM);
  check(cavs_sgemm_splitk(tA, tB, M, N, K, 1.f, A, lda, B, ldb, beta, C, ldc, ws, ws_.capacity() * 4, stream_));
  c_gemm_flops_ += 2.0 * M * N * K;
  c_launches_ += 1;
}

// flops of a product that its block hint declares to be zero or unwanted (the kernels skip them
// tile by tile)
static double hinted_flops(const cavs_gemm_desc &q) {
  double mnk = 0;
  if (q.zero_kind == CAVS_GEMM_A_ZERO && !q.transA)
    mnk = (double)std::min(q.zero_rows, q.M) * std::max(0, q.K - q.zero_col) * q.N;
  else if (q.zero_kind == CAVS_GEMM_B_ZERO && !q.transB)
    mnk = (double)std::min(q.zero_rows, q.K) * std::max(0, q.N - q.zero_col) * q.M;
  return 2.0 * mnk;
}

void Engine::gemm_group(const std::vector<cavs_gemm_desc> &products) {
  const int count = (int)products.size();
  float *ws = workspace(cavs_sgemm_group_workspace(count, products.data()));
  ProfScope ps(this, K_GEMM);
  check(cavs_sgemm_group(count, products.data(), ws, ws_.capacity() * 4, stream_));
  for (const cavs_gemm_desc &q : products) {
    c_gemm_flops_ += 2.0 * q.M * q.N * q.K;
    c_gemm_flops_hinted_ += hinted_flops(q);
  }
  c_launches_ += 1;
}

void Engine::gemm_splitk(int tA, int tB, int M, int N, int K, const float *A, int lda,
                         const float *B, int ldb, float *C, int ldc) {
  gemm(tA, tB, M, N, K, A, lda, B, ldb, 0.f, C, ldc);
}

void Engine::gather(float *out, int ld_out, const float *src, int ld_src, const int *ids, int n,
                    int w) {
  ProfScope ps(this, K_GATHER);
  check(cavs_gather_rows(out, ld_out, src, ld_src, ids, n, w, stream_));
  c_gather_rows_ += n;
  c_gather_bytes_ += (8.0 * w + 4.0) * n;
  c_launches_ += 1;
}

void Engine::scatter(float *dst, int ld_dst, const int *ids, const float *inp, int ld_inp, int n,
                     int w) {
  ProfScope ps(this, K_SCATTER);
  check(cavs_scatter_rows(dst, ld_dst, ids, inp, ld_inp, n, w, stream_));
  c_scatter_rows_ += n;
  c_scatter_bytes_ += (8.0 * w + 4.0) * n;
  c_launches_ += 1;
}

// Growing a buffer frees the old storage, which enqueued kernels may still read.
void Engine::ensure(DeviceArray<float> &a, size_t n) {
  if (n <= a.capacity()) return;
  check(cavs_stream_sync(stream_));
  a.reserve(n);
}

// the identity list 0, 1, 2, ... of at least n entries
void Engine::ensure_iota(size_t n) {
  if (cell_iota_n_ >= n) return;
  std::vector<int> iota(n);
  for (size_t i = 0; i < n; i++) iota[i] = (int)i;
  sync();
  cell_iota_.reserve(n);
  check(cavs_memcpy_h2d(cell_iota_.get(), iota.data(), n * 4, stream_));
  check(cavs_stream_sync(stream_));
  cell_iota_n_ = n;
}

// ------------------------------------------------------------------ memory manager
// Every edge of F is a [rows, width] buffer in which round r lives at rows
// [offset_r, offset_r + n_r): row index == tensor id for every edge, and forward
// activations persist for the backward pass (cavs/midend/op_context.cc:13-40,
// cavs/midend/tensor.cc:311-321).  The reference sizes each edge for MAX_NODE = B*maxlen
// rows (cavs/frontend/cxx/graphsupport.cc:34-35); here rows follow the batch's actual
// total length, and the edges that live for one round only are sized by the widest round.
void Engine::reserve_edges() {
  const size_t H = cfg_.H, N = N_;
  if ((size_t)cap_ < N) cap_ = (int)grow(N, cap_);
  if (rcap_ < sched_->max_round) rcap_ = (int)grow(sched_->max_round, rcap_);
  const size_t cap = cap_, rc = rcap_, mw = mw_;
  auto R = [&](DeviceArray<float> &a, size_t n) { ensure(a, n); };
  R(msg_, cap * mw);
  R(pool_, cap * mw);
  R(dpool_, cap * mw);
  R(GO_, cap * H);
  R(dGO_, cap * H);
  R(dret_, cap * H);
  R(G_, cap * nch_ * mw);
  R(r_dmsg_, rc * mw);
  R(r_dG_, rc * nch_ * mw);
  if (cell_) {
    const CellSpec &c = *cell_;
    if (c.NX > 0) {
      R(xs_, cap);
      if (xs_prev_.capacity() < cap) {
        R(xs_prev_, cap);
        emb_sparse_valid_ = false;
      }
      R(e_, cap * E_);
      R(de_, cap * E_);
      R(xW_, cap * c.NX * H);
    }
    for (size_t ci = 0; ci < cells_.size(); ci++) {
      CellStage &st = cells_[ci];
      const CellSpec &k = *st.spec;
      R(st.sv, cap * std::max(1, k.NSV) * H);   // what a vertex keeps for the backward pass
      R(st.asrc, cap * k.asrc.size() * H);      // the products' left operands by slab row
      R(st.d, cap * k.ND * H);                  // the gradient rows
      // elementwise part of the message gradients: by slab row (one launch per backward round), or
      // by row of the round and child (two launches)
      R(st.ds, std::max(cap * k.SI * H, rc * k.K * k.SI * H));
      R(st.bt, (size_t)2 * k.blocks() * H * H);  // the weight blocks tile-major, as they are and transposed
      R(st.colsum, (size_t)k.ND * H);
      if (ci + 1 < cells_.size()) {
        R(st.rows, cap * k.S * H);
        R(st.drows, cap * k.S * H);
      }
    }
    if (cells_.size() > 1) ensure_iota(cap);
  } else if (cfg_.model != CAVS_MODEL_TREEFC) {
    R(xs_, cap);
    if (xs_prev_.capacity() < cap) {  // the list of dirty rows does not survive a reallocation
      R(xs_prev_, cap);
      emb_sparse_valid_ = false;
    }
    R(e_, cap * ld_e_);
    if (ld_e_ != E_ && e_ones_rows_ < cap) {  // (re)allocated: zero padding and the column of ones
      std::vector<float> col(ld_e_, 0.f);
      col[E_] = 1.f;
      ones_col_.reserve(ld_e_);
      check(cavs_memcpy_h2d(ones_col_.get(), col.data(), col.size() * 4, stream_));
      check(cavs_stream_sync(stream_));
      check(cavs_zero(e_.get(), cap * ld_e_ * 4, stream_));
      check(cavs_bias_add_rows(e_.get(), e_.get(), ones_col_.get(), (int)cap, ld_e_, stream_));
      e_ones_rows_ = cap;
    }
    R(de_, cap * E_);
    R(xW_, cap * 4 * H);
    R(dxW_, cap * 4 * H);
    R(gates_, cap * 6 * H);
    R(dc_, cap * H);
  } else {
    if (cfg_.use_x) R(xs_, cap * H);
    R(dxW_, cap * H);
    R(r_z_, rc * H);
  }
  if (fused_rows() > 0 && !cell_) R(UT_, (size_t)(cfg_.model == CAVS_MODEL_TREEFC ? 2 : 4) * H * H);
  if (fused_rows() > 0 && ((cfg_.model == CAVS_MODEL_TREELSTM && (cavs_round_packed_ok(1, H) || cavs_round_packed_ok(65, H))) ||
                           (cfg_.model == CAVS_MODEL_LSTM && (cavs_lstm_round_packed_ok(1, H) || cavs_lstm_round_packed_ok(65, H)))))
    R(Upk_, (size_t)4 * H * H);
  if (cfg_.model == CAVS_MODEL_TREELSTM) {
    R(hlr_, cap * H);
    R(dF_, cap * 2 * H);
    R(r_hU_, rc * 3 * H);
    R(r_hUf_, rc * 2 * H);
    R(r_dhlr_, rc * H);
  }
  if (cfg_.loss == CAVS_LOSS_SOFTMAX) {
    R(logits_, cap * cfg_.C);
    R(dlogits_, cap * cfg_.C);
    R(loss_, cap);
  } else {
    R(loss_, std::max<size_t>(cap, 2 * H + 2));
    R(logits_, (size_t)sched_->B * H + 1);   // root rows / |h| scratch
    R(dlogits_, std::max<size_t>((size_t)sched_->B * H, cap * H));
  }
}

// One upload per step (the reference copies a list from pageable memory before every
// Gather / Scatter / Pull, cavs/backend/op_impl_graphop.cu:68,149,241,308):
//   t2j   [N]      tensor id -> global vertex id (Pull, FunctionPopRet)
//   pair  [N]      per slab row: pool row the forward Scatter writes and the backward
//                  Gather reads, or -1 (root, or past the end of the compacted list)
//   child [nch*N]  per slab row and child: pool row the forward Gather reads and the
//                  backward Scatter writes
//   roots [B]      vertex ids of the roots (sum-of-squares loss)
void Engine::upload_index_arena() {
  const Schedule &s = *sched_;
  const int N = N_;
  const bool want_forest = !cfg_.split_backward_rounds && fused_rows() > 0;
  const bool want_tail = want_forest && tail_limit() > 0;
  const size_t total = (size_t)N * (2 + nch_) + s.B + (want_forest ? (size_t)N * (nch_ + 1) : 0) + (want_tail ? (size_t)N : 0);
  // Two sets of buffers (pinned staging + device lists) alternate, and the copy runs on a stream
  // of its own: the lists of step k + 1 are built and uploaded while the kernels of step k run,
  // instead of the copy sitting in the compute stream between two steps.  A set is rewritten only
  // after everything that read its device lists has finished (the step before last).
  HostLists &h = hlists_[hlists_slot_];
  hlists_slot_ ^= 1;
  if (!sched_stream_) check(cavs_stream_create(&sched_stream_));
  if (!h.free_ev) check(cavs_event_create(&h.free_ev));
  if (!h.up_ev) check(cavs_event_create(&h.up_ev));
  if (h.busy) {
    auto w0 = std::chrono::steady_clock::now();
    check(cavs_event_sync(h.free_ev));
    wait_ms_ = std::chrono::duration<float, std::milli>(std::chrono::steady_clock::now() - w0).count();
    h.busy = false;
  }
  h.host.reserve(total);
  h.dev.reserve(grow(total, h.dev.capacity()));
  int *t2j = h.host.get(), *pair = t2j + N, *child = pair + N, *roots = child + (size_t)nch_ * N;
  std::string err = build_index_lists(s, nch_, cfg_.pairing, t2j, pair, child, roots);
  if (!err.empty()) fail(CAVS_EUNSUPPORTED, err);
  forest_ = want_forest && build_forest_lists(s, nch_, fused_rows(), pair, child, roots + s.B, roots + s.B + (size_t)nch_ * N, &n_orphans_);
  plan_head_chunks(roots + s.B + (size_t)nch_ * N);
  tail_ = TailPlan();
  int *tail_rows = roots + s.B + (size_t)N * (nch_ + 1);
  if (want_tail && forest_) build_tail_plan(roots + s.B, tail_rows);
  check(cavs_memcpy_h2d(h.dev.get(), h.host.get(), total * sizeof(int), sched_stream_));
  check(cavs_event_record(h.up_ev, sched_stream_));
  check(cavs_event_sync(h.up_ev));  // a few microseconds; the compute stream is still busy with the previous step
  last_free_ev_ = h.free_ev;
  last_busy_ = &h.busy;
  d_t2j_ = h.dev.get();
  d_pair_ = d_t2j_ + N;
  d_child_ = d_pair_ + N;
  d_roots_ = d_child_ + (size_t)nch_ * N;
  d_kid_rows_ = want_forest ? d_roots_ + s.B : nullptr;
  d_orphans_ = want_forest ? d_kid_rows_ + (size_t)nch_ * N : nullptr;
  d_tail_rows_ = want_tail ? d_orphans_ + N : nullptr;
}

// ------------------------------------------------------------------ step
namespace {
// 64-bit mix over the feed's words (not cryptographic: a hit is confirmed by comparing the bytes)
uint64_t hash_feed(const int32_t *g, size_t n, int B, int maxlen, int pairing) {
  uint64_t h = 0x9e3779b97f4a7c15ull ^ ((uint64_t)B << 32) ^ (uint64_t)maxlen ^ ((uint64_t)pairing << 60);
  size_t i = 0;
  for (; i + 2 <= n; i += 2) {
    uint64_t w;
    std::memcpy(&w, g + i, 8);
    h = (h ^ w) * 0xff51afd7ed558ccdull;
    h ^= h >> 32;
  }
  if (i < n) h = (h ^ (uint32_t)g[i]) * 0xc4ceb9fe1a85ec53ull;
  return h ^ (h >> 29);
}
}  // namespace

Engine::Plan *Engine::find_plan(const int *graph, int B, int maxlen, uint64_t hash) {
  for (auto &p : plans_)
    if (p->hash == hash && p->B == B && p->maxlen == maxlen && p->pairing == cfg_.pairing &&
        std::memcmp(p->graph.data(), graph, sizeof(int32_t) * (size_t)B * maxlen) == 0)
      return p.get();
  return nullptr;
}

// Keeps what this step's scheduling produced: the schedule and a compact device copy of its lists.
void Engine::remember_plan(const int *graph, int B, int maxlen, uint64_t hash) {
  std::unique_ptr<Plan> p;
  if ((int)plans_.size() >= cfg_.plan_cache) {
    // the least recently used plan goes; kernels still in flight may be reading its lists
    size_t lru = 0;
    for (size_t i = 1; i < plans_.size(); i++)
      if (plans_[i]->last_used < plans_[lru]->last_used) lru = i;
    check(cavs_stream_sync(stream_));
    p = std::move(plans_[lru]);
    p->drop_graphs();
    plans_.erase(plans_.begin() + lru);
  } else {
    p = std::make_unique<Plan>();
  }
  const size_t N = N_, nk = (size_t)nch_ * N;
  p->hash = hash;
  p->B = B;
  p->maxlen = maxlen;
  p->pairing = cfg_.pairing;
  p->graph.assign(graph, graph + (size_t)B * maxlen);
  p->sched = sched_;
  p->lists_on_host = sched_lists_on_host_;
  p->n_orphans = n_orphans_;
  p->forest = forest_;
  p->last_used = ++plan_clock_;
  p->tail = tail_;
  p->head_chunks = head_chunks_;
  p->lists.reserve(2 * N + 2 * nk + B + N + N);
  int *base = p->lists.get();
  const bool kids = d_kid_rows_ != nullptr;
  check(cavs_memcpy_d2d(base, d_t2j_, N * 4, stream_));
  check(cavs_memcpy_d2d(base + N, d_pair_, N * 4, stream_));
  check(cavs_memcpy_d2d(base + 2 * N, d_child_, nk * 4, stream_));
  check(cavs_memcpy_d2d(base + 2 * N + nk, d_roots_, (size_t)B * 4, stream_));
  if (kids) {
    check(cavs_memcpy_d2d(base + 2 * N + nk + B, d_kid_rows_, nk * 4, stream_));
    check(cavs_memcpy_d2d(base + 2 * N + 2 * nk + B, d_orphans_, (size_t)n_orphans_ * 4, stream_));
  }
  if (tail_.first >= 0) check(cavs_memcpy_d2d(base + 3 * N + 2 * nk + B, d_tail_rows_, tail_.rows * 4, stream_));
  // this step reads the copy as well, so that the buffers the lists were built in are free again
  d_t2j_ = base;
  d_pair_ = base + N;
  d_child_ = base + 2 * N;
  d_roots_ = base + 2 * N + nk;
  d_kid_rows_ = kids ? base + 2 * N + nk + B : nullptr;
  d_orphans_ = kids ? base + 2 * N + 2 * nk + B : nullptr;
  d_tail_rows_ = base + 3 * N + 2 * nk + B;
  plans_.push_back(std::move(p));
}

void Engine::schedule_on_host(const int *graph, int B, int maxlen) {
  auto t0 = std::chrono::steady_clock::now();
  auto fresh = std::make_shared<Schedule>();
  std::string err = build_schedule(graph, B, maxlen, (cfg_.opt & CAVS_OPT_BATCHING) != 0, fresh.get());
  sched_ms_ = std::chrono::duration<float, std::milli>(std::chrono::steady_clock::now() - t0).count();
  if (!err.empty()) fail(CAVS_EINVAL, "graph feed rejected: " + err);
  if (fresh->executed != fresh->N)
    fail(CAVS_EUNSUPPORTED, "the batch holds a single-vertex sample; the reference never executes such a vertex "
                            "(graph_scheduler.cc:180) and leaves its rows undefined");
  sched_ = fresh;
  sched_lists_on_host_ = true;
  N_ = sched_->N;
  upload_index_arena();
}

// The graph feed goes to the device, cavs_schedule_arena builds every list there, the host gets
// the round offsets back and drives the rounds with them.  The scheduler's kernels run on a
// stream of their own, so that waiting for the offsets does not wait for the previous step.
void Engine::schedule_on_device(const int *graph, int B, int maxlen) {
  auto t0 = std::chrono::steady_clock::now();
  DeviceSched &d = dsched_[dsched_slot_];
  dsched_slot_ ^= 1;
  if (!sched_stream_) check(cavs_stream_create(&sched_stream_));
  if (!d.free_ev) check(cavs_event_create(&d.free_ev));
  if (d.busy) {  // the step before last read these lists
    auto w0 = std::chrono::steady_clock::now();
    check(cavs_event_sync(d.free_ev));
    wait_ms_ = std::chrono::duration<float, std::milli>(std::chrono::steady_clock::now() - w0).count();
    d.busy = false;
  }
  const size_t BM = (size_t)B * maxlen, nmeta = (size_t)maxlen + 9;
  const size_t need = BM * (2 + 2 * (size_t)nch_) + 2 * (size_t)B;
  d.graph_host.reserve(BM);
  d.meta_host.reserve(nmeta);
  d.graph_dev.reserve(BM);
  d.meta_dev.reserve(nmeta);
  d.lists.reserve(need);
  d.cap = (long)BM;
  const size_t sbytes = cavs_schedule_arena_scratch(B, maxlen);
  dsched_scratch_.reserve(sbytes / 4 + 1);
  std::memcpy(d.graph_host.get(), graph, BM * sizeof(int));
  check(cavs_memcpy_h2d(d.graph_dev.get(), d.graph_host.get(), BM * sizeof(int), sched_stream_));
  int *t2j = d.lists.get(), *pair = t2j + BM, *child = pair + BM, *kid = child + (size_t)nch_ * BM,
      *roots = kid + (size_t)nch_ * BM, *orph = roots + B;
  check(cavs_schedule_arena(d.graph_dev.get(), B, maxlen, nch_, cfg_.pairing, t2j, pair, child, kid, roots, orph, d.cap,
                            d.meta_dev.get(), dsched_scratch_.get(), sbytes, sched_stream_));
  check(cavs_memcpy_d2h(d.meta_host.get(), d.meta_dev.get(), nmeta * sizeof(int), sched_stream_));
  check(cavs_stream_sync(sched_stream_));
  c_launches_ += 5;
  const int *meta = d.meta_host.get();
  const int N = meta[0], R = meta[1], bad = meta[2];
  if (bad) {
    std::string why;
    if (bad & 1) why += " a sample has no -1 terminator within maxlen;";
    if (bad & 2) why += " a parent id is out of range;";
    if (bad & 8) why += " the batch holds a single-vertex sample, which the reference never executes (graph_scheduler.cc:180);";
    if (bad & 4) why += std::string(" a vertex has children, but not ") + (nch_ == 2 ? "two children" : "one child") +
                        " (the round mixes vertices with and without a child);";
    if (bad & 16) why += " vertices never become ready: the parent array holds a cycle;";
    fail((bad & 8) ? CAVS_EUNSUPPORTED : CAVS_EINVAL, "graph feed rejected:" + why);
  }
  // the rounds, as far as the loops over them need: offsets, sizes, which one holds the leaves
  auto fresh = std::make_shared<Schedule>();
  Schedule &s = *fresh;
  s.B = B;
  s.maxlen = maxlen;
  s.N = s.executed = N;
  s.batching = true;
  s.round2offset.assign(meta + 8, meta + 8 + R + 1);
  for (int r = 0; r < R; r++) {
    Round rd{};
    rd.offset = meta[8 + r];
    rd.n = meta[8 + r + 1] - meta[8 + r];
    // only whether the gather ranges are empty is read from a schedule without lists
    rd.gather_end[0] = rd.gather_end[1] = r > 0 ? rd.n : 0;
    if (nch_ == 1) rd.gather_end[1] = 0;
    s.rounds.push_back(rd);
    s.max_round = std::max(s.max_round, rd.n);
  }
  for (int k = R - 1; k >= 0; k--) s.bwd_rounds.push_back(k);
  s.leaf_prefix = R > 0 ? meta[9] : 0;
  sched_ = fresh;
  sched_lists_on_host_ = false;
  N_ = N;
  d_t2j_ = t2j;
  d_pair_ = pair;
  d_child_ = child;
  d_kid_rows_ = kid;
  d_roots_ = roots;
  d_orphans_ = orph;
  // every sample has one root, so B slab rows send no message; the message flow of a well-formed
  // batch is a forest by construction, what remains to ask is whether every round with children
  // runs as a fused launch
  n_orphans_ = B;
  forest_ = !cfg_.split_backward_rounds && fused_rows() > 0;
  for (int r = 1; r < R && forest_; r++) forest_ = s.rounds[r].n <= fused_rows();
  // The tail launches want whole trees of the message flow dealt to their groups, which is host
  // work on the children-by-slab-row list: it comes back (2N ints), the groups' row lists go up.
  tail_ = TailPlan();
  if (forest_ && nch_ == 2 && tail_limit() > 0 && N > 0) {
    d.kid_host.reserve(2 * (size_t)N);
    d.tail_host.reserve(N);
    check(cavs_memcpy_d2h(d.kid_host.get(), kid, 2 * (size_t)N * sizeof(int), sched_stream_));
    check(cavs_stream_sync(sched_stream_));
    build_tail_plan(d.kid_host.get(), d.tail_host.get());
    if (tail_.first >= 0) {
      d.tail_dev.reserve(grow(N, d.tail_dev.capacity()));
      check(cavs_memcpy_h2d(d.tail_dev.get(), d.tail_host.get(), tail_.rows * sizeof(int), sched_stream_));
      check(cavs_stream_sync(sched_stream_));
      d_tail_rows_ = d.tail_dev.get();
    }
  }
  last_free_ev_ = d.free_ev;
  last_busy_ = &d.busy;
  sched_ms_ = std::chrono::duration<float, std::milli>(std::chrono::steady_clock::now() - t0).count();
}

const Schedule &Engine::schedule() {
  if (!sched_lists_on_host_ && N_ > 0) {
    const size_t N = N_, nk = (size_t)nch_ * N;
    std::vector<int> t2j(N), pair(N), child(nk), roots(sched_->B);
    check(cavs_memcpy_d2h(t2j.data(), d_t2j_, N * 4, stream_));
    check(cavs_memcpy_d2h(pair.data(), d_pair_, N * 4, stream_));
    check(cavs_memcpy_d2h(child.data(), d_child_, nk * 4, stream_));
    check(cavs_memcpy_d2h(roots.data(), d_roots_, (size_t)sched_->B * 4, stream_));
    check(cavs_stream_sync(stream_));
    auto full = std::make_shared<Schedule>();
    schedule_from_lists(sched_->B, sched_->maxlen, N_, nch_, sched_->round2offset.data(), (int)sched_->rounds.size(), t2j.data(),
                        pair.data(), child.data(), roots.data(), full.get());
    for (auto &p : plans_)
      if (p->sched == sched_) {  // the cached plan gets the complete schedule too
        p->sched = full;
        p->lists_on_host = true;
      }
    sched_ = full;
    sched_lists_on_host_ = true;
  }
  return *sched_;
}

// ------------------------------------------------------------------ step
void Engine::begin_step(const int *graph, int B, int maxlen) {
  auto t0 = std::chrono::steady_clock::now();
  if (!graph || B <= 0 || maxlen <= 0) fail(CAVS_EINVAL, "graph feed rejected: empty graph feed");
  if (last_free_ev_) {  // everything that reads the previous step's lists is enqueued by now
    check(cavs_event_record(last_free_ev_, stream_));
    *last_busy_ = true;
    last_free_ev_ = nullptr;
  }
  c_gather_rows_ = c_scatter_rows_ = c_gemm_flops_ = c_gemm_flops_hinted_ = c_launches_ = c_gather_bytes_ = c_scatter_bytes_ = 0;
  c_round_flops_ = 0;
  c_tail_rounds_ = c_tail_launches_ = 0;
  bias_jobs_.clear();
  head_chunks_.clear();  // (planned with the host scheduler's lists only)
  pending_tasks_.clear();  // (a step that failed half way may have left a job for a backward pass that never ran)
  wait_ms_ = 0.f;
  uint64_t hash = 0;
  Plan *hit = nullptr;
  if (cfg_.plan_cache > 0) {
    hash = hash_feed(graph, (size_t)B * maxlen, B, maxlen, cfg_.pairing);
    hit = find_plan(graph, B, maxlen, hash);
  }
  hit_plan_ = hit;
  if (hit) {
    // a batch structure seen before: its schedule and its lists are where the last such step left them
    hit->last_used = ++plan_clock_;
    c_plan_hits_ += 1;
    scheduler_used_ = 2;
    sched_ = hit->sched;
    sched_lists_on_host_ = hit->lists_on_host;
    N_ = sched_->N;
    n_orphans_ = hit->n_orphans;
    const bool want_forest = !cfg_.split_backward_rounds && fused_rows() > 0;
    forest_ = hit->forest && want_forest;
    const size_t N = N_, nk = (size_t)nch_ * N;
    const int *base = hit->lists.get();
    d_t2j_ = base;
    d_pair_ = base + N;
    d_child_ = base + 2 * N;
    d_roots_ = base + 2 * N + nk;
    d_kid_rows_ = base + 2 * N + nk + B;
    d_orphans_ = base + 2 * N + 2 * nk + B;
    d_tail_rows_ = base + 3 * N + 2 * nk + B;
    tail_ = (forest_ && tail_limit() > 0) ? hit->tail : TailPlan();
    if (forest_ && !cfg_.graph_replay) head_chunks_ = hit->head_chunks;
    sched_ms_ = 0.f;
  } else {
    tail_ = TailPlan();  // (the host-built lists bring a new one)
    const bool on_device = cfg_.schedule_mode == 1 && (cfg_.opt & CAVS_OPT_BATCHING);
    // (one wavefront per sample with its parent row in LDS: a limit of the kernels, and the caller's to know)
    if (on_device && maxlen > 2048)
      fail(CAVS_EUNSUPPORTED, "the device scheduler takes samples of at most 2048 vertices (maxlen = " + std::to_string(maxlen) +
                                  "); use schedule_mode 0, the host scheduler");
    if (on_device) schedule_on_device(graph, B, maxlen); else schedule_on_host(graph, B, maxlen);
    scheduler_used_ = on_device ? 1 : 0;
    if (cfg_.plan_cache > 0) {
      c_plan_misses_ += 1;
      remember_plan(graph, B, maxlen, hash);
    }
  }
  reserve_edges();
  parse_ms_ = std::chrono::duration<float, std::milli>(std::chrono::steady_clock::now() - t0).count();
}

void Engine::forward_only(const int *graph, int B, int maxlen, const float *x_dev, float *graph_out) {
  state_epoch_++;
  begin_step(graph, B, maxlen);
  const bool reads_x = cell_ ? cell_->NX > 0 || cell_->XD > 0 : (cfg_.model != CAVS_MODEL_TREEFC || cfg_.use_x);
  if (reads_x && !x_dev) fail(CAVS_EINVAL, "vertex input feed is null");
  d_x_ = x_dev;
  check(cavs_event_record(ev_[0], stream_));
  fwd_out_ = graph_out ? graph_out : GO_.get();
  out_folded_ = false;
  head_chunked_ = false;
  model_forward();
  pop_ret(fwd_out_);
  check(cavs_event_record(ev_[1], stream_));
  ev_valid_ = true;
  ev_bwd_valid_ = false;
}

void Engine::update_bias_jobs(float lr, std::vector<cavs_task> *out, std::vector<const float *> *updated) {
  for (const BiasJob &j : bias_jobs_) updated->push_back(param(j.param).w);
  settle_bias_jobs(lr, out);
}

void Engine::backward_only(const float *dgraph_out, bool settle_biases) {
  if (!dgraph_out || N_ == 0) fail(CAVS_EINVAL, "backward_only needs d graph_out of a forward pass");
  state_epoch_++;
  d_dgo_ = dgraph_out;
  head_chunked_ = false;
  check(cavs_event_record(ev_[2], stream_));
  model_backward();
  if (settle_biases) settle_bias_jobs(0.f, nullptr);  // no update follows in here: the bias gradients are delivered now
  check(cavs_event_record(ev_[3], stream_));
  ev_bwd_valid_ = true;
}

// The forward rounds, the loss head and the backward rounds of a step (everything between the
// feeds and the parameter update).  While a graph is being recorded the timing events stay out of it.
void Engine::run_passes(bool backward) {
  if (!capturing_) check(cavs_event_record(ev_[0], stream_));
  fwd_out_ = GO_.get();
  out_folded_ = false;
  head_chunked_ = backward && !head_chunks_.empty() && !profile_ && !capturing_ && cfg_.loss == CAVS_LOSS_SOFTMAX;
  model_forward();
  pop_ret(GO_.get());
  if (!capturing_) check(cavs_event_record(ev_[1], stream_));
  ev_valid_ = !capturing_;
  head_forward_backward(backward);
  d_dgo_ = dGO_.get();
  did_backward_ = backward;
  ev_bwd_valid_ = false;
  if (backward) {
    if (!capturing_) check(cavs_event_record(ev_[2], stream_));
    model_backward();
    if (!capturing_) check(cavs_event_record(ev_[3], stream_));
    ev_bwd_valid_ = !capturing_;
  }
}

Engine::StepSig Engine::step_signature(const void *x, const void *labels, bool backward) const {
  StepSig g;
  g.x = x;
  g.labels = labels;
  g.xs = xs_.get();
  g.xs_prev = xs_prev_.get();
  g.backward = backward;
  g.emb_sparse_valid = emb_sparse_valid_;
  g.emb_cleared = emb_cleared_;
  g.upk_valid = upk_valid_;
  g.wfct_valid = wfct_valid_;
  g.emb_dirty_n = emb_dirty_n_;
  g.pairing = cfg_.pairing;
  g.e_ones_rows = e_ones_rows_;
  g.alloc_epoch = device_array_epoch().load();
  g.state_epoch = state_epoch_;
  return g;
}

Engine::StepState Engine::step_state() const {
  StepState st;
  st.did_backward = did_backward_;
  st.out_folded = out_folded_;
  st.emb_sparse_valid = emb_sparse_valid_;
  st.emb_cleared = emb_cleared_;
  st.upk_valid = upk_valid_;
  st.wfct_valid = wfct_valid_;
  st.tail_pending = tail_pending_;
  st.fwd_out = fwd_out_;
  st.d_dgo = d_dgo_;
  st.xs = xs_.get();
  st.emb_dirty_n = emb_dirty_n_;
  st.bias_jobs = bias_jobs_;
  st.pending_tasks = pending_tasks_;
  const double c[10] = {c_round_flops_, c_gather_rows_, c_scatter_rows_, c_gemm_flops_, c_gemm_flops_hinted_,
                        c_launches_,    c_gather_bytes_, c_scatter_bytes_, c_tail_rounds_, c_tail_launches_};
  std::copy(c, c + 10, st.counters);
  return st;
}

void Engine::restore_step_state(const StepState &st) {
  did_backward_ = st.did_backward;
  out_folded_ = st.out_folded;
  emb_sparse_valid_ = st.emb_sparse_valid;
  emb_cleared_ = st.emb_cleared;
  upk_valid_ = st.upk_valid;
  wfct_valid_ = st.wfct_valid;
  tail_pending_ = tail_pending_ || st.tail_pending;
  fwd_out_ = st.fwd_out;
  d_dgo_ = st.d_dgo;
  if (xs_.get() != st.xs) xs_.swap(xs_prev_);
  emb_dirty_n_ = st.emb_dirty_n;
  bias_jobs_ = st.bias_jobs;
  pending_tasks_ = st.pending_tasks;
  c_round_flops_ = st.counters[0];
  c_gather_rows_ = st.counters[1];
  c_scatter_rows_ = st.counters[2];
  c_gemm_flops_ = st.counters[3];
  c_gemm_flops_hinted_ = st.counters[4];
  c_launches_ = st.counters[5];
  c_gather_bytes_ = st.counters[6];
  c_scatter_bytes_ = st.counters[7];
  c_tail_rounds_ = st.counters[8];
  c_tail_launches_ = st.counters[9];
  ev_valid_ = ev_bwd_valid_ = false;
}

void Engine::step(const int *graph, int B, int maxlen, const void *x, const void *labels,
                  bool on_device, bool backward, float lr) {
  auto step_t0 = std::chrono::steady_clock::now();
  struct StepTimer {
    Engine *e;
    std::chrono::steady_clock::time_point t0;
    ~StepTimer() { e->host_step_ms_ = std::chrono::duration<float, std::milli>(std::chrono::steady_clock::now() - t0).count(); }
  } step_timer{this, step_t0};
  begin_step(graph, B, maxlen);
  const int N = N_, H = cfg_.H;
  const bool needs_x = cfg_.model != CAVS_MODEL_TREEFC || cfg_.use_x;
  const size_t xw = cfg_.model == CAVS_MODEL_TREEFC ? H : 1;
  if (needs_x && !x) fail(CAVS_EINVAL, "vertex input feed is null");
  if (cfg_.loss == CAVS_LOSS_SOFTMAX && !labels) fail(CAVS_EINVAL, "label feed is null");
  if (on_device) {
    d_x_ = static_cast<const float *>(x);
    d_labels_ = static_cast<const float *>(labels);
  } else {
    if (needs_x) {
      ensure(x_in_, grow((size_t)N * xw, x_in_.capacity()));
      check(cavs_memcpy_h2d(x_in_.get(), x, (size_t)N * xw * 4, stream_));
      d_x_ = x_in_.get();
    }
    if (cfg_.loss == CAVS_LOSS_SOFTMAX) {
      ensure(labels_in_, grow(N, labels_in_.capacity()));
      check(cavs_memcpy_h2d(labels_in_.get(), labels, (size_t)N * 4, stream_));
      d_labels_ = labels_in_.get();
    }
    // pageable sources: make sure the copies are done before the caller reuses them
    check(cavs_stream_sync(stream_));
  }

  // A batch structure seen before, on the same feed buffers, with the session in the state it was
  // in the last time: the passes below as one recorded graph of launches.
  Plan *plan = hit_plan_;
  const bool may_replay = cfg_.graph_replay && plan && on_device && !profile_ && pending_tasks_.empty() && !plan->graph_off;
  StepGraph *recorded = nullptr;
  bool record = false;
  StepSig sig;
  if (may_replay) {
    sig = step_signature(x, labels, backward);
    for (StepGraph &g : plan->graphs)
      if (g.sig == sig) recorded = &g;
    // (a plan whose signatures keep changing -- new feed buffers every step -- stops recording)
    if (!recorded) record = plan->recordings++ < 6;
  }
  if (recorded) {
    check(cavs_graph_launch(recorded->exec, stream_));
    restore_step_state(recorded->after);
    c_graph_replays_ += 1;
  } else if (record) {
    const StepState before = step_state();
    void *exec = nullptr;
    bool ok = false;
    check(cavs_graph_capture_begin(stream_));
    capturing_ = true;
    try {
      run_passes(backward);
      capturing_ = false;
      check(cavs_graph_capture_end(stream_, &exec));
      ok = true;
    } catch (const Error &e) {  // something in there had to wait for the stream (a buffer that grew): not this time
      const std::string why = e.what();
      const int left = capturing_ ? cavs_graph_capture_end(stream_, nullptr) : CAVS_OK;
      capturing_ = false;
      plan->graph_off = true;
      // (seen on ROCm 7.2: a capture that was invalidated cannot be ended, and the stream refuses
      // everything from then on -- better said once than met at every later call)
      if (left != CAVS_OK)
        fail(CAVS_EHIP, "recording the launches of a step failed (" + why + ") and the stream did not leave the failed capture (" +
                            cavs_last_error() + "): this session cannot go on; create it without graph_replay");
    }
    if (ok) {
      if (plan->graphs.size() >= 4) {
        cavs_graph_destroy(plan->graphs.front().exec);
        plan->graphs.erase(plan->graphs.begin());
      }
      plan->graphs.push_back({exec, sig, step_state()});
      check(cavs_graph_launch(exec, stream_));  // (recording enqueued nothing)
      c_graph_replays_ += 1;
    } else {
      restore_step_state(before);
      plan->graph_off = true;
      run_passes(backward);
    }
  } else {
    run_passes(backward);
  }
  if (backward) {
    aux_join();  // (the head's weight gradients)
    if (lr != 0.f) {
      // w -= lr * g (cavs/backend/op_impl_sgd.cu); the embedding table by its looked-up rows
      // only: every other row of its gradient is zero, so the dense update would not move it
      // all of it in one launch: the updates touch disjoint tensors
      std::vector<cavs_task> tasks;
      if (update_guard()) tasks.push_back({CAVS_TASK_GUARD, 0.f, 0, 0, 0, const_cast<int *>(update_guard()), nullptr, nullptr, nullptr});
      std::vector<std::string> by_job;
      for (const BiasJob &j : bias_jobs_) by_job.push_back(j.param);
      settle_bias_jobs(lr, &tasks);
      for (auto &kv : params_) {
        Param &p = *kv.second;
        if (std::find(by_job.begin(), by_job.end(), kv.first) != by_job.end()) continue;  // updated by the job that delivers its gradient
        if (kv.first == "Emb" && emb_dirty_n_ == N) {
          const int E = (int)(p.n / cfg_.V);
          if (emb_stamp_.capacity() < (size_t)cfg_.V) {
            emb_stamp_.reserve(cfg_.V);
            check(cavs_zero(emb_stamp_.get(), (size_t)cfg_.V * 4, stream_));
          }
          tasks.push_back({CAVS_TASK_EMBED_SGD, lr, N, E, ++emb_epoch_, p.w, p.g, xs_prev_.get(), emb_stamp_.get()});
          continue;
        }
        // the recurrent weights, a wide head's weights: the update and the copy the kernels read in one job
        if (update_jobs(p.w, p.g, lr, &tasks)) {
          // a caller's own tensor may be written behind the engine's back
          if (p.w != p.own_w.get()) (kv.first == "Wfc" ? wfct_valid_ : upk_valid_) = false;
          continue;
        }
        tasks.push_back({CAVS_TASK_SGD, lr, (long long)p.n, 0, 0, p.w, p.g, nullptr, nullptr});
      }
      check(cavs_run_tasks((int)tasks.size(), tasks.data(), stream_));
      c_launches_ += 1;
    } else {
      settle_bias_jobs(0.f, nullptr);
    }
  }
}

// FunctionPopRet (cavs/backend/op_impl_graphop.cu:304-318): GraphOutput[tids_to_jobids[t]] =
// ret[t].  Push's slab copy is folded in: the h half of the message slab is the return value.
void Engine::model_forward() {
  switch (cfg_.model) {
    case CAVS_MODEL_TREELSTM: treelstm_forward(); break;
    case CAVS_MODEL_LSTM: lstm_forward(); break;
    case CAVS_MODEL_CELL: cell_forward(); break;
    default: treefc_forward();
  }
}

void Engine::model_backward() {
  switch (cfg_.model) {
    case CAVS_MODEL_TREELSTM: treelstm_backward(); break;
    case CAVS_MODEL_LSTM: lstm_backward(); break;
    case CAVS_MODEL_CELL: cell_backward(); break;
    default: treefc_backward();
  }
}

void Engine::pop_ret(float *graph_out) {
  if (out_folded_) return;  // already written by the rounds
  scatter(graph_out, cfg_.H, d_t2j_, msg_.get(), mw_, N_, cfg_.H);
}

// ------------------------------------------------------------------ Tree-LSTM
// apps/paper/tree-lstm-cavs.cc:129-172.  Everything that does not depend on the children
// (Pull, EmbeddingLookup, x*W) is hoisted out of the round loop and done once for all N
// vertices in tensor-id order; rounds of leaves skip the child GEMMs because their
// gathered rows are zero.
// The fused round kernels need the batch scheduler's rounds (every vertex of an internal
// round has both children) and H in whole MFMA tiles.
int Engine::fused_rows() const {
  if (!(cfg_.opt & CAVS_OPT_BATCHING) || cfg_.H % 32 != 0) return 0;
  if (cell_) return 1 << 30;  // the generated kernels take rounds of any size
  if (cfg_.fused_round_rows < 0) return 0;
  // measured crossover with the separate launches: about 2400 rows at H=512, 1500 at H=1024
  return cfg_.fused_round_rows > 0 ? cfg_.fused_round_rows : (cfg_.H <= 512 ? 2048 : 1024);
}

void Engine::treelstm_forward() {
  const int N = N_, H = cfg_.H, E = E_;
  const float *W = param("W").w, *U = param("U").w, *Bv = param("Bv").w;
  const int fused = fused_rows();
  bool any_packed = false;
  if (Upk_.capacity() > 0)
    for (const Round &r : sched_->rounds) any_packed |= !leaf_round(r) && r.n <= fused && cavs_round_packed_ok(r.n, H);
  if (any_packed && !upk_valid_) {  // U was written by somebody else since the last update here
    cavs_task pack[2] = {{CAVS_TASK_SGD_PACK, 0.f, H, 3 * H, 0, Upk_.get(), const_cast<float *>(U), nullptr, nullptr},
                         {CAVS_TASK_SGD_PACK, 0.f, H, H, 0, Upk_.at((size_t)3 * H * H), const_cast<float *>(U) + (size_t)3 * H * H, nullptr,
                          nullptr}};
    check(cavs_run_tasks(2, pack, stream_));
    c_launches_ += 1;
    upk_valid_ = U == param("U").own_w.get();
  }
  // Pull of the word id, the lookup and x * W: one launch
  {
    ProfScope ps(this, K_GEMM);
    // (a leaf gathers zero rows, so its forget gates multiply zero: their columns of x * W are not wanted)
    check(cavs_embed_pull_sgemm(xW_.get(), 4 * H, e_.get(), ld_e_, xs_.get(), d_x_, d_t2j_, param("Emb").w, N, E, W, 4 * H, 4 * H,
                                sched_->leaf_prefix, 3 * H, stream_));
  }
  c_gemm_flops_ += 2.0 * N * 4 * H * E;
  c_gemm_flops_hinted_ += 2.0 * sched_->leaf_prefix * H * E;
  c_launches_ += 1;
  if (!sched_->batching) {  // leaves are interleaved with internal vertices: their child rows must read as zero
    check(cavs_zero(G_.get(), (size_t)N * 2 * 2 * H * 4, stream_));
    check(cavs_zero(hlr_.get(), (size_t)N * H * 4, stream_));
  }
  // with the fused path on, Push + FunctionPopRet ride along in the rounds' epilogues (also in the
  // gate launch of a round that runs its products as separate GEMMs)
  out_folded_ = fused > 0 && fwd_out_ != nullptr;
  float *go = out_folded_ ? fwd_out_ : nullptr;
  // the last rounds, a few vertices each: one launch for all of them
  const size_t tail_from = (tail_.first >= 0 && any_packed) ? (size_t)tail_.first : sched_->rounds.size();
  for (size_t rk = 0; rk < sched_->rounds.size(); rk++) {
    const Round &r = sched_->rounds[rk];
    if (rk == tail_from) {
      CAVS_TIMED(K_ROUND, cavs_treelstm_tail_fwd(pool_.get(), d_child_, d_pair_, xW_.get(), 4 * H, Upk_.get(), Bv, G_.get(), hlr_.get(),
                                                 gates_.get(), out_folded_ ? nullptr : msg_.get(), go, d_t2j_, d_tail_rows_,
                                                 (int)tail_.nrounds.size(), tail_.nrounds.data(), tail_.start.data(), tail_.count.data(),
                                                 tail_.flags.data(), tail_.max_rounds, H, reinterpret_cast<unsigned *>(tail_sync_.get()), kTailSpins, 0,
                                                 stream_));
      c_round_flops_ += tail_.flops;
      c_gather_rows_ += 2.0 * tail_.vertices;
      c_scatter_rows_ += tail_.vertices;
      c_launches_ += 1;
      c_tail_launches_ += 1;
      c_tail_rounds_ += (double)(sched_->rounds.size() - tail_from);
      tail_pending_ = true;
      break;
    }
    const size_t off = r.offset;
    // the message slab is only read back by FunctionPopRet; when the rounds write the output
    // rows themselves nobody reads it and the fused launches skip it
    float *msg = out_folded_ ? nullptr : msg_.at(off * 2 * H);
    if (leaf_round(r) && fused > 0) {  // (elementwise: a round of any size)
      CAVS_TIMED(K_GATES, cavs_treelstm_round_leaves_fwd(pool_.get(), d_pair_ + off, xW_.at(off * 4 * H), 4 * H, Bv, gates_.at(off * 6 * H),
                                                         msg, go, d_t2j_ + off, r.n, H, stream_));
      c_scatter_rows_ += r.n;
      c_launches_ += 1;
      continue;
    } else if (leaf_round(r)) {
      CAVS_TIMED(K_GATES, cavs_treelstm_gates_fwd(xW_.at(off * 4 * H), 4 * H, nullptr, nullptr, nullptr, Bv,
                                    gates_.at(off * 6 * H), msg, r.n, H, stream_));
    } else if (r.n <= fused) {
      // Gather, both recurrent products, the gates and Scatter in one launch
      if (any_packed && cavs_round_packed_ok(r.n, H))
        CAVS_TIMED(K_ROUND, cavs_treelstm_round_fwd_packed(pool_.get(), d_child_ + 2 * off, d_pair_ + off, xW_.at(off * 4 * H), 4 * H, U,
                                                           Upk_.get(), Bv, G_.at(2 * off * 2 * H), hlr_.at(off * H),
                                                           gates_.at(off * 6 * H), msg, go, d_t2j_ + off, r.n, H, stream_));
      else
        CAVS_TIMED(K_ROUND, cavs_treelstm_round_fwd(pool_.get(), d_child_ + 2 * off, d_pair_ + off, xW_.at(off * 4 * H), 4 * H, U, Bv,
                                                    G_.at(2 * off * 2 * H), hlr_.at(off * H), gates_.at(off * 6 * H), msg, go,
                                                    d_t2j_ + off, r.n, H, stream_));
      c_round_flops_ += 2.0 * r.n * H * 5.0 * H;
      c_gather_rows_ += 2.0 * r.n;
      c_scatter_rows_ += r.n;
      c_launches_ += 1;
      continue;
    } else {
      float *G = G_.at(2 * off * 2 * H), *hlr = hlr_.at(off * H);
      {
        ProfScope ps(this, K_GATHER);
        check(cavs_gather_children(G, hlr, pool_.get(), d_child_ + 2 * off, r.n, 2 * H, H, stream_));
      }
      c_gather_rows_ += 2.0 * r.n;
      c_gather_bytes_ += 2.0 * r.n * (16.0 * H + 4) + 4.0 * r.n * H;
      c_launches_ += 1;
      gemm(0, 0, r.n, 3 * H, H, hlr, H, U, 3 * H, 0.f, r_hU_.get(), 3 * H);
      gemm(0, 0, 2 * r.n, H, H, G, 2 * H, U + (size_t)3 * H * H, H, 0.f, r_hUf_.get(), H);
      if (fused > 0) {  // the gates with Scatter and Push / PopRet folded in
        CAVS_TIMED(K_GATES, cavs_treelstm_gates_fwd_scatter(xW_.at(off * 4 * H), 4 * H, r_hU_.get(), r_hUf_.get(), G, Bv, gates_.at(off * 6 * H),
                                                            msg, pool_.get(), d_pair_ + off, go, d_t2j_ + off, r.n, H, stream_));
        c_scatter_rows_ += r.n;
        c_launches_ += 1;
        continue;
      }
      CAVS_TIMED(K_GATES, cavs_treelstm_gates_fwd(xW_.at(off * 4 * H), 4 * H, r_hU_.get(), r_hUf_.get(), G, Bv,
                                    gates_.at(off * 6 * H), msg, r.n, H, stream_));
    }
    c_launches_ += 1;
    scatter(pool_.get(), 2 * H, d_pair_ + off, msg, 2 * H, r.n, 2 * H);
  }
}

void Engine::treelstm_backward() {
  const int N = N_, H = cfg_.H, E = E_;
  const float *W = param("W").w, *U = param("U").w;
  const int fused = fused_rows();
  // grad of Push is Pull: read through the list by the gate kernels of the fused path, or gathered up front
  const bool dret_folded = fused > 0;
  if (!dret_folded && !forest_) gather(dret_.get(), H, d_dgo_, H, d_t2j_, N, H);
  if (!sched_->batching) check(cavs_zero(dF_.get(), (size_t)N * 2 * H * 4, stream_));
  // one launch per round when the message flow is a forest (below); then, if every such launch has
  // a packed variant, the transposed weights are written tile-major instead of plain
  bool packed = forest_;
  for (const Round &r : sched_->rounds)
    if (!leaf_round(r) && !cavs_round_packed_ok(r.n, H)) packed = false;
  // one launch per round when the message flow is a forest: the roots' gate gradients first, then
  // every round hands d h, d c on to its children and does their gate gradients in its epilogue
  const bool folded = forest_;
  // (those of the roots depend on nothing the opening launch writes and ride in it)
  const bool roots_ride = folded && fused > 0 && H % 4 == 0 && n_orphans_ > 0;
  std::vector<cavs_task> opening;
  if (fused > 0) {  // U_iou^T and U_f^T: the B operand of the children products, k-major
    const int kind = packed ? CAVS_TASK_PACK_T : CAVS_TASK_TRANSPOSE;
    opening.push_back({kind, 0.f, H, 3 * H, 0, UT_.get(), const_cast<float *>(U), nullptr, nullptr});
    opening.push_back({kind, 0.f, H, H, 0, UT_.at((size_t)3 * H * H), const_cast<float *>(U) + (size_t)3 * H * H, nullptr, nullptr});
  }
  if (roots_ride)
    opening.push_back({CAVS_TASK_TREELSTM_GATES_ROWS, 0.f, n_orphans_, H, (long long)sched_->leaf_prefix | ((long long)(4 * H) << 32),
                       const_cast<int *>(d_orphans_), const_cast<float *>(d_dgo_), const_cast<int *>(d_t2j_), gates_.get(), G_.get(),
                       dxW_.get(), dF_.get(), dc_.get()});
  backward_prologue(opening, true);
  if (folded && !roots_ride) {
    CAVS_TIMED(K_GATES, cavs_treelstm_bwd_gates_rows(d_orphans_, n_orphans_, d_dgo_, d_t2j_, gates_.get(), G_.get(), dxW_.get(), 4 * H,
                                                     dF_.get(), dc_.get(), sched_->leaf_prefix, H, stream_));
    c_launches_ += 1;
  }
  // the first rounds of the backward pass, a few vertices each: one launch for all of them
  size_t tail_n = 0;
  if (folded && packed && tail_.first >= 0) {
    tail_n = sched_->rounds.size() - (size_t)tail_.first;
    // (the backward order is the forward order reversed: the launches' rounds are its first tail_n)
    if (sched_->bwd_rounds.size() < tail_n || sched_->bwd_rounds[tail_n - 1] != tail_.first) tail_n = 0;
  }
  if (tail_n > 0) {
    CAVS_TIMED(K_ROUND, cavs_treelstm_tail_bwd(dxW_.get(), 4 * H, dF_.get(), dc_.get(), UT_.get(), d_kid_rows_, gates_.get(), G_.get(), d_dgo_,
                                               d_t2j_, sched_->leaf_prefix, d_tail_rows_, (int)tail_.nrounds.size(), tail_.nrounds.data(),
                                               tail_.bstart.data(), tail_.bcount.data(), tail_.bflags.data(), tail_.max_rounds, H,
                                               reinterpret_cast<unsigned *>(tail_sync_.get()), kTailSpins, 0, stream_));
    c_gather_rows_ += tail_.vertices;
    c_round_flops_ += tail_.flops;
    c_scatter_rows_ += 2.0 * tail_.vertices;
    c_launches_ += 1;
    c_tail_launches_ += 1;
    c_tail_rounds_ += (double)tail_n;
    tail_pending_ = true;
  }
  for (size_t bi = tail_n; bi < sched_->bwd_rounds.size(); bi++) {
    const int k = sched_->bwd_rounds[bi];
    const Round &r = sched_->rounds[k];
    const size_t off = r.offset;
    if (folded) {
      c_gather_rows_ += r.n;
      if (leaf_round(r)) continue;
      CAVS_TIMED(K_ROUND, (packed ? cavs_treelstm_round_bwd_children_gates_packed : cavs_treelstm_round_bwd_children_gates)(
                              dxW_.get(), 4 * H, dF_.get(), dc_.get(), UT_.get(), d_kid_rows_ + 2 * off, gates_.get(), G_.get(), d_dgo_,
                              d_t2j_, (int)off, r.n, sched_->leaf_prefix, H, stream_));
      c_round_flops_ += 2.0 * r.n * H * 5.0 * H;
      c_scatter_rows_ += 2.0 * r.n;
      c_launches_ += 1;
      continue;
    }
    if (r.n <= fused) {
      // Gather of the message gradient, gate gradients and the Scatter of d c_child in one
      // launch; the children's d h (both products and their Scatter) in a second
      const bool leaf = leaf_round(r);
      const int *child = leaf ? nullptr : d_child_ + 2 * off;
      float *dxW = dxW_.at(off * 4 * H), *dF = leaf ? nullptr : dF_.at(2 * off * H);
      CAVS_TIMED(K_GATES, cavs_treelstm_round_bwd_gates(dpool_.get(), d_pair_ + off, child, dret_folded ? d_dgo_ : dret_.at(off * H),
                                                        dret_folded ? d_t2j_ + off : nullptr, gates_.at(off * 6 * H),
                                                        leaf ? nullptr : G_.at(2 * off * 2 * H), dxW, 4 * H, dF, r.n, H, stream_));
      c_gather_rows_ += r.n;
      c_launches_ += 1;
      if (!leaf) {
        CAVS_TIMED(K_ROUND, cavs_treelstm_round_bwd_children(dxW, 4 * H, dF, UT_.get(), child, dpool_.get(), r.n, H, stream_));
        c_round_flops_ += 2.0 * r.n * H * 5.0 * H;
        c_scatter_rows_ += 2.0 * r.n;
        c_launches_ += 1;
      }
      continue;
    }
    if (fused > 0) {
      // a round too large for the fused children launch: the same gate launch (it reads the message
      // gradient through the scatter list and hands d c on to the children's pool rows), the two
      // products as GEMMs, and the h halves scattered
      const bool leaf = leaf_round(r);
      float *dxW = dxW_.at(off * 4 * H), *dF = leaf ? nullptr : dF_.at(2 * off * H);
      CAVS_TIMED(K_GATES, cavs_treelstm_round_bwd_gates(dpool_.get(), d_pair_ + off, leaf ? nullptr : d_child_ + 2 * off, d_dgo_, d_t2j_ + off,
                                                        gates_.at(off * 6 * H), leaf ? nullptr : G_.at(2 * off * 2 * H), dxW, 4 * H, dF, r.n, H,
                                                        stream_));
      c_gather_rows_ += r.n;
      c_launches_ += 1;
      if (leaf) continue;
      gemm(0, 1, r.n, H, 3 * H, dxW, 4 * H, U, 3 * H, 0.f, r_dhlr_.get(), H);
      {
        float *ws = workspace(cavs_sgemm_splitk_workspace(2 * r.n, H, H));
        ProfScope ps(this, K_GEMM);
        check(cavs_sgemm_addrows(0, 1, 2 * r.n, H, H, dF, H, U + (size_t)3 * H * H, H, r_dhlr_.get(), H, 1, r_dG_.get(), 2 * H, ws,
                                 ws_.capacity() * 4, stream_));
      }
      c_gemm_flops_ += 2.0 * 2 * r.n * H * H;
      c_launches_ += 1;
      scatter(dpool_.get(), 2 * H, d_child_ + 2 * off, r_dG_.get(), 2 * H, 2 * r.n, H);
      continue;
    }
    // grad of Scatter is Gather on the recorded scatter list; rows without an entry read zero
    gather(r_dmsg_.get(), 2 * H, dpool_.get(), 2 * H, d_pair_ + off, r.n, 2 * H);
    if (leaf_round(r)) {
      CAVS_TIMED(K_GATES, cavs_treelstm_gates_bwd(r_dmsg_.get(), dret_.at(off * H), gates_.at(off * 6 * H), nullptr,
                                    dxW_.at(off * 4 * H), 4 * H, nullptr, nullptr, r.n, H, stream_));
      c_launches_ += 1;
      continue;
    }
    float *dxW = dxW_.at(off * 4 * H), *dF = dF_.at(2 * off * H);
    CAVS_TIMED(K_GATES, cavs_treelstm_gates_bwd(r_dmsg_.get(), dret_.at(off * H), gates_.at(off * 6 * H),
                                  G_.at(2 * off * 2 * H), dxW, 4 * H, dF, r_dG_.get(), r.n, H, stream_));
    c_launches_ += 1;
    // dh_lr = [d_i|d_o|d_u] * U_iou^T ;  dh_{l,r} = dh_lr + d_f{l,r} * U_f^T
    gemm(0, 1, r.n, H, 3 * H, dxW, 4 * H, U, 3 * H, 0.f, r_dhlr_.get(), H);
    {
      float *ws = workspace(cavs_sgemm_splitk_workspace(2 * r.n, H, H));
      ProfScope ps(this, K_GEMM);
      check(cavs_sgemm_addrows(0, 1, 2 * r.n, H, H, dF, H, U + (size_t)3 * H * H, H, r_dhlr_.get(), H, 1,
                               r_dG_.get(), 2 * H, ws, ws_.capacity() * 4, stream_));
    }
    c_gemm_flops_ += 2.0 * 2 * r.n * H * H;
    c_launches_ += 1;
    // grad of Gather(child) is Scatter on the recorded gather lists
    scatter(dpool_.get(), 2 * H, d_child_ + 2 * off, r_dG_.get(), 2 * H, 2 * r.n, 2 * H);
  }
  // weight gradients once over all rows (OPT_BATCHING semantics; without it the reference
  // accumulates the same sums round by round)
  // leaves contribute exact zeros to dU, and the f columns of their rows of dxW are exact zeros
  const int lp = sched_->leaf_prefix;
  float *dU = param("U").g;
  const bool bias_row = bias_row_ok();  // the ones column of e_ turns row E of dW into the column sums of dxW
  gemm_group_embedding_backward({
      {0, 1, N, E, 4 * H, 1.f, 0.f, dxW_.get(), 4 * H, W, 4 * H, de_.get(), E, CAVS_GEMM_A_ZERO, lp, 3 * H},
      // (all four padding columns of e_ take part, so that the product keeps 16-byte operand loads)
      {1, 0, bias_row ? ld_e_ : E, 4 * H, N, 1.f, 0.f, e_.get(), ld_e_, dxW_.get(), 4 * H, param("W").g, 4 * H, CAVS_GEMM_B_ZERO, lp,
       3 * H},
      {1, 0, H, 3 * H, N - lp, 1.f, 0.f, hlr_.at((size_t)lp * H), H, dxW_.at((size_t)lp * 4 * H), 4 * H, dU, 3 * H},
      {1, 0, H, H, 2 * (N - lp), 1.f, 0.f, G_.at((size_t)2 * lp * 2 * H), 2 * H, dF_.at((size_t)2 * lp * H), H,
       dU + (size_t)3 * H * H, H},
  }, E);
  // bias blocks [i|f|u|o] from dxW columns [i|o|u|f]
  if (bias_row) {
    // settled by the launch that ends the step (or right after this pass); block k of the row
    // ([i|o|u|f]) lands in bias block map[k] ([i|f|u|o])
    bias_jobs_.push_back({"Bv", param("W").g + param("W").n, 1, H, 4, 0 | (3 << 4) | (2 << 8) | (1 << 12)});
    return;
  }
  const int dst_block[4] = {0, 3, 2, 1};  // dxW block k ([i|o|u|f]) lands in bias block dst_block[k]
  const size_t cs_bytes = cavs_colsum_blocks_workspace(N, H, 4);
  float *cs_ws = workspace(cs_bytes);
  check(cavs_colsum_blocks(param("Bv").g, dxW_.get(), 4 * H, N, H, 4, dst_block, cs_ws, cs_bytes, stream_));
  c_launches_ += 2;
}

// The gradient of W lives in the engine's own array, which has the spare row.
bool Engine::bias_row_ok() const {
  if (cfg_.model != CAVS_MODEL_TREELSTM) return false;
  // free only while the extra rows stay inside the last row tile of the product (E = 300: yes;
  // E = 1024 would grow the 128-row tiling from 8 to 9 tiles)
  if ((E_ + 4 + 127) / 128 != (E_ + 127) / 128) return false;
  const Param &w = *params_.at("W");
  return w.g == w.own_g.get();
}

// One launch leaves the chunk sums; the job that ends the step adds them up in index order.
void Engine::bias_gradient(const std::string &name, const float *inp, int n, int w, DeviceArray<float> &parts, void *stream) {
  const size_t bytes = cavs_colsum_blocks_workspace(n, w, 1);
  if (parts.capacity() * 4 < bytes) {
    check(cavs_stream_sync(stream_));
    parts.reserve(bytes / 4 + 1);
  }
  check(cavs_colsum_blocks(nullptr, inp, w, n, w, 1, nullptr, parts.get(), parts.capacity() * 4, stream ? stream : stream_));
  c_launches_ += 1;
  bias_jobs_.push_back({name, parts.get(), cavs_colsum_parts(n), w, 1, 0});
}

// out [w] = column sums of inp [n, w], chunks of rows added in index order
void Engine::colsum_fixed(float *out, const float *inp, int n, int w) {
  if (w == 1) {  // a short vector to a scalar: one workgroup
    cavs_task t{CAVS_TASK_SUM_PARTS, 0.f, n, 1, 1, const_cast<float *>(inp), out, nullptr, nullptr};
    check(cavs_run_tasks(1, &t, stream_));
    c_launches_ += 1;
    return;
  }
  if (n <= 64) {  // a single chunk of rows: cavs_colsum adds nothing atomically
    check(cavs_colsum(out, inp, w, n, w, 0, stream_));
    c_launches_ += 1;
    return;
  }
  const int identity[1] = {0};
  const size_t bytes = cavs_colsum_blocks_workspace(n, w, 1);
  float *ws = workspace(bytes);
  check(cavs_colsum_blocks(out, inp, w, n, w, 1, identity, ws, bytes, stream_));
  c_launches_ += 2;
}

bool Engine::has_bias_job(const std::string &name) const {
  for (const BiasJob &j : bias_jobs_)
    if (j.param == name) return true;
  return false;
}

// Each pending row set -> the parameter's gradient, and the update of the parameter with it when
// lr != 0: as jobs of `tasks` if given, else as a launch of their own.
void Engine::settle_bias_jobs(float lr, std::vector<cavs_task> *tasks) {
  if (bias_jobs_.empty()) return;
  std::vector<cavs_task> own;
  for (const BiasJob &j : bias_jobs_) {
    Param &b = param(j.param);
    cavs_task t{CAVS_TASK_BLOCKS_SGD, lr, j.bw, j.nb, j.map | ((long long)j.parts << 32), lr != 0.f ? b.w : nullptr,
                const_cast<float *>(j.src), b.g, nullptr};
    (tasks ? *tasks : own).push_back(t);
  }
  bias_jobs_.clear();
  if (!own.empty()) {
    check(cavs_run_tasks((int)own.size(), own.data(), stream_));
    c_launches_ += 1;
  }
}

// EmbeddingLookup_grad (cavs/backend/op_impl_embedding.cu:58-92): scatter-add of the rows of
// de into a zeroed table.  The table is kept zero outside the rows of the previous step, so
// clearing it costs those rows, not the vocabulary.
// The transposed weights of the fused backward rounds and -- `with_embedding` -- the clearing of
// the embedding gradient (the rows the previous step looked up) do not depend on each other:
// one launch.
void Engine::backward_prologue(std::vector<cavs_task> tasks, bool with_embedding) {
  tasks.insert(tasks.end(), pending_tasks_.begin(), pending_tasks_.end());
  pending_tasks_.clear();
  if (with_embedding) {
    Param &emb = param("Emb");
    if (emb.g == emb.own_g.get() && emb_sparse_valid_) {
      if (emb_dirty_n_ > 0)
        tasks.push_back({CAVS_TASK_ZERO_ROWS, 0.f, emb_dirty_n_, (long long)(emb.n / cfg_.V), 0, emb.g, xs_prev_.get(), nullptr, nullptr});
      emb_cleared_ = true;
    }
  }
  if (tasks.empty()) return;
  CAVS_TIMED(K_OTHER, cavs_run_tasks((int)tasks.size(), tasks.data(), stream_));
  c_launches_ += 1;
}

// `products[0]` is de = dxW * W^T; its rows go on into the embedding gradient in the launch that
// reduces the group's K splits (cavs_sgemm_group_embed_bwd).
void Engine::gemm_group_embedding_backward(const std::vector<cavs_gemm_desc> &products, int E) {
  Param &emb = param("Emb");
  const bool owned = emb.g == emb.own_g.get();
  if (emb_cleared_) {
    emb_cleared_ = false;  // the prologue of this backward pass did it
  } else if (owned && emb_sparse_valid_) {
    if (emb_dirty_n_ > 0) check(cavs_embed_zero_rows(emb.g, xs_prev_.get(), emb_dirty_n_, E, stream_));
    c_launches_ += 1;
  } else {
    check(cavs_zero(emb.g, emb.n * 4, stream_));
    c_launches_ += 1;
  }
  const int count = (int)products.size();
  float *ws = workspace(cavs_sgemm_group_workspace(count, products.data()));
  {
    ProfScope ps(this, K_GEMM);
    check(cavs_sgemm_group_embed_bwd(count, products.data(), 0, emb.g, xs_.get(), ws, ws_.capacity() * 4, stream_));
  }
  for (const cavs_gemm_desc &q : products) {
    c_gemm_flops_ += 2.0 * q.M * q.N * q.K;
    c_gemm_flops_hinted_ += hinted_flops(q);
  }
  c_launches_ += 2;
  xs_.swap(xs_prev_);  // this step's ids: the rows that are dirty now
  emb_dirty_n_ = N_;
  emb_sparse_valid_ = owned;
}

// ------------------------------------------------------------------ chain LSTM
// apps/paper/seq-lstm-cavs.cc:62-86
void Engine::lstm_forward() {
  const int N = N_, H = cfg_.H;
  const float *Wx = param("W").w, *Wh = Wx + (size_t)4 * H * H, *Bv = param("Bv").w;
  {  // Pull of the token id, the lookup and x * W_x: one launch
    ProfScope ps(this, K_GEMM);
    check(cavs_embed_pull_sgemm(xW_.get(), 4 * H, e_.get(), H, xs_.get(), d_x_, d_t2j_, param("Emb").w, N, H, Wx, 4 * H, 4 * H, 0, 0,
                                stream_));
  }
  c_gemm_flops_ += 2.0 * N * 4 * H * H;
  c_launches_ += 1;
  if (!sched_->batching) check(cavs_zero(G_.get(), (size_t)N * 2 * H * 4, stream_));
  const int fused = fused_rows();
  bool any_packed = false;
  if (Upk_.capacity() > 0)
    for (const Round &r : sched_->rounds) any_packed |= !leaf_round(r) && r.n <= fused && cavs_lstm_round_packed_ok(r.n, H);
  if (any_packed && !upk_valid_) {  // W' was written by somebody else since the last update here
    cavs_task pack{CAVS_TASK_SGD_PACK, 0.f, H, 4 * H, 0, Upk_.get(), const_cast<float *>(Wh), nullptr, nullptr};
    check(cavs_run_tasks(1, &pack, stream_));
    c_launches_ += 1;
    upk_valid_ = Wx == param("W").own_w.get();
  }
  out_folded_ = fused > 0 && sched_->max_round <= fused && fwd_out_ != nullptr;
  float *go = out_folded_ ? fwd_out_ : nullptr;
  for (const Round &r : sched_->rounds) {
    const size_t off = r.offset;
    float *a = xW_.at(off * 4 * H), *msg = msg_.at(off * 2 * H), *G = nullptr;
    if (r.n <= fused) {  // one launch: Gather, h*W', gates, Scatter, Push/PopRet
      if (leaf_round(r)) {
        CAVS_TIMED(K_GATES, cavs_lstm_round_leaves_fwd(pool_.get(), d_pair_ + off, a, 4 * H, Bv, gates_.at(off * 5 * H), msg, go,
                                                       d_t2j_ + off, r.n, H, stream_));
      } else {
        const bool pk = any_packed && cavs_lstm_round_packed_ok(r.n, H);
        CAVS_TIMED(K_ROUND, (pk ? cavs_lstm_round_fwd_packed : cavs_lstm_round_fwd)(
                                pool_.get(), d_child_ + off, d_pair_ + off, a, 4 * H, pk ? Upk_.get() : Wh, Bv, G_.at(off * 2 * H),
                                gates_.at(off * 5 * H), msg, go, d_t2j_ + off, r.n, H, stream_));
        c_round_flops_ += 2.0 * r.n * H * 4.0 * H;
        c_gather_rows_ += r.n;
      }
      c_scatter_rows_ += r.n;
      c_launches_ += 1;
      continue;
    }
    if (!leaf_round(r)) {
      G = G_.at(off * 2 * H);
      gather(G, 2 * H, pool_.get(), 2 * H, d_child_ + off, r.n, 2 * H);
      gemm(0, 0, r.n, 4 * H, H, G, 2 * H, Wh, 4 * H, 1.f, a, 4 * H);  // a += h_p * W'
    }
    CAVS_TIMED(K_GATES, cavs_lstm_gates_fwd(a, 4 * H, nullptr, G, Bv, gates_.at(off * 5 * H), msg, r.n, H, stream_));
    c_launches_ += 1;
    scatter(pool_.get(), 2 * H, d_pair_ + off, msg, 2 * H, r.n, 2 * H);
  }
}

void Engine::lstm_backward() {
  const int N = N_, H = cfg_.H;
  const float *Wx = param("W").w, *Wh = Wx + (size_t)4 * H * H;
  const int fused = fused_rows();
  const bool dret_folded = fused > 0 && sched_->max_round <= fused;
  if (!dret_folded && !forest_) gather(dret_.get(), H, d_dgo_, H, d_t2j_, N, H);
  bool packed = forest_;  // as in treelstm_backward
  for (const Round &r : sched_->rounds)
    if (!leaf_round(r) && !cavs_lstm_round_packed_ok(r.n, H)) packed = false;
  if (fused > 0) {  // W'^T: the B operand of d h_prev = da * W'^T, k-major
    backward_prologue({{packed ? CAVS_TASK_PACK_T : CAVS_TASK_TRANSPOSE, 0.f, H, 4 * H, 0, UT_.get(), const_cast<float *>(Wh), nullptr,
                        nullptr}},
                      true);
  } else {
    backward_prologue({}, true);
  }
  const bool folded = forest_;  // one launch per round, as in treelstm_backward
  // a wide head in chunks: d h comes in slab order, chunk by chunk, the last rounds' first
  const float *dret = head_chunked_ ? dret_.get() : d_dgo_;
  const int *dret_rows = head_chunked_ ? cell_iota_.get() : d_t2j_;
  int chunk = head_chunked_ ? (int)head_chunks_.size() : 0;
  if (folded && !head_chunked_) {
    CAVS_TIMED(K_GATES, cavs_lstm_bwd_gates_rows(d_orphans_, n_orphans_, d_dgo_, d_t2j_, gates_.get(), G_.get(), dxW_.get(), 4 * H,
                                                 dc_.get(), sched_->leaf_prefix, H, stream_));
    c_launches_ += 1;
  }
  for (int k : sched_->bwd_rounds) {
    const Round &r = sched_->rounds[k];
    const size_t off = r.offset;
    float *da = dxW_.at(off * 4 * H);
    while (head_chunked_ && chunk > 0 && (chunk == (int)head_chunks_.size() || k - 1 < head_chunks_[chunk].round0)) {
      // a round's launch also runs the gate gradients of its rows' children, the rows of the round
      // before: that round's chunk must have its d h.  Then the rows of the chunk nobody sends a
      // gradient to.
      chunk--;
      const HeadChunk &h = head_chunks_[chunk];
      check(cavs_stream_wait_event(stream_, chunk_done_ev_[chunk]));
      if (h.orph1 > h.orph0) {
        check(cavs_lstm_bwd_gates_rows(d_orphans_ + h.orph0, h.orph1 - h.orph0, dret, dret_rows, gates_.get(), G_.get(), dxW_.get(), 4 * H,
                                       dc_.get(), sched_->leaf_prefix, H, stream_));
        c_launches_ += 1;
      }
    }
    if (folded) {
      c_gather_rows_ += r.n;
      if (leaf_round(r)) continue;
      CAVS_TIMED(K_ROUND, (packed ? cavs_lstm_round_bwd_children_gates_packed : cavs_lstm_round_bwd_children_gates)(
                              dxW_.get(), 4 * H, dc_.get(), UT_.get(), d_kid_rows_ + off, gates_.get(), G_.get(), dret, dret_rows, (int)off,
                              r.n, sched_->leaf_prefix, H, stream_));
      c_round_flops_ += 2.0 * r.n * H * 4.0 * H;
      c_scatter_rows_ += r.n;
      c_launches_ += 1;
      continue;
    }
    if (r.n <= fused) {
      const bool leaf = leaf_round(r);
      const int *child = leaf ? nullptr : d_child_ + off;
      CAVS_TIMED(K_GATES, cavs_lstm_round_bwd_gates(dpool_.get(), d_pair_ + off, child, dret_folded ? d_dgo_ : dret_.at(off * H),
                                                    dret_folded ? d_t2j_ + off : nullptr, gates_.at(off * 5 * H),
                                                    leaf ? nullptr : G_.at(off * 2 * H), da, 4 * H, r.n, H, stream_));
      c_gather_rows_ += r.n;
      c_launches_ += 1;
      if (!leaf) {
        CAVS_TIMED(K_ROUND, cavs_round_bwd_children(da, 4 * H, 4 * H, UT_.get(), H, 1, child, dpool_.get(), 2 * H, r.n, H, stream_));
        c_round_flops_ += 2.0 * r.n * H * 4.0 * H;
        c_scatter_rows_ += r.n;
        c_launches_ += 1;
      }
      continue;
    }
    gather(r_dmsg_.get(), 2 * H, dpool_.get(), 2 * H, d_pair_ + off, r.n, 2 * H);
    if (leaf_round(r)) {
      CAVS_TIMED(K_GATES, cavs_lstm_gates_bwd(r_dmsg_.get(), dret_.at(off * H), gates_.at(off * 5 * H), nullptr, da, 4 * H,
                                nullptr, r.n, H, stream_));
      c_launches_ += 1;
      continue;
    }
    CAVS_TIMED(K_GATES, cavs_lstm_gates_bwd(r_dmsg_.get(), dret_.at(off * H), gates_.at(off * 5 * H), G_.at(off * 2 * H), da,
                              4 * H, r_dG_.get(), r.n, H, stream_));
    c_launches_ += 1;
    gemm(0, 1, r.n, H, 4 * H, da, 4 * H, Wh, 4 * H, 0.f, r_dG_.get(), 2 * H);  // dh_p = da * W'^T
    scatter(dpool_.get(), 2 * H, d_child_ + off, r_dG_.get(), 2 * H, r.n, 2 * H);
  }
  const int lp = sched_->leaf_prefix;
  float *dW = param("W").g;
  gemm_group_embedding_backward({
      {0, 1, N, H, 4 * H, 1.f, 0.f, dxW_.get(), 4 * H, Wx, 4 * H, de_.get(), H},
      {1, 0, H, 4 * H, N, 1.f, 0.f, e_.get(), H, dxW_.get(), 4 * H, dW, 4 * H},
      {1, 0, H, 4 * H, N - lp, 1.f, 0.f, G_.at((size_t)lp * 2 * H), 2 * H, dxW_.at((size_t)lp * 4 * H), 4 * H,
       dW + (size_t)4 * H * H, 4 * H},
  }, H);
  bias_gradient("Bv", dxW_.get(), N, 4 * H, bias_parts_);
}

// ------------------------------------------------------------------ Tree-FC
// apps/paper/tree-fc-cavs.cc:28-36 (optionally with a bias and a Pull'ed input row)
void Engine::treefc_forward() {
  const int N = N_, H = cfg_.H;
  const float *W = param("W").w;
  const float *Bv = cfg_.use_bias ? param("Bv").w : nullptr;
  if (cfg_.use_x) gather(xs_.get(), H, d_x_, H, d_t2j_, N, H);
  if (!sched_->batching) check(cavs_zero(G_.get(), (size_t)N * 2 * H * 4, stream_));
  const int fused = fused_rows();
  out_folded_ = fused > 0 && sched_->max_round <= fused && fwd_out_ != nullptr;
  float *go = out_folded_ ? fwd_out_ : nullptr;
  for (const Round &r : sched_->rounds) {
    const size_t off = r.offset;
    const float *xin = cfg_.use_x ? xs_.at(off * H) : nullptr;
    float *msg = msg_.at(off * H);
    if (r.n <= fused) {  // one launch: Gather, [h_l;h_r]*W, activation, Scatter, Push/PopRet
      if (leaf_round(r)) {
        CAVS_TIMED(K_GATES, cavs_treefc_round_leaves_fwd(pool_.get(), d_pair_ + off, Bv, xin, msg, go, d_t2j_ + off, r.n, H, cfg_.act,
                                                         stream_));
      } else {
        CAVS_TIMED(K_ROUND, cavs_treefc_round_fwd(pool_.get(), d_child_ + 2 * off, d_pair_ + off, W, Bv, xin, G_.at(2 * off * H), msg, go,
                                                  d_t2j_ + off, r.n, H, cfg_.act, stream_));
        c_round_flops_ += 2.0 * r.n * H * 2.0 * H;
        c_gather_rows_ += 2.0 * r.n;
      }
      c_scatter_rows_ += r.n;
      c_launches_ += 1;
      continue;
    }
    if (leaf_round(r)) {
      CAVS_TIMED(K_GATES, cavs_treefc_fwd(nullptr, Bv, xin, msg, r.n, H, cfg_.act, stream_));
    } else {
      float *G = G_.at(2 * off * H);  // row b = [G0 | G1] of vertex b
      {
        ProfScope ps(this, K_GATHER);
        check(cavs_gather_children(G, nullptr, pool_.get(), d_child_ + 2 * off, r.n, H, 0, stream_));
      }
      c_gather_rows_ += 2.0 * r.n;
      c_gather_bytes_ += 2.0 * r.n * (8.0 * H + 4);
      c_launches_ += 1;
      gemm(0, 0, r.n, H, 2 * H, G, 2 * H, W, H, 0.f, r_z_.get(), H);
      CAVS_TIMED(K_GATES, cavs_treefc_fwd(r_z_.get(), Bv, xin, msg, r.n, H, cfg_.act, stream_));
    }
    c_launches_ += 1;
    scatter(pool_.get(), H, d_pair_ + off, msg, H, r.n, H);
  }
}

void Engine::treefc_backward() {
  const int N = N_, H = cfg_.H;
  const float *W = param("W").w;
  const int fused = fused_rows();
  const bool dret_folded = fused > 0 && sched_->max_round <= fused;
  if (!dret_folded && !forest_) gather(dret_.get(), H, d_dgo_, H, d_t2j_, N, H);
  if (fused > 0) {  // W^T [H, 2H]: the B operand of d[h_l;h_r] = dz * W^T, k-major
    backward_prologue({{CAVS_TASK_TRANSPOSE, 0.f, 2 * H, H, 0, UT_.get(), const_cast<float *>(W), nullptr, nullptr}}, false);
  } else {
    backward_prologue({}, false);
  }
  const bool folded = forest_;  // one launch per round, as in treelstm_backward
  if (folded) {
    CAVS_TIMED(K_GATES, cavs_treefc_bwd_rows(d_orphans_, n_orphans_, d_dgo_, d_t2j_, msg_.get(), dxW_.get(), H, cfg_.act, stream_));
    c_launches_ += 1;
  }
  for (int k : sched_->bwd_rounds) {
    const Round &r = sched_->rounds[k];
    const size_t off = r.offset;
    float *dz = dxW_.at(off * H);
    if (folded) {
      c_gather_rows_ += r.n;
      if (leaf_round(r)) continue;
      CAVS_TIMED(K_ROUND, cavs_treefc_round_bwd_children_act(dxW_.get(), UT_.get(), d_kid_rows_ + 2 * off, msg_.get(), d_dgo_, d_t2j_,
                                                             (int)off, r.n, H, cfg_.act, stream_));
      c_round_flops_ += 2.0 * r.n * H * 2.0 * H;
      c_scatter_rows_ += 2.0 * r.n;
      c_launches_ += 1;
      continue;
    }
    if (r.n <= fused) {
      CAVS_TIMED(K_GATES, cavs_treefc_round_bwd(dpool_.get(), d_pair_ + off, dret_folded ? d_dgo_ : dret_.at(off * H),
                                                dret_folded ? d_t2j_ + off : nullptr, msg_.at(off * H), dz, r.n, H, cfg_.act, stream_));
      c_gather_rows_ += r.n;
      c_launches_ += 1;
      if (!leaf_round(r)) {
        CAVS_TIMED(K_ROUND, cavs_round_bwd_children(dz, H, H, UT_.get(), 2 * H, 2, d_child_ + 2 * off, dpool_.get(), H, r.n, H, stream_));
        c_round_flops_ += 2.0 * r.n * H * 2.0 * H;
        c_scatter_rows_ += 2.0 * r.n;
        c_launches_ += 1;
      }
      continue;
    }
    gather(r_dmsg_.get(), H, dpool_.get(), H, d_pair_ + off, r.n, H);
    CAVS_TIMED(K_GATES, cavs_treefc_bwd(r_dmsg_.get(), dret_.at(off * H), msg_.at(off * H), dz, r.n, H, cfg_.act, stream_));
    c_launches_ += 1;
    if (leaf_round(r)) continue;
    gemm(0, 1, r.n, 2 * H, H, dz, H, W, H, 0.f, r_dG_.get(), 2 * H);
    scatter(dpool_.get(), H, d_child_ + 2 * off, r_dG_.get(), H, 2 * r.n, H);
  }
  const int lp = sched_->leaf_prefix;
  gemm_splitk(1, 0, 2 * H, H, N - lp, G_.at((size_t)2 * lp * H), 2 * H, dxW_.at((size_t)lp * H), H,
              param("W").g, H);
  if (cfg_.use_bias) {
    bias_gradient("Bv", dxW_.get(), N, H, bias_parts_);
  }
}

// ------------------------------------------------------------------ a vertex function on generated kernels
// The general shape (cell.h): x * W for all vertices up front, then per round one launch per cell of
// the chain (a function of one stage is a chain of one) that gathers, multiplies, runs the
// elementwise part and scatters.  Backward, a function of one stage over a batch whose message
// flow is a forest takes one launch per round, which hands d(state) on to the children and runs
// their elementwise part; anything else two launches per round and cell, with the message
// gradients going through the gradients of the rows the cells write.  Then the weight gradients as
// products over all rows.
void Engine::cell_launch(int ci, int k, unsigned gx, unsigned gy, unsigned gz, unsigned block, long off, long n, const int *rows, const float *go) {
  CellStage &st = cells_[ci];
  const CellSpec &c = *st.spec;
  const bool first = ci == 0, last = ci + 1 == (int)cells_.size();
  union Slot {
    const void *p;
    long long i;
  } a[CA_SLOTS];
  std::memset(a, 0, sizeof a);
  // a cell in the middle of a chain gathers row v of the cell before and writes row v of its own
  a[CA_POOL].p = last ? pool_.get() : st.rows.get();
  a[CA_PAIR].p = last ? d_pair_ : cell_iota_.get();
  a[CA_DPOOL].p = last ? dpool_.get() : st.drows.get();
  a[CA_POOL_IN].p = first ? pool_.get() : cells_[ci - 1].rows.get();
  a[CA_CHILD].p = first ? d_child_ : cell_iota_.get();
  a[CA_DPOOL_IN].p = first ? dpool_.get() : cells_[ci - 1].drows.get();
  a[CA_KIDS].p = first ? d_kid_rows_ : cell_iota_.get();
  {
    // the cell whose rows this one gathers
    const int pi = first ? (int)cells_.size() - 1 : ci - 1;
    CellStage &ft = cells_[pi];
    a[CA_FT_SV].p = ft.sv.get();
    a[CA_FT_D].p = ft.d.get();
    a[CA_FT_DS].p = ft.ds.get();
    a[CA_FT_POOL_IN].p = pi == 0 ? pool_.get() : cells_[pi - 1].rows.get();
    a[CA_FT_CHILD].p = pi == 0 ? d_child_ : cell_iota_.get();
    a[CA_FT_KIDS].p = pi == 0 ? d_kid_rows_ : cell_iota_.get();
  }
  a[CA_T2J].p = d_t2j_;
  a[CA_ROWS].p = rows;
  a[CA_XW].p = xW_.get();
  a[CA_SV].p = st.sv.get();
  a[CA_ASRC].p = st.asrc.get();
  a[CA_GO].p = go;
  a[CA_D].p = st.d.get();
  a[CA_DS].p = st.ds.get();
  a[CA_BT].p = st.bt.get();
  a[CA_COLSUM].p = st.colsum.get();
  a[CA_X].p = d_x_;
  a[CA_OFF].i = off;
  a[CA_N].i = n;
  for (size_t i = 0; i < c.params.size(); i++) {
    const Param &p = param(c.params[i].name);
    a[CA_PARAM0 + i].p = p.w;
    a[CA_PARAM0 + CA_MAX_PARAMS + i].p = p.g;
  }
  check(cavs_cell_launch(st.module, k, gx, gy, gz, block, a, sizeof a, stream_));
  c_launches_ += 1;
}

void Engine::cell_forward() {
  const CellSpec &c0 = *cells_[0].spec;
  const int N = N_, H = cfg_.H;
  if (!sched_->batching) fail(CAVS_EUNSUPPORTED, "the lowered vertex function needs the batch scheduler (OPT_BATCHING)");
  if (c0.NX > 0) {
    ProfScope ps(this, K_GEMM);
    check(cavs_embed_pull_sgemm(xW_.get(), c0.NX * H, e_.get(), ld_e_, xs_.get(), d_x_, d_t2j_, param("Emb").w, N, E_,
                                param(c0.params[c0.W.param].name).w + c0.W.offset, c0.NX * H, c0.NX * H, 0, 0, stream_));
    c_gemm_flops_ += 2.0 * N * c0.NX * H * E_;
    c_launches_ += 1;
  }
  out_folded_ = true;  // the rounds write the pushed value by vertex id themselves
  for (size_t ci = 0; ci < cells_.size(); ci++) {
    // the weights may have changed since the last step (the caller's optimizer writes them): both
    // tile-major copies are rewritten, a few microseconds
    ProfScope ps(this, K_OTHER);
    const CellSpec &c = *cells_[ci].spec;
    cell_launch((int)ci, CK_PACK, (unsigned)(((size_t)2 * c.blocks() * H * H / 4 + 255) / 256), 1, 1, 256, 0, 0, nullptr, fwd_out_);
  }
  for (const Round &r : sched_->rounds)
    for (size_t ci = 0; ci < cells_.size(); ci++) {
      const CellSpec &c = *cells_[ci].spec;
      if (ci == 0 && leaf_round(r)) {  // (a later cell's one child is the vertex itself: it always has it)
        ProfScope ps(this, K_GATES);
        cell_launch(0, CK_LEAVES, (unsigned)(((size_t)r.n * H + 255) / 256), 1, 1, 256, r.offset, r.n, nullptr, fwd_out_);
      } else {
        ProfScope ps(this, K_ROUND);
        cell_launch((int)ci, CK_FWD, H / 16, (r.n + 15) / 16, 1, 64u * c.waves, r.offset, r.n, nullptr, fwd_out_);
        c_round_flops_ += 2.0 * r.n * c.terms() * H * H;
        c_gather_rows_ += (double)c.K * r.n;
      }
      c_scatter_rows_ += r.n;
    }
}

void Engine::cell_backward() {
  const CellSpec &c0 = *cells_[0].spec;
  const int N = N_, H = cfg_.H, lp = sched_->leaf_prefix;
  const int L = (int)cells_.size();
  backward_prologue({}, c0.NX > 0);
  // a parameter F reads only parts of: the rest of its gradient is zero
  {
    std::vector<long> covered(c0.params.size(), 0);
    if (c0.NX > 0) covered[c0.W.param] += (long)E_ * c0.NX * H;
    std::vector<std::pair<int, long>> seen;
    for (const CellStage &st : cells_) {
      for (const CellProduct &p : st.spec->products)
        for (const CellTerm &t : p.terms) {
          const auto key = std::make_pair(p.B.param, p.B.offset + t.brow * p.ldb + p.col);
          if (std::find(seen.begin(), seen.end(), key) != seen.end()) continue;
          seen.push_back(key);
          covered[p.B.param] += (long)H * H;
        }
      for (const CellBias &b : st.spec->biases)
        if (!b.add) covered[b.ref.param] += H;
    }
    for (size_t i = 0; i < c0.params.size(); i++)
      if (c0.params[i].name != "Emb" && covered[i] < c0.params[i].size) {
        check(cavs_zero(param(c0.params[i].name).g, (size_t)c0.params[i].size * 4, stream_));
        c_launches_ += 1;
      }
  }
  if (forest_) {
    // every message is read exactly once: a cell's launch completes the gradient of the rows it
    // gathered -- the states of the round's children for the first cell, the rows of the cell before
    // for the others -- and runs the elementwise part of the cell that wrote them at once.  The
    // vertices without a reader go first.
    if (n_orphans_ > 0) {
      ProfScope ps(this, K_GATES);
      cell_launch(L - 1, CK_BWD_ROWS, (unsigned)(((size_t)n_orphans_ * H + 255) / 256), 1, 1, 256, 0, n_orphans_, d_orphans_, d_dgo_);
    }
    for (int k : sched_->bwd_rounds) {
      const Round &r = sched_->rounds[k];
      c_gather_rows_ += r.n;
      for (int ci = L - 1; ci >= 0; ci--) {
        if (ci == 0 && leaf_round(r)) continue;
        const CellSpec &c = *cells_[ci].spec;
        ProfScope ps(this, K_ROUND);
        cell_launch(ci, CK_BWD, H / 16, (r.n + 15) / 16, 1, 64u * c.waves, r.offset, r.n, nullptr, d_dgo_);
        c_round_flops_ += 2.0 * r.n * c.terms() * H * H;
        c_scatter_rows_ += (double)c.K * r.n;
      }
    }
  } else {
    // any other batch: two launches per round and cell, the message gradients going through the
    // gradient of the rows the cells write, as in the reference (rows of the message pool nobody
    // wrote read as zero)
    check(cavs_zero(dpool_.get(), (size_t)N * mw_ * 4, stream_));
    c_launches_ += 1;
    for (int k : sched_->bwd_rounds) {
      const Round &r = sched_->rounds[k];
      for (int ci = L - 1; ci >= 0; ci--) {
        const CellSpec &c = *cells_[ci].spec;
        {
          ProfScope ps(this, K_GATES);
          cell_launch(ci, CK_BWD_GATES, (unsigned)(((size_t)r.n * H + 255) / 256), 1, 1, 256, r.offset, r.n, nullptr, d_dgo_);
        }
        c_gather_rows_ += r.n;
        if (ci == 0 && leaf_round(r)) continue;
        ProfScope ps(this, K_ROUND);
        cell_launch(ci, CK_BWD_POOL, H / 16, (r.n + 15) / 16, 1, 64u * c.waves, r.offset, r.n, nullptr, d_dgo_);
        c_round_flops_ += 2.0 * r.n * c.terms() * H * H;
        c_scatter_rows_ += (double)c.K * r.n;
      }
    }
  }
  // the weight gradients, once over all rows.  A product that writes where an earlier one of the
  // list wrote adds to it, one launch later (a weight block several products read; d e of several
  // cells); the rest go up to eight to a launch.
  std::vector<std::vector<cavs_gemm_desc>> waves(1);
  struct Written {
    const float *first;
    int n, ldc, times;
  };
  std::vector<Written> written;
  auto add = [&](cavs_gemm_desc d) {
    int before = 0;
    bool known = false;
    for (Written &w : written)
      if (w.first == d.C) {
        if (w.n != d.N || w.ldc != d.ldc)
          fail(CAVS_EUNSUPPORTED, "products of the lowered vertex function read overlapping but different blocks of one weight");
        before = w.times++;
        known = true;
      }
    if (!known) written.push_back({d.C, d.N, d.ldc, 1});
    d.beta = before ? 1.f : 0.f;
    if ((int)waves.size() <= before) waves.resize(before + 1);
    waves[before].push_back(d);
  };
  if (c0.NX > 0) {
    float *W = param(c0.params[c0.W.param].name).w + c0.W.offset, *dW = param(c0.params[c0.W.param].name).g + c0.W.offset;
    // d e first: the launch that reduces the first group of a function of one stage also scatters it into the table's gradient
    for (const CellStage &st : cells_) {
      const CellSpec &c = *st.spec;
      if (c.xw_hi <= c.xw_lo) continue;
      const int w = (c.xw_hi - c.xw_lo) * H;
      add({0, 1, N, E_, w, 1.f, 0.f, st.d.at((size_t)c.xw_lo * H), c.ND * H, W + (size_t)c.xw_lo * H, c.NX * H, de_.get(), E_});
    }
    for (const CellStage &st : cells_) {
      const CellSpec &c = *st.spec;
      if (c.xw_hi <= c.xw_lo) continue;
      const int w = (c.xw_hi - c.xw_lo) * H;
      add({1, 0, E_, w, N, 1.f, 0.f, e_.get(), ld_e_, st.d.at((size_t)c.xw_lo * H), c.ND * H, dW + (size_t)c.xw_lo * H, c.NX * H});
    }
  }
  for (size_t ci = 0; ci < cells_.size(); ci++) {
    const CellStage &st = cells_[ci];
    const CellSpec &c = *st.spec;
    const int ldd = c.ND * H, lda = (int)c.asrc.size() * H;
    const int r0 = ci == 0 ? lp : 0;  // (the first cell's left operands are zero in the rows of leaves)
    struct Run {
      int asrc, dcol, param, ldb, width;
      long view, brow, col;
      long at() const { return view + brow * ldb + col; }
    };
    std::vector<Run> runs;  // terms whose operands, columns and gradient blocks are adjacent go as one product
    for (const CellProduct &p : c.products)
      for (const CellTerm &t : p.terms) {
        if (!runs.empty()) {
          Run &q = runs.back();
          if (q.asrc == t.asrc && q.param == p.B.param && q.view == p.B.offset && q.ldb == p.ldb && q.brow == t.brow &&
              q.col + q.width == p.col && q.dcol + q.width / H == p.dcol) {
            q.width += H;
            continue;
          }
        }
        runs.push_back({t.asrc, p.dcol, p.B.param, p.ldb, H, p.B.offset, t.brow, p.col});
      }
    for (const Run &q : runs) {
      float *C = param(c.params[q.param].name).g + q.at();
      if (N > r0) {
        add({1, 0, H, q.width, N - r0, 1.f, 0.f, st.asrc.at((size_t)r0 * lda + (size_t)q.asrc * H), lda,
             st.d.at((size_t)r0 * ldd + (size_t)q.dcol * H), ldd, C, q.ldb});
      } else {  // a batch of single vertices: nothing was multiplied
        for (int row = 0; row < H; row++) check(cavs_zero(C + (size_t)row * q.ldb, (size_t)q.width * 4, stream_));
      }
    }
  }
  // (overlapping but different blocks of one weight would need more than "the same first element")
  constexpr size_t kGroup = 8;  // products per cavs_sgemm_group launch
  bool embedded = false;
  for (size_t wv = 0; wv < waves.size(); wv++) {
    const std::vector<cavs_gemm_desc> &w = waves[wv];
    size_t at = 0;
    if (wv == 0 && c0.NX > 0 && L == 1 && !w.empty()) {  // d e is complete after this launch
      const size_t take = std::min(w.size(), kGroup);
      gemm_group_embedding_backward(std::vector<cavs_gemm_desc>(w.begin(), w.begin() + take), E_);
      at = take;
      embedded = true;
    }
    for (; at < w.size(); at += kGroup) gemm_group(std::vector<cavs_gemm_desc>(w.begin() + at, w.begin() + std::min(w.size(), at + kGroup)));
  }
  if (c0.NX > 0 && !embedded) embedding_backward_rows();
  for (size_t ci = 0; ci < cells_.size(); ci++) {
    const CellStage &st = cells_[ci];
    if (st.spec->biases.empty()) continue;
    colsum_fixed(st.colsum.get(), st.d.get(), N, st.spec->ND * H);
    ProfScope ps(this, K_OTHER);
    cell_launch((int)ci, CK_BIAS, (H + 255) / 256, 1, 1, 256, 0, 0, nullptr, d_dgo_);
  }
}

// EmbeddingLookup_grad as a launch of its own: rows of de_ added into the table's gradient.
void Engine::embedding_backward_rows() {
  Param &emb = param("Emb");
  const bool owned = emb.g == emb.own_g.get();
  if (emb_cleared_) {
    emb_cleared_ = false;
  } else if (owned && emb_sparse_valid_) {
    if (emb_dirty_n_ > 0) check(cavs_embed_zero_rows(emb.g, xs_prev_.get(), emb_dirty_n_, E_, stream_));
    c_launches_ += 1;
  } else {
    check(cavs_zero(emb.g, emb.n * 4, stream_));
    c_launches_ += 1;
  }
  check(cavs_embed_bwd(emb.g, xs_.get(), de_.get(), E_, N_, E_, stream_));
  c_launches_ += 1;
  xs_.swap(xs_prev_);
  emb_dirty_n_ = N_;
  emb_sparse_valid_ = owned;
}

// ------------------------------------------------------------------ loss head
void Engine::head_forward_backward(bool backward) {
  const int N = N_, H = cfg_.H, C = cfg_.C, B = sched_->B;
  if (head_chunked_) {
    head_in_chunks();
    return;
  }
  if (cfg_.loss == CAVS_LOSS_SOFTMAX) {
    // FullyConnected + SoftmaxEntropyLoss (cavs/backend/op_impl_fullyconnected_cublas.cc:71-79,
    // op_impl_softmax_entropy_logits_loss.cu:94-140) and their gradients (:150-163, :212-250)
    Param &Wfc = param("Wfc"), &bfc = param("bfc");
    const size_t head_bytes = cavs_fc_softmax_xent_workspace(N, H, C);
    if (head_bytes > 0) {  // few classes: the whole head and its gradients in one launch; the sum of
                           // its weight-gradient partials rides in the launch that opens backward
      if (head_parts_.capacity() * 4 < head_bytes) {
        check(cavs_stream_sync(stream_));  // the last step's jobs may still read the old buffer
        head_parts_.reserve(head_bytes / 4 + 1);
      }
      check(cavs_fc_softmax_xent(GO_.get(), Wfc.w, bfc.w, d_labels_, loss_.get(), logits_.get(), backward ? dGO_.get() : nullptr,
                                 nullptr, nullptr, head_parts_.get(), head_bytes, N, H, C, stream_));
      if (backward)
        pending_tasks_.push_back({CAVS_TASK_SUM_PARTS, 0.f, cavs_fc_softmax_xent_parts(N), (long long)C * H + C, (long long)C * H,
                                  head_parts_.get(), Wfc.g, bfc.g, nullptr});
      c_launches_ += 1;
      return;
    }
    // A wide head multiplies by a transposed copy of the weights, [H, C]: with C contiguous both
    // products that read them run a tenth faster (7331 x 10000 x 512: logits 760 -> 677 us, d GO
    // 782 -> 688), which pays for the copy (20 MB) several times over.
    // The update writes the copy along with the weights (update_jobs); it is made here only
    // when somebody else has written them since.
    const bool wide = wide_head();
    if (wide) ensure_wfct();
    {  // logits = GO * Wfc^T + bfc: the bias rides in the product's epilogue (row r adds D[r >> 30] = D[0])
      float *ws = workspace(cavs_sgemm_splitk_workspace(N, C, H));
      ProfScope ps(this, K_GEMM);
      if (wide)
        check(cavs_sgemm_addrows(0, 0, N, C, H, GO_.get(), H, WfcT_.get(), C, bfc.w, C, 30, logits_.get(), C, ws, ws_.capacity() * 4, stream_));
      else
        check(cavs_sgemm_addrows(0, 1, N, C, H, GO_.get(), H, Wfc.w, H, bfc.w, C, 30, logits_.get(), C, ws, ws_.capacity() * 4, stream_));
      c_gemm_flops_ += 2.0 * N * C * H;
      c_launches_ += 1;
    }
    check(cavs_softmax_xent(loss_.get(), backward ? dlogits_.get() : nullptr, logits_.get(), d_labels_, N, C, stream_));
    c_launches_ += 1;
    if (backward) {
      const cavs_gemm_desc dWd{1, 0, C, H, N, 1.f, 0.f, dlogits_.get(), C, GO_.get(), H, Wfc.g, H};
      const cavs_gemm_desc dGd = wide ? cavs_gemm_desc{0, 1, N, H, C, 1.f, 0.f, dlogits_.get(), C, WfcT_.get(), C, dGO_.get(), H}
                                      : cavs_gemm_desc{0, 0, N, H, C, 1.f, 0.f, dlogits_.get(), C, Wfc.w, H, dGO_.get(), H};
      // (not in a session that records graphs: on this runtime a capture on the session's stream comes
      // out invalidated once that stream has waited for an event of another stream)
      if (wide && !profile_ && !cfg_.graph_replay) {
        // Only d GraphOutput is on the way of the backward rounds.  The weight and bias gradients are
        // wanted at the update: they run on the side stream, under the rounds.
        aux_open();
        aux_workspace(cavs_sgemm_group_workspace(1, &dWd));
        // (forked behind the d GraphOutput product: side by side the two would only share the chip)
        gemm_group({dGd});
        check(cavs_event_record(aux_fork_ev_, stream_));
        check(cavs_stream_wait_event(aux_stream_, aux_fork_ev_));
        check(cavs_sgemm_group_beside(1, &dWd, ws_aux_.get(), ws_aux_.capacity() * 4, aux_stream_));
        c_gemm_flops_ += 2.0 * dWd.M * dWd.N * dWd.K;
        c_launches_ += 1;
        bias_gradient("bfc", dlogits_.get(), N, C, head_bias_parts_, aux_stream_);
        check(cavs_event_record(aux_join_ev_, aux_stream_));
        aux_pending_ = true;
      } else {
        // both read d logits and write different outputs: one launch when they are small
        gemm_group({dWd, dGd});
        bias_gradient("bfc", dlogits_.get(), N, C, head_bias_parts_);
      }
    }
    return;
  }
  float *tmp = logits_.get(), *colacc = loss_.get() + 1;
  if (cfg_.loss == CAVS_LOSS_ROOT_SQ) {
    // sum over roots of h^2; gradient 2h on root rows, zero elsewhere
    gather(tmp, H, GO_.get(), H, d_roots_, B, H);
    check(cavs_ew_unary(CAVS_EW_SQUARE, dlogits_.get(), tmp, (size_t)B * H, 0, stream_));
    colsum_fixed(colacc, dlogits_.get(), B, H);
    colsum_fixed(loss_.get(), colacc, H, 1);
    c_launches_ += 1;  // the squares
    if (backward) {
      check(cavs_zero(dGO_.get(), (size_t)N * H * 4, stream_));
      check(cavs_scale(dlogits_.get(), tmp, 2.f, (size_t)B * H, stream_));
      c_launches_ += 2;
      scatter(dGO_.get(), H, d_roots_, dlogits_.get(), H, B, H);
    }
  } else {
    // Reduce_sum is a sum of absolute values whose gradient op is a constant fill
    // (cavs/backend/op_impl_blas1_cublas.cc:62-77, cavs/backend/op_decl_reduction.cc:19-28)
    check(cavs_ew_unary(CAVS_EW_ABS, dlogits_.get(), GO_.get(), (size_t)N * H, 0, stream_));
    colsum_fixed(colacc, dlogits_.get(), N, H);
    colsum_fixed(loss_.get(), colacc, H, 1);
    c_launches_ += 1;
    if (backward) {
      check(cavs_fill(dGO_.get(), 1.f, (size_t)N * H, stream_));
      c_launches_ += 1;
    }
  }
}

void Engine::ensure_wfct() {
  if (wfct_valid_) return;
  Param &Wfc = param("Wfc");
  const size_t C = cfg_.C, H = cfg_.H;
  if (WfcT_.capacity() < C * H) {
    check(cavs_stream_sync(stream_));
    WfcT_.reserve(C * H);
  }
  check(cavs_transpose(WfcT_.get(), Wfc.w, cfg_.C, cfg_.H, stream_));
  c_launches_ += 1;
  wfct_valid_ = Wfc.w == Wfc.own_w.get();
}

void Engine::aux_open() {
  if (aux_stream_) return;
  check(cavs_stream_create(&aux_stream_));
  check(cavs_event_create(&aux_fork_ev_));
  check(cavs_event_create(&aux_join_ev_));
}

float *Engine::aux_workspace(size_t bytes) {
  if (ws_aux_.capacity() * 4 < bytes) {
    check(cavs_stream_sync(aux_stream_));
    ws_aux_.reserve(bytes / 4 + 1);
  }
  return ws_aux_.get();
}

// Which rounds go into which chunk of a wide head that runs beside the backward rounds: equal
// shares of the rows, cut at round boundaries.  Two chunks by default -- measured on the 10 000-class
// chain LSTM (7 000 rows, 99 rounds): 3.93 ms per step with two halves (3.99 / 4.03 with the cut at
// 35 or 65 / 20 or 80 % of the rows), 4.04 with three chunks, 4.19 with four or with the head in
// one piece between the passes: a chunk's products lose efficiency with their size, and the rounds
// that run beside a product take 12-20 us each instead of 7-10.
void Engine::plan_head_chunks(const int *orphans_host) {
  head_chunks_.clear();
  const Schedule &s = *sched_;
  const int R = (int)s.rounds.size(), N = s.N;
  if (cfg_.head_chunks < 0 || cfg_.model != CAVS_MODEL_LSTM || !wide_head() || !s.batching || !forest_ || cfg_.graph_replay || R < 8 ||
      N < 256)
    return;
  const int K = cfg_.head_chunks > 0 ? std::min(cfg_.head_chunks, (int)kHeadChunks) : 2;
  int k = 0;
  for (int c = 0; c < K; c++) {
    HeadChunk h;
    h.round0 = k;
    h.row0 = k < R ? s.rounds[k].offset : N;
    const double upto = (double)(c + 1) / K;
    while (k < R && (c == K - 1 || s.rounds[k].offset + s.rounds[k].n <= upto * N || k == h.round0)) k++;
    h.round1 = k;
    h.row1 = k < R ? s.rounds[k].offset : N;
    if (h.round1 > h.round0) head_chunks_.push_back(h);
  }
  if (head_chunks_.size() < 2) {
    head_chunks_.clear();
    return;
  }
  for (HeadChunk &h : head_chunks_) {  // (the list is in ascending order of slab rows)
    h.orph0 = (int)(std::lower_bound(orphans_host, orphans_host + n_orphans_, h.row0) - orphans_host);
    h.orph1 = (int)(std::lower_bound(orphans_host, orphans_host + n_orphans_, h.row1) - orphans_host);
  }
}

// Chunk k on the side stream: logits of its rows (h straight out of the message rows), loss and
// d logits, d h.
void Engine::head_chunk(int k) {
  const HeadChunk &h = head_chunks_[k];
  const int n = h.row1 - h.row0, H = cfg_.H, C = cfg_.C;
  if (n > 0) {
    const size_t r0 = h.row0;
    float *ws = aux_workspace(cavs_sgemm_splitk_workspace(n, C, H));
    check(cavs_sgemm_addrows(0, 0, n, C, H, msg_.at(r0 * mw_), (int)mw_, WfcT_.get(), C, param("bfc").w, C, 30, logits_.at(r0 * C), C, ws,
                             ws_aux_.capacity() * 4, aux_stream_));
    check(cavs_softmax_xent_part(loss_slab_.at(r0), dlogits_.at(r0 * C), logits_.at(r0 * C), labels_slab_.at(r0), n, C, N_, aux_stream_));
    const cavs_gemm_desc dh{0, 1, n, H, C, 1.f, 0.f, dlogits_.at(r0 * C), C, WfcT_.get(), C, dret_.at(r0 * H), H};
    ws = aux_workspace(cavs_sgemm_group_workspace(1, &dh));
    check(cavs_sgemm_group_beside(1, &dh, ws, ws_aux_.capacity() * 4, aux_stream_));
    c_gemm_flops_ += 4.0 * n * C * H;
    c_launches_ += 3;
  }
  if (!chunk_done_ev_[k]) check(cavs_event_create(&chunk_done_ev_[k]));
  check(cavs_event_record(chunk_done_ev_[k], aux_stream_));
}

// The whole head on the side stream, behind the forward rounds: the chunks last first (the backward
// rounds start at the end), then what only the update and the caller wait for -- loss and d h by
// vertex id, the head's weight and bias gradients.
void Engine::head_in_chunks() {
  const int N = N_, H = cfg_.H, C = cfg_.C;
  ensure_wfct();
  aux_open();
  ensure_iota(cap_);
  ensure(labels_slab_, grow((size_t)N, labels_slab_.capacity()));
  ensure(loss_slab_, grow((size_t)N, loss_slab_.capacity()));
  check(cavs_event_record(aux_fork_ev_, stream_));
  check(cavs_stream_wait_event(aux_stream_, aux_fork_ev_));
  check(cavs_gather_rows(labels_slab_.get(), 1, d_labels_, 1, d_t2j_, N, 1, aux_stream_));
  for (int k = (int)head_chunks_.size() - 1; k >= 0; k--) head_chunk(k);
  check(cavs_scatter_rows(loss_.get(), 1, d_t2j_, loss_slab_.get(), 1, N, 1, aux_stream_));
  check(cavs_scatter_rows(dGO_.get(), H, d_t2j_, dret_.get(), H, N, H, aux_stream_));
  Param &Wfc = param("Wfc");
  const cavs_gemm_desc dWd{1, 0, C, H, N, 1.f, 0.f, dlogits_.get(), C, msg_.get(), (int)mw_, Wfc.g, H};
  float *ws = aux_workspace(cavs_sgemm_group_workspace(1, &dWd));
  check(cavs_sgemm_group_beside(1, &dWd, ws, ws_aux_.capacity() * 4, aux_stream_));
  c_gemm_flops_ += 2.0 * dWd.M * dWd.N * dWd.K;
  c_launches_ += 4;
  bias_gradient("bfc", dlogits_.get(), N, C, head_bias_parts_, aux_stream_);
  check(cavs_event_record(aux_join_ev_, aux_stream_));
  aux_pending_ = true;
}

// The session's stream takes up what the side stream has been doing.
void Engine::aux_join() {
  if (!aux_pending_) return;
  check(cavs_stream_wait_event(stream_, aux_join_ev_));
  aux_pending_ = false;
}

void Engine::sync() {
  aux_join();
  check(cavs_stream_sync(stream_));
  tail_check();
}

void Engine::fetch(const std::string &what, float *host, size_t n) {
  const size_t N = N_, H = cfg_.H;
  const float *src = nullptr;
  size_t want = 0;
  if (what == "loss") {
    src = loss_.get();
    want = cfg_.loss == CAVS_LOSS_SOFTMAX ? N : 1;
  } else if (what == "graph_out") {
    src = GO_.get();
    want = N * H;
  } else if (what == "dgraph_out") {
    src = dGO_.get();
    want = N * H;
  } else if (what == "msg_pool") {
    src = pool_.get();
    want = N * mw_;
  } else {
    fail(CAVS_EINVAL, "unknown result '" + what + "'");
  }
  if (N == 0) fail(CAVS_EINVAL, "no step has run yet");
  if (n != want || !host) fail(CAVS_EINVAL, "'" + what + "' holds " + std::to_string(want) + " floats, got " + std::to_string(n));
  check(cavs_memcpy_d2h(host, src, want * 4, stream_));
  check(cavs_stream_sync(stream_));
  tail_check();
}

float Engine::timing(const std::string &name) {
  float ms = 0.f;
  if (name == "GraphParsing") return parse_ms_;
  // host-side split of a step: building the schedule, waiting for the index staging buffer
  // of two steps ago (i.e. for the device), and the whole enqueueing call
  if (name == "HostSchedule") return sched_ms_;
  if (name == "HostWait") return wait_ms_;
  if (name == "HostStep") return host_step_ms_;
  if (name == "RNNForward" && ev_valid_) {
    check(cavs_event_elapsed_ms(&ms, ev_[0], ev_[1]));
    return ms;
  }
  if (name == "RNNBackward" && ev_bwd_valid_) {
    check(cavs_event_elapsed_ms(&ms, ev_[2], ev_[3]));
    return ms;
  }
  fail(CAVS_EINVAL, "no timing named '" + name + "' for the last step");
}

double Engine::counter(const std::string &key) const {
  if (key == "gather_rows") return c_gather_rows_;
  if (key == "scatter_rows") return c_scatter_rows_;
  if (key == "gather_bytes") return c_gather_bytes_;
  if (key == "scatter_bytes") return c_scatter_bytes_;
  if (key == "gemm_flops") return c_gemm_flops_;
  if (key == "gemm_flops_hinted") return c_gemm_flops_hinted_;
  if (key == "round_flops") return c_round_flops_;
  if (key == "launches") return c_launches_;
  if (key == "rounds") return (double)sched_->rounds.size();
  if (key == "tail_rounds") return c_tail_rounds_;
  if (key == "tail_launches") return c_tail_launches_;
  if (key == "scheduler") return (double)scheduler_used_;
  if (key == "tail_ready") return tail_ready_ ? 1.0 : 0.0;
  if (key == "tail_first_round") return (double)tail_.first;
  if (key == "tail_lists_max") return (double)tail_.lists_max;
  if (key == "tail_tiles_max") return (double)tail_.tiles_max;
  if (key == "tail_vertices") return tail_.vertices;
  if (key == "head_chunks") return head_chunked_ ? (double)head_chunks_.size() : 0.0;  // of the last step
  if (key == "graph_replays") return c_graph_replays_;
  if (key == "plan_hits") return c_plan_hits_;
  if (key == "plan_misses") return c_plan_misses_;
  fail(CAVS_EINVAL, "unknown counter '" + key + "'");
}

}  // namespace cavs
