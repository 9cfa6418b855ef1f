// The forward / backward round loops over a batch of instance graphs for the three
// vertex functions, on top of the C ABI of the HIP backend.  Restates, for these F,
// what the reference spreads over GraphStatement::Run / GraphGradStatement::Run
// (cavs/midend/statement.cc:43-123), GraphSession's memory layout
// (cavs/midend/graph_session.cc:45-206) and BatchingWeightUpdater
// (cavs/midend/batch_weight_updater.h:12-84).
#ifndef CAVS_HOST_ENGINE_H_
#define CAVS_HOST_ENGINE_H_

#include <cstdint>
#include <map>
#include <memory>
#include <string>
#include <deque>
#include <vector>

#include "cavs_session.h"
#include "cell.h"
#include "device.h"
#include "scheduler.h"

namespace cavs {

struct Param {
  float *w = nullptr, *g = nullptr;  // owned storage below, or bound to a caller's tensors
  DeviceArray<float> own_w, own_g;
  size_t n = 0;
};

class Engine {
 public:
  // external_stream: enqueue on the caller's stream instead of creating one
  // cell: the generated kernels of cfg.model == CAVS_MODEL_CELL
  explicit Engine(const cavs_session_config &cfg, void *external_stream = nullptr, std::shared_ptr<const CellSpec> cell = nullptr);
  ~Engine();

  // Points a parameter and its gradient at device memory owned by the caller (the front
  // end's Variable tensors) instead of the engine's own copies.  g may be null: then the
  // engine keeps the gradient in its own buffer (read it with grad_ptr()).
  void bind_param(const std::string &name, float *w, float *g);
  // where the next backward pass leaves the gradient of `name` (null: the engine's own buffer)
  void bind_param_grad(const std::string &name, float *g) {
    state_epoch_++;
    Param &p = param(name);
    p.g = g ? g : p.own_g.get();
  }
  const float *grad_ptr(const std::string &name) { return param(name).g; }
  // For a caller that applies w -= lr * g to bound parameters itself (the front end's optimizer):
  // when w is the recurrent weights whose tile-major copy the forward rounds read, appends the
  // jobs of a cavs_run_tasks launch that update them and the copy together and returns true --
  // the copy then counts as current until the parameter is bound elsewhere; otherwise false, and
  // the caller's plain update will do.  Such a caller must route every write of w through here.
  bool update_jobs(float *w, float *g, float lr, std::vector<cavs_task> *out);
  float *graph_out_ptr() const { return GO_.get(); }
  // The two halves of step() for a caller that runs the loss head itself: forward F into
  // graph_out [N,H] (vertex order), then backward F from d graph_out.
  void forward_only(const int *graph, int B, int maxlen, const float *x_dev, float *graph_out);
  // settle_biases = false leaves the bias gradients that exist as rows still to be added up
  // (row E of dW, chunk sums) pending: the caller then takes them with update_bias_jobs() into the
  // launch that applies its parameter updates, instead of a launch of their own here.
  void backward_only(const float *dgraph_out, bool settle_biases = true);
  // The pending bias jobs as jobs of the caller's update launch: each delivers the gradient and
  // applies w -= lr * g to the bias parameter.  `updated` receives the weight pointers they cover.
  void update_bias_jobs(float lr, std::vector<cavs_task> *out, std::vector<const float *> *updated);
  // A job for the launch that opens the next backward pass (it runs before anything of that pass).
  void queue_prologue_task(const cavs_task &t) { pending_tasks_.push_back(t); }
  void set_pairing(int pairing) {
    if (pairing != cfg_.pairing) state_epoch_++;
    cfg_.pairing = pairing;
  }
  void set_param(const std::string &name, const float *host, size_t n);
  void get_param(const std::string &name, float *host, size_t n, bool grad);
  void step(const int *graph, int B, int maxlen, const void *x, const void *labels,
            bool on_device, bool backward, float lr);
  void sync();
  void fetch(const std::string &what, float *host, size_t n);
  float timing(const std::string &name);
  double counter(const std::string &key) const;
  // Per-kernel-class device time: when enabled every launch is bracketed by a pair of
  // events on the session's stream; read() waits for the stream and sums them.
  enum KernelClass { K_GEMM = 0, K_GATHER, K_SCATTER, K_GATES, K_OTHER, K_ROUND, K_CLASSES };
  void profile_enable(bool on);
  void profile_read(int cls, double *total_ms, double *launches);
  // The last step's schedule with all its lists.  When the device scheduler built it, the host
  // holds the rounds only; the lists are then read back and the schedule completed (synchronises).
  const Schedule &schedule();
  void *stream() const { return stream_; }
  int total_length() const { return sched_->N; }

 private:
  Param &param(const std::string &name);
  void add_param(const std::string &name, size_t n, size_t extra_grad = 0);
  void reserve_edges();
  void ensure(DeviceArray<float> &a, size_t n);  // grow after draining the stream
  void upload_index_arena();
  // one model each: forward rounds, backward rounds + deferred weight gradients
  void treelstm_forward();
  void treelstm_backward();
  void lstm_forward();
  void lstm_backward();
  void treefc_forward();
  void treefc_backward();
  void cell_forward();
  void cell_backward();
  void model_forward();
  void model_backward();
  void pop_ret(float *graph_out);
  void begin_step(const int *graph, int B, int maxlen);
  void head_forward_backward(bool backward);
  // counted wrappers
  float *workspace(size_t bytes);
  void gemm(int tA, int tB, int M, int N, int K, const float *A, int lda, const float *B, int ldb,
            float beta, float *C, int ldc);
  // independent products in one launch (cavs_sgemm_group)
  void gemm_group(const std::vector<cavs_gemm_desc> &products);
  void backward_prologue(std::vector<cavs_task> tasks, bool with_embedding);
  void gemm_splitk(int tA, int tB, int M, int N, int K, const float *A, int lda, const float *B,
                   int ldb, float *C, int ldc);
  void gather(float *out, int ld_out, const float *src, int ld_src, const int *ids, int n, int w);
  void scatter(float *dst, int ld_dst, const int *ids, const float *inp, int ld_inp, int n, int w);
  bool leaf_round(const Round &r) const {
    return r.gather_begin[0] == r.gather_end[0] && r.gather_begin[1] == r.gather_end[1];
  }

  struct Span {
    int cls;
    void *a, *b;
  };
  struct ProfScope {  // times the kernels launched during its lifetime (cavs_profile_arm)
    Engine *e;
    Span s;
    bool on;
    ProfScope(Engine *eng, int cls);
    ~ProfScope();
  };
  void *prof_event();
  bool profile_ = false;
  std::vector<Span> spans_;
  std::vector<void *> prof_events_;
  size_t prof_used_ = 0;

  cavs_session_config cfg_;
  void *stream_ = nullptr;
  bool own_stream_ = true;
  void *ev_[4] = {nullptr, nullptr, nullptr, nullptr};  // fwd begin/end, bwd begin/end
  bool ev_valid_ = false, ev_bwd_valid_ = false;
  float parse_ms_ = 0.f, sched_ms_ = 0.f, wait_ms_ = 0.f, host_step_ms_ = 0.f;
  std::map<std::string, std::unique_ptr<Param>> params_;

  std::shared_ptr<Schedule> sched_ = std::make_shared<Schedule>();
  bool sched_lists_on_host_ = true;  // false: the device scheduler built the lists, sched_ holds the rounds only
  bool did_backward_ = false;
  float *fwd_out_ = nullptr;   // where the forward pass returns h by vertex id
  bool out_folded_ = false;    // the rounds wrote it themselves
  int N_ = 0, cap_ = 0, rcap_ = 0, E_ = 0, mw_ = 0, nch_ = 1;

  // per-step device index arena: [t2j | pair | child | roots | kid_rows | orphans]
  struct HostLists {  // host-built lists: pinned staging, their device copy, and who still reads it
    PinnedArray<int> host;
    DeviceArray<int> dev;
    void *free_ev = nullptr, *up_ev = nullptr;
    bool busy = false;
  } hlists_[2];
  int hlists_slot_ = 0;
  // the event to record, and the flag to raise, once the current step's kernels are all enqueued
  void *last_free_ev_ = nullptr;
  bool *last_busy_ = nullptr;
  const int *d_t2j_ = nullptr, *d_pair_ = nullptr, *d_child_ = nullptr, *d_roots_ = nullptr;
  // Tree-LSTM, message flow of the batch is a forest: children by slab row, and the slab rows
  // nobody sends a message to
  const int *d_kid_rows_ = nullptr, *d_orphans_ = nullptr;
  int n_orphans_ = 0;
  bool forest_ = false;

  // ---- schedule on the device (cfg.schedule_mode 1): the graph feed goes up, cavs_schedule_arena
  // builds every list there, and only the round offsets come back.  Two sets of buffers alternate,
  // so that the lists of step k + 1 are built while the kernels of step k still read theirs.
  struct DeviceSched {
    PinnedArray<int> graph_host, meta_host, kid_host, tail_host;
    DeviceArray<int> graph_dev, lists, meta_dev, tail_dev;
    long cap = 0;          // rows per list
    void *free_ev = nullptr;  // recorded once everything that read `lists` has been enqueued
    bool busy = false;
  } dsched_[2];
  DeviceArray<int> dsched_scratch_;
  void *sched_stream_ = nullptr;
  int dsched_slot_ = 0;
  void schedule_on_device(const int *graph, int B, int maxlen);
  void schedule_on_host(const int *graph, int B, int maxlen);
  void point_lists(const int *base, long cap);

  // ---- the rounds near the roots as one launch per direction (cavs_treelstm_tail_fwd / _bwd)
  // What those launches run, for one batch structure: the rounds from `first` on, their rows dealt
  // to the groups by whole trees of the message flow (no message crosses groups).
  struct TailPlan : TailLists {
    double flops = 0, vertices = 0;
  };

  // ---- plan cache (cfg.plan_cache entries): the schedule and the device lists of a graph feed,
  // keyed by the feed's bytes, so that a batch structure seen before costs neither the scheduler
  // nor an upload
  // ---- replay of a cached plan's launches (cfg.graph_replay): the forward pass, the loss head and
  // the backward pass of a step as one recorded graph.  What such a graph does depends on more than
  // the batch structure: on the feed buffers and on the state the session was in when the step began
  // (which rows of the embedding gradient are dirty, whether the repacked weights are current, which
  // of the two id buffers is this step's ...).  StepSig is all of that, StepState is what the
  // recorded step left behind on the host; a graph is replayed only under an equal signature and the
  // state it left is then put in place as if the launches had been issued one by one.
  struct StepSig {
    const void *x = nullptr, *labels = nullptr, *xs = nullptr, *xs_prev = nullptr;
    bool backward = false, emb_sparse_valid = false, emb_cleared = false, upk_valid = false, wfct_valid = false;
    int emb_dirty_n = 0, pairing = 0;
    size_t e_ones_rows = 0;
    uint64_t alloc_epoch = 0, state_epoch = 0;
    bool operator==(const StepSig &o) const {
      return x == o.x && labels == o.labels && xs == o.xs && xs_prev == o.xs_prev && backward == o.backward &&
             emb_sparse_valid == o.emb_sparse_valid && emb_cleared == o.emb_cleared && upk_valid == o.upk_valid &&
             wfct_valid == o.wfct_valid && emb_dirty_n == o.emb_dirty_n && pairing == o.pairing && e_ones_rows == o.e_ones_rows &&
             alloc_epoch == o.alloc_epoch && state_epoch == o.state_epoch;
    }
  };
  struct BiasJob {
    std::string param;
    const float *src;
    int parts;
    long long bw, nb, map;
  };
  struct StepState {
    bool did_backward = false, out_folded = false, emb_sparse_valid = false, emb_cleared = false, upk_valid = false,
         wfct_valid = false, tail_pending = false;
    float *fwd_out = nullptr;
    const float *d_dgo = nullptr;
    const void *xs = nullptr;
    int emb_dirty_n = 0;
    std::vector<BiasJob> bias_jobs;
    std::vector<cavs_task> pending_tasks;
    double counters[10] = {0};
  };
  struct StepGraph {
    void *exec = nullptr;
    StepSig sig;
    StepState after;
  };
  StepSig step_signature(const void *x, const void *labels, bool backward) const;
  StepState step_state() const;
  void restore_step_state(const StepState &st);
  void run_passes(bool backward);  // forward rounds, loss head, backward rounds of a step
  bool capturing_ = false;
  uint64_t state_epoch_ = 0;  // bumped by every call other than step() that changes what a step enqueues
  double c_graph_replays_ = 0;

  // a chunk of the loss head of a wide classifier that runs beside the backward rounds (below)
  struct HeadChunk {
    int row0 = 0, row1 = 0;      // slab rows
    int round0 = 0, round1 = 0;  // rounds [round0, round1)
    int orph0 = 0, orph1 = 0;    // positions in the list of vertices nobody sends a gradient to
  };
  struct Plan {
    ~Plan() { drop_graphs(); }
    void drop_graphs() {
      for (StepGraph &g : graphs) cavs_graph_destroy(g.exec);
      graphs.clear();
      graph_off = false;
      recordings = 0;
    }
    std::vector<StepGraph> graphs;
    bool graph_off = false;  // recording failed once: ordinary steps from then on
    int recordings = 0;
    uint64_t hash = 0;
    int B = 0, maxlen = 0, pairing = 0;
    std::vector<int32_t> graph;
    std::shared_ptr<Schedule> sched;
    bool lists_on_host = true;
    DeviceArray<int> lists;  // [t2j | pair | child | roots | kid_rows | orphans], N rows each
    int n_orphans = 0;
    bool forest = false;
    TailPlan tail;
    std::vector<HeadChunk> head_chunks;
    uint64_t last_used = 0;
  };
  std::vector<std::unique_ptr<Plan>> plans_;
  uint64_t plan_clock_ = 0;
  double c_plan_hits_ = 0, c_plan_misses_ = 0;
  int scheduler_used_ = 0;  // who produced the last step's lists: 0 host scheduler, 1 device scheduler, 2 plan cache
  Plan *hit_plan_ = nullptr;  // the cached plan this step runs on (null: it was scheduled afresh)
  Plan *find_plan(const int *graph, int B, int maxlen, uint64_t hash);
  void remember_plan(const int *graph, int B, int maxlen, uint64_t hash);

  // feeds
  DeviceArray<float> x_in_, labels_in_;
  const float *d_x_ = nullptr, *d_labels_ = nullptr, *d_dgo_ = nullptr;

  // edges (rows = tensor ids unless marked round-local)
  DeviceArray<float> xs_, e_, xW_, G_, hlr_, gates_, msg_, pool_, GO_, dGO_, dret_, dpool_, dxW_,
      dF_, de_, logits_, dlogits_, loss_, ws_;
  DeviceArray<float> r_hU_, r_hUf_, r_dmsg_, r_dG_, r_dhlr_, r_z_;  // round-local
  DeviceArray<float> dc_;  // [N, H] d c of every vertex (folded backward rounds)
  // Embedding gradient: only the rows looked up in a step are non-zero, so the table is
  // cleared and updated by those rows.  xs_prev_ lists the rows the last backward pass wrote.
  DeviceArray<float> xs_prev_;
  DeviceArray<int> emb_stamp_;
  int emb_dirty_n_ = 0, emb_epoch_ = 0;
  bool emb_sparse_valid_ = true;  // the table is zero outside xs_prev_[0, emb_dirty_n_)
  bool emb_cleared_ = false;      // the backward prologue of this step already cleared those rows
  std::vector<cavs_task> pending_tasks_;  // jobs queued for the launch that opens backward
  // Tree-LSTM: e_ carries a column of ones after its E columns, so that the deferred product
  // e^T * dxW yields the bias gradient (column sums of dxW) as row E of dW for free
  int ld_e_ = 0;
  size_t e_ones_rows_ = 0;       // rows of e_ whose ones column is initialised
  DeviceArray<float> ones_col_;  // [ld_e_]: 1 at column E
  bool bias_row_ok() const;
  // Bias gradients that exist as rows still to be added up and / or permuted (row E of dW; the
  // chunk sums of a column sum): delivered, and the parameter updated, by one job each of the
  // launch that ends the step.
  std::vector<BiasJob> bias_jobs_;
  DeviceArray<float> bias_parts_, head_bias_parts_;
  // column sums of inp [n, w] as the gradient of `name`, in a fixed order
  void bias_gradient(const std::string &name, const float *inp, int n, int w, DeviceArray<float> &parts, void *stream = nullptr);
  void colsum_fixed(float *out, const float *inp, int n, int w);
  bool has_bias_job(const std::string &name) const;
  void settle_bias_jobs(float lr, std::vector<cavs_task> *tasks);
  DeviceArray<float> head_parts_;         // weight-gradient partials of the classifier head
  void gemm_group_embedding_backward(const std::vector<cavs_gemm_desc> &products, int E);
  DeviceArray<float> UT_;  // transposed recurrent weights for the fused backward rounds
  // The recurrent weights (Tree-LSTM: U; chain LSTM: W') tile-major for the packed forward rounds.
  // Written by the job that applies their SGD update; current while nobody else has written them
  // since (set_param, a caller's own tensor).
  DeviceArray<float> Upk_;
  bool upk_valid_ = false;
  DeviceArray<float> WfcT_;  // [H, C] copy of a wide head's weights (head_forward_backward)
  bool wfct_valid_ = false;
  bool wide_head() const;
  // rounds of at most this many rows run as fused launches (0: none)
  int fused_rows() const;

  // (the tail launches, continued)
  TailPlan tail_;
  const int *d_tail_rows_ = nullptr;
  DeviceArray<int> tail_sync_;  // the launches' sync block
  bool tail_ready_ = false;     // the device ran the probe's workgroups all at once, each group on one XCD
  bool tail_pending_ = false;   // a tail launch was enqueued since the status word was last read
  double c_tail_rounds_ = 0, c_tail_launches_ = 0;
  int tail_limit() const;       // rows per group and round a tail launch may take (0: no tail launches)
  void tail_setup();
  // fills tail_ and writes the groups' row lists to `rows_out` (room for N ints) from the host copy of
  // the children-by-slab-row lists of a batch whose message flow is a forest
  void build_tail_plan(const int *kid_rows, int *rows_out);
 public:
  // After the stream has drained: reads the status word of the tail launches.  A launch that gave
  // up leaves the results of the steps since undefined (their parameter updates were skipped: they
  // watch the word); the session goes on with one launch per round and this call fails.
  void tail_check();
  // the word a parameter-update launch must watch (CAVS_TASK_GUARD), or null
  const int *update_guard() const { return tail_ready_ ? tail_sync_.get() + 1 : nullptr; }
 private:

  // ---- a side stream for work of the backward pass that nothing waits for before the update: the
  // weight gradient of a wide classifier head (0.6 ms at 7331 x 10000 x 512) runs there while the
  // backward rounds -- a chain of short dependent launches that leaves most of the chip idle -- run
  // on the session's stream.  Forked from an event behind the head's loss kernel, joined by an event
  // the update launch (or whoever reads the gradients first) waits for.
  void *aux_stream_ = nullptr, *aux_fork_ev_ = nullptr, *aux_join_ev_ = nullptr;
  bool aux_pending_ = false;   // work on the side stream that the session's stream has not waited for yet
  DeviceArray<float> ws_aux_;  // its products' split-K workspace
  void aux_join();
  void aux_open();  // creates the side stream and its events
  void ensure_wfct();  // the transposed copy of a wide head's weights, if somebody else wrote them since

  // ---- a wide loss head in chunks (chain LSTM), beside the rounds
  // The head of a wide classifier is three large products per vertex row, the rounds of a chain LSTM
  // two hundred short dependent launches that leave most of the chip idle.  The head reads a vertex's
  // h and hands back d h: nothing in it couples rows, so it runs on the side stream over chunks of
  // slab rows (= ranges of rounds), last chunk first, so that the backward rounds, which start at
  // the last round, can begin when the last chunk's d h is there and go on while the earlier chunks'
  // is computed.  (Not under the forward rounds: their 512-thread workgroups find no room beside a
  // large product's and a round then takes as long as the product.)  Rows are taken in slab order
  // (h straight out of the message rows, labels gathered once, d h where the backward launches
  // read it with the identity list).
  static constexpr int kHeadChunks = 4;
  std::vector<HeadChunk> head_chunks_;  // of this step's schedule; empty: the head runs in one piece
  bool head_chunked_ = false;           // this pass runs it in chunks
  void *chunk_done_ev_[kHeadChunks] = {};
  DeviceArray<float> labels_slab_, loss_slab_;
  void plan_head_chunks(const int *orphans_host);
  void head_chunk(int k);   // enqueues chunk k's logits, loss and d h on the side stream
  void head_in_chunks();    // after the forward rounds: all chunks, then what only the update waits for
  float *aux_workspace(size_t bytes);

  // ---- a vertex function on generated kernels (CAVS_MODEL_CELL)
  // A function of several stages is a chain of cells (CellSpec::next); every cell has its module
  // and its per-vertex rows.  A cell before the last writes `rows` by slab row, which the next one
  // gathers through the identity list; `drows` is the gradient of those rows.
  struct CellStage {
    std::shared_ptr<const CellSpec> spec;
    void *module = nullptr;
    DeviceArray<float> sv, asrc, d, ds, bt, colsum, rows, drows;
  };
  std::shared_ptr<const CellSpec> cell_;  // the head of the chain
  std::deque<CellStage> cells_;  // (the arrays do not move)
  DeviceArray<int> cell_iota_;  // 0, 1, 2, ...: "the child of slab row v is slab row v" (also: "d h of slab row v is row v")
  size_t cell_iota_n_ = 0;
  void ensure_iota(size_t n);
  // one launch of kernel `k` of cell `ci`'s module
  void cell_launch(int ci, int k, unsigned gx, unsigned gy, unsigned gz, unsigned block, long off, long n, const int *rows, const float *go);
  void embedding_backward_rows();

  // counters of the last step
  double c_round_flops_ = 0;
  double c_gather_rows_ = 0, c_scatter_rows_ = 0, c_gemm_flops_ = 0, c_gemm_flops_hinted_ = 0, c_launches_ = 0,
         c_gather_bytes_ = 0, c_scatter_bytes_ = 0;
};

}  // namespace cavs
#endif
