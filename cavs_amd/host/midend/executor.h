// Session of the front end: owns the device tensors of a program, interprets the
// main-scope operators, and runs the vertex function over the rounds of a batch
// (cavs/midend/session_simple.cc:56-108, statement.cc:8-123, graph_session.cc:45-206).
// Two ways to run F: op by op through the backend's C ABI (the reference's execution
// model), or -- when F is recognised as one of the vertex functions the fused round
// kernels implement -- lowered onto cavs::Engine.
#ifndef CAVS_HOST_MIDEND_EXECUTOR_H_
#define CAVS_HOST_MIDEND_EXECUTOR_H_

#include <map>
#include <memory>
#include <string>
#include <vector>

#include "../device.h"
#include "../engine.h"
#include "../scheduler.h"
#include "graph.h"

namespace cavs {
namespace mid {

struct Tensor {
  DeviceArray<float> own;
  float *base = nullptr;   // own.get() or a view into another tensor
  long width = 1;          // elements per row (per-vertex tensors) or total (static)
  bool per_vertex = false; // rows follow the batch: [rows, width]
  long rows = 1;           // current row count of a per-vertex tensor
  size_t count() const { return (size_t)(per_vertex ? rows * width : width); }
};

// A device-resident feed goes through two sets of buffers (pinned staging + device copy) that
// alternate from Run to Run; the copies run on a stream of their own, so that the feeds of Run
// k + 1 go up while the kernels of Run k are still running, instead of sitting in the compute
// stream between two steps.  A set is rewritten only after the Run that read it has finished.
struct FeedStage {
  PinnedArray<char> slot[2];
  DeviceArray<float> dev[2];
};

struct HostTensor {  // C_Tensor of the C API
  std::string name;
  std::vector<int> shape;
  std::vector<char> data;
};

struct Lowering;  // recognised vertex function bound to Engine parameters

class Executor {
 public:
  Executor(int opt, const std::string &name);
  ~Executor();
  void run(const std::vector<std::string> &outputs, std::vector<HostTensor *> *results,
           const std::vector<std::pair<std::string, const HostTensor *>> &feeds);
  void set_variable(const std::string &name, const float *data, size_t n);
  long read_tensor(const std::string &name, float *out, size_t cap);
  bool uses_fused_path() const { return lowered_; }
  int fused_kernel_count() const { return fused_groups_; }
  int fused_path_kind() const;  // 0: F runs op by op; 1: hand-written round kernels; 2: generated ones
  void set_lowering_mode(int m) { lowering_mode_ = m; compiled_version_ = -1; }
  void set_pairing(int p) { pairing_ = p; compiled_version_ = -1; }

 private:
  struct RoundCtx {
    long off = 0, n = 0;
    bool in_function = false;
    bool in_round_loop = false;  // one of the backward rounds: reduced outputs were zeroed before the loop
  };
  void compile();
  void init_variables();
  Tensor &tensor(const std::string &name);
  Tensor *find_tensor(const std::string &name);
  float *view(const std::string &name, const RoundCtx &c, long *count, long *width);
  void exec(const OpDef &d, const RoundCtx &c);
  void run_graph_output(const OpDef &d);
  void exec_fused(const OpDef &d, const RoundCtx &c);
  std::vector<OpDef> fused(const std::vector<OpDef> &prog, const std::vector<const std::vector<OpDef> *> &others,
                           const std::vector<std::string> &extra_live);
  void run_graph_output_grad(const OpDef &d);
  void upload_lists();
  void lowered_forward(const int32_t *graph, int B, int maxlen, float *graph_out);
  void lowered_backward(const OpDef &d);
  void forward_needed(const std::vector<std::string> &targets, std::vector<const Node *> *order);
  const Edge *edge(const std::string &name) const;
  float *workspace(size_t bytes);

  int opt_;
  std::string name_;
  void *stream_ = nullptr;
  int compiled_version_ = -1;
  // 0: never lower F; 1: hand-written kernels, else generated ones; 2: generated ones only; 3: the same,
  // with the backward rounds split as for a batch whose message flow is no forest
  int lowering_mode_ = 1;
  bool lowered_ = false;
  int pairing_ = 0;
  std::map<std::string, std::unique_ptr<Tensor>> tensors_;
  std::map<std::string, FeedStage> feed_stages_;
  // this Run: the head's gradient partials are summed by the engine's backward prologue; the
  // engine's pending bias gradients are settled by the launch that applies the updates
  bool head_defer_ = false, defer_bias_ = false;
  DeviceArray<float> head_parts_;
  void *copy_stream_ = nullptr;
  void *feeds_up_ev_ = nullptr;                 // the current Run's feeds have arrived
  void *run_done_ev_[2] = {nullptr, nullptr};   // everything a Run enqueued has finished, by Run parity
  bool run_busy_[2] = {false, false};
  int run_parity_ = 0;
  bool dirty_ = false;  // device work queued by a Run that returned without waiting for it
  std::map<std::string, std::vector<float>> pending_vars_;  // SetVariable before compile
  bool vars_initialised_ = false;

  // per-step state of the vertex function
  Schedule sched_;
  long N_ = 0;
  int nch_ = 0;          // Gather children used by F
  long pool_w_ = 0, ret_w_ = 0, arg_w_ = 0;
  DeviceArray<float> pool_, dpool_, ret_, ws_;
  PinnedArray<int> idx_host_;
  DeviceArray<int> idx_dev_;
  const int *d_t2j_ = nullptr, *d_pair_ = nullptr, *d_child_[2] = {nullptr, nullptr};
  const float *func_arg_ = nullptr;   // vertex placeholder on the device
  const float *dgo_ = nullptr;        // d GraphOutput during the backward function
  // programs of the vertex function as executed (after the fusion pass when OPT_FUSION is set)
  std::vector<OpDef> func_fwd_, func_bwd_, func_def_;
  std::vector<std::string> round_zero_;  // reduced outputs of the per-round generated kernels: zeroed before the backward loop
  std::vector<OpDef> main_all_;
  // The lowered F writes a parameter's gradient where the main scope wants it: when the gradients
  // of all the slices of a Variable come out of the lowered F and only get added into the
  // Variable's zero-filled gradient, the engine's gradient array is bound to that place and the
  // Fill and PartialAccumulate operators are skipped.
  struct GradBind {
    std::string param, dst;  // engine parameter; main-scope gradient tensor
    long offset;             // the parameter's gradient starts at tensor(dst).base + offset
  };
  // A classifier head FullyConnected -> SoftmaxEntropyLoss whose gradients the program also
  // wants runs as one call (cavs_fc_softmax_xent) at the FullyConnected operator, on the lowered
  // path, whenever the batch's shape fits that entry point; the three other operators are skipped.
  struct HeadFuse {
    int fc = -1, loss = -1;           // indices into fwd
    int loss_grad = -1, fc_grad = -1; // indices into bwd
    int seed = -1;                    // the ConstOp that seeds d loss, if nobody else reads it
  };
  struct MainProgram {
    std::vector<OpDef> fwd, bwd;
    std::vector<char> skip_bwd;
    std::vector<GradBind> binds;
    HeadFuse head;
  };
  void plan_fused_head(MainProgram *mp) const;
  bool run_fused_head(const MainProgram &mp);
  float *output_storage(const std::string &name, long *count);
  void plan_gradient_binds(MainProgram *mp) const;
  const std::vector<GradBind> *binds_ = nullptr;  // of the program being run
  std::map<std::string, MainProgram> main_cache_;  // keyed by the requested targets
  std::map<std::string, void *> fused_handles_;    // kernel name -> compiled module
  int fused_groups_ = 0;
  std::unique_ptr<Engine> engine_;
  std::unique_ptr<Lowering> lowering_;
};

}  // namespace mid
}  // namespace cavs
#endif
