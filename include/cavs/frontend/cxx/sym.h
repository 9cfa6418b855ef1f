// Symbolic front end: every call builds one OpDef and either registers it with the
// graph or, between FuncDefineBegin/End, appends it to the vertex function being
// declared.  Same class, method names and argument meaning as the reference's
// cavs/frontend/cxx/sym.h:16-208 so that applications written against it compile
// unchanged.  Operators outside the F-over-G path (Conv, Maxpooling, the cuDNN LSTM,
// MNIST/Data readers) are not declared.
#ifndef CAVS_FRONTEND_CXX_SYM_H_
#define CAVS_FRONTEND_CXX_SYM_H_

#include <memory>
#include <string>
#include <tuple>
#include <utility>
#include <vector>

#include "cavs/frontend/c_api.h"
#include "cavs/proto/op_def.h"
#include "cavs/util/logging.h"

using std::string;

class Sym {
 public:
  typedef std::pair<string, std::vector<OpDef::AttrDef>> ATTRIBUTE;

  Sym() = default;
  explicit Sym(const OpDef &op_def);
  Sym(float constant);  // ConstOp of shape {1}

  const string &output(int idx) const { CHECK(idx < def().output_size()); return def().output(idx); }
  int output_size() const { return def().output_size(); }
  std::vector<string> output() const { return def().output(); }
  std::vector<int> shape(int idx) const { CHECK(idx < def().shape_size()) << def().DebugString(); return def().shape(idx).dims; }
  DataType type() const { return def().dtype(); }
  DeviceType device() const { return def().device(); }
  const string &op_name() const { return def().name(); }
  const OpDef &def() const { CHECK(node_.get()); return node_->op_def; }
  OpDef *mutable_def() { CHECK(node_.get()); return &node_->op_def; }
  const void *data() const { CHECK(node_.get()); return node_->raw_data; }
  void **mutable_data() { CHECK(node_.get()); return &node_->raw_data; }

  // sources
  static Sym Variable(DataType type, const std::vector<int> &shape, const ATTRIBUTE &filler = Ones(),
                      string device = "GPU");
  static Sym Placeholder(DataType type, const std::vector<int> &shape, string device = "GPU");
  static Sym Constant(DataType type, float value, const std::vector<int> &shape, string device = "GPU");
  // unary
  static Sym Abs(const Sym &a, string device = "GPU");
  static Sym Square(const Sym &a, string device = "GPU");
  static Sym Reduce_mean(const Sym &a, string device = "GPU");
  static Sym Reduce_sum(const Sym &a, string device = "GPU");
  static Sym Optimizer(const Sym &a);
  static Sym Optimizer(const Sym &a, std::vector<Sym> variables, float lr, float clip = 0.f, int iters = 1,
                       const string &projections = "");
  static Sym Relu(const Sym &a, string device = "GPU");
  static Sym Sigmoid(const Sym &a, string device = "GPU");
  static Sym Tanh(const Sym &a, string device = "GPU");
  static Sym Flatten(const Sym &a);
  static Sym Slice(const Sym &a, int offset, int stride);
  static Sym Mirror(const Sym &a);
  static std::tuple<Sym, Sym> Split2(const Sym &a);
  static std::tuple<Sym, Sym, Sym> Split3(const Sym &a);
  static std::tuple<Sym, Sym, Sym, Sym> Split4(const Sym &a);
  // binary
  static Sym Add(const Sym &a, const Sym &b, string device = "GPU");
  static Sym Sub(const Sym &a, const Sym &b, string device = "GPU");
  static Sym Mul(const Sym &a, const Sym &b, string device = "GPU");
  static Sym MatMul(const Sym &a, const Sym &b, string device = "GPU");
  static Sym SoftmaxEntropyLoss(const Sym &a, const Sym &b, string device = "GPU");
  static Sym Equal(const Sym &a, const Sym &b, string device = "GPU");
  static Sym EmbeddingLookup(const Sym &a, const Sym &b, string device = "GPU");
  static Sym ControlDependency(const Sym &a, const Sym &b);
  static Sym Reshape(const Sym &a, const std::vector<int> &shape);
  static Sym Expand_dims(const Sym &a, int axis);
  static Sym FullyConnected(const Sym &x, const Sym &w, const Sym &b, string device = "GPU");
  static Sym Concat(const std::vector<Sym> &syms, string device = "GPU");
  // fillers
  static ATTRIBUTE Ones();
  static ATTRIBUTE Zeros();
  static ATTRIBUTE Const(float c);
  static ATTRIBUTE Uniform(float minval, float maxval);
  static ATTRIBUTE Xavier();
  static ATTRIBUTE NormalRandom();
  // debug
  void print();
  const void *eval() const { return data(); }

  // member forms
  Sym Abs() { return Abs(*this); }
  Sym Square() { return Square(*this); }
  Sym Reduce_mean() { return Reduce_mean(*this); }
  Sym Reduce_sum() { return Reduce_sum(*this); }
  Sym Optimizer() { return Optimizer(*this); }
  Sym Optimizer(std::vector<Sym> variables, float lr, float clip = 0.f, int iters = 1, const string &projection = "") {
    return Optimizer(*this, variables, lr, clip, iters, projection);
  }
  Sym Relu() { return Relu(*this); }
  Sym Sigmoid() { return Sigmoid(*this); }
  Sym Tanh() { return Tanh(*this); }
  Sym Flatten() { return Flatten(*this); }
  Sym Slice(int offset, int stride) { return Slice(*this, offset, stride); }
  Sym Mirror() { return Mirror(*this); }
  std::tuple<Sym, Sym> Split2() { return Split2(*this); }
  std::tuple<Sym, Sym, Sym> Split3() { return Split3(*this); }
  std::tuple<Sym, Sym, Sym, Sym> Split4() { return Split4(*this); }
  Sym SoftmaxEntropyLoss(const Sym &b) { return SoftmaxEntropyLoss(*this, b); }
  Sym EmbeddingLookup(const Sym &b) { return EmbeddingLookup(*this, b); }
  Sym ControlDependency(const Sym &b) { return ControlDependency(*this, b); }
  Sym Reshape(const std::vector<int> &shape) { return Reshape(*this, shape); }
  Sym Expand_dims(int axis) { return Expand_dims(*this, axis); }
  Sym FullyConnected(const Sym &w, const Sym &b) { return FullyConnected(*this, w, b); }

  friend Sym operator+(const Sym &a, const Sym &b) { return Add(a, b); }
  friend Sym operator-(const Sym &a, const Sym &b) { return Sub(a, b); }
  friend Sym operator*(const Sym &a, const Sym &b) { return Mul(a, b); }

 private:
  struct node_t {
    OpDef op_def;
    void *raw_data = nullptr;
  };
  std::shared_ptr<node_t> node_;
};

// Recording state of a vertex-function declaration (cavs/frontend/cxx/sym.h:181-208).
class FuncConf {
 public:
  static void FuncDefineBegin(const string &name) { Get()->name_ = name; Get()->def_.set_name(name); }
  static FunctionDef FuncDefineEnd(const string &name) {
    CHECK(name == Get()->name_);
    FunctionDef ret = Get()->def_;
    Get()->name_.clear();
    Get()->def_.Clear();
    return ret;
  }
  static bool CheckInFunc() { return !Get()->name_.empty(); }
  static FunctionDef *mutable_funcdef() { CHECK(CheckInFunc()); return &Get()->def_; }

 private:
  static FuncConf *Get() { static FuncConf fc; return &fc; }
  string name_;
  FunctionDef def_;
};

#endif
