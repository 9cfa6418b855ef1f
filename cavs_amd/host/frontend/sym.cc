// Sym: one OpDef per call.  Outside a function declaration the definition is
// registered through the C API (which also returns the inferred shape); inside one it
// is appended to the FunctionDef being recorded (cavs/frontend/cxx/sym.cc:14-49).
#include "cavs/frontend/cxx/sym.h"

#include <cstdlib>
#include <iomanip>

#include "cavs/util/op_def_builder.h"

using std::vector;

Sym::Sym(const OpDef &op_def) {
  node_ = std::make_shared<node_t>();
  node_->op_def = op_def;
  static int next_id = 0;
  if (def().output_size() == 0) mutable_def()->add_output(op_name() + "_" + std::to_string(next_id++));
  if (FuncConf::CheckInFunc()) {
    CHECK(op_name() != "Optimizer") << "an optimizer cannot be declared inside a vertex function";
    *FuncConf::mutable_funcdef()->add_ops() = def();
    return;
  }
  string bytes;
  def().SerializeToString(&bytes);
  if (op_name() == "Optimizer") {
    C_AddOptimizerOp(bytes.data(), bytes.size());
  } else if (op_name() == "ControlDependency") {
    C_AddControlDependency(bytes.data(), bytes.size());
  } else {
    int *dim = nullptr;
    size_t n = 0;
    C_AddOp(bytes.data(), bytes.size(), &dim, &n);
    CHECK_NOTNULL(dim);
    mutable_def()->clear_shape();
    TensorShapeDef *s = mutable_def()->add_shape();
    for (size_t i = 0; i < n; i++) s->add_dim(dim[i]);
    std::free(dim);
  }
}

Sym::Sym(float c) {
  *this = Sym(OpDefBuilder("ConstOp").Dtype(DT_FLOAT).Device("GPU").Shape({1}).AttrSingle("init", c).Finalize());
}

static OpDef unary(const char *name, const Sym &a, const string &device) {
  return OpDefBuilder(name).Input(a.output(0)).Dtype(a.type()).Device(device).Finalize();
}
static OpDef binary(const char *name, const Sym &a, const Sym &b, const string &device) {
  CHECK(a.type() == b.type());
  CHECK(a.output_size() == 1 && b.output_size() == 1);
  return OpDefBuilder(name).Input(a.output(0)).Input(b.output(0)).Dtype(a.type()).Device(device).Finalize();
}
static string dev_of(const Sym &a) { return a.device() == CPU ? "CPU" : "GPU"; }

Sym Sym::Variable(DataType type, const vector<int> &shape, const ATTRIBUTE &filler, string device) {
  CHECK(!shape.empty());
  return Sym(OpDefBuilder("Variable").Dtype(type).Label(filler.first).Device(device).Shape(shape).Attr(filler.second).Finalize());
}
Sym Sym::Placeholder(DataType type, const vector<int> &shape, string device) {
  CHECK(!shape.empty());
  return Sym(OpDefBuilder("Placeholder").Dtype(type).Device(device).Shape(shape).Finalize());
}
Sym Sym::Constant(DataType type, float value, const vector<int> &shape, string device) {
  CHECK(!shape.empty());
  return Sym(OpDefBuilder("ConstOp").Dtype(type).Device(device).Shape(shape).AttrSingle("init", value).Finalize());
}
Sym Sym::Abs(const Sym &a, string device) { return Sym(unary("Abs", a, device)); }
Sym Sym::Square(const Sym &a, string device) { return Sym(unary("Square", a, device)); }
Sym Sym::Reduce_mean(const Sym &a, string device) { return Sym(unary("Reduce_mean", a, device)); }
Sym Sym::Reduce_sum(const Sym &a, string device) { return Sym(unary("Reduce_sum", a, device)); }
Sym Sym::Relu(const Sym &a, string device) { return Sym(unary("Relu", a, device)); }
Sym Sym::Sigmoid(const Sym &a, string device) { return Sym(unary("Sigmoid", a, device)); }
Sym Sym::Tanh(const Sym &a, string device) { return Sym(unary("Tanh", a, device)); }

Sym Sym::Optimizer(const Sym &a) {
  CHECK(a.output_size() == 1);
  return Sym(OpDefBuilder("Optimizer").Input(a.output(0)).Dtype(a.type()).AttrSingle("Learning_rate", 1.f)
                 .AttrSingle("Iters", 1).AttrSingle("Solver", "SGD").Finalize());
}
Sym Sym::Optimizer(const Sym &a, vector<Sym> variables, float lr, float clip, int iters, const string &projection) {
  CHECK(iters > 0);
  CHECK(a.output_size() == 1);
  vector<string> vars;
  for (auto &v : variables) vars.push_back(v.output(0));
  return Sym(OpDefBuilder("Optimizer").Input(a.output(0)).Dtype(a.type()).AttrList("Vars", vars)
                 .AttrSingle("Learning_rate", lr).AttrSingle("Clip", clip).AttrSingle("Iters", iters)
                 .AttrSingle("Projection", projection).AttrSingle("Solver", "SGD").Finalize());
}

static OpDef aliasing(const char *name, const Sym &a) {
  return OpDefBuilder(name).Input(a.output(0)).Dtype(a.type()).Device(dev_of(a)).AttrSingle("ShareMemory", true).Finalize();
}
Sym Sym::Flatten(const Sym &a) { return Sym(aliasing("Flatten", a)); }
Sym Sym::Mirror(const Sym &a) { return Sym(aliasing("Mirror", a)); }
Sym Sym::Reshape(const Sym &a, const vector<int> &shape) {
  return Sym(OpDefBuilder("Reshape").Input(a.output(0)).Dtype(a.type()).Device(dev_of(a)).Shape(shape)
                 .AttrSingle("ShareMemory", true).Finalize());
}
Sym Sym::Expand_dims(const Sym &a, int axis) {
  return Sym(OpDefBuilder("Expand_dims").Input(a.output(0)).Dtype(a.type()).Device(dev_of(a))
                 .AttrSingle("ShareMemory", true).AttrSingle("Axis", axis).Finalize());
}
Sym Sym::Slice(const Sym &a, int offset, int stride) {
  return Sym(OpDefBuilder("Slice").Input(a.output(0)).Dtype(a.type()).Device(dev_of(a)).AttrSingle("Axis", 0)
                 .AttrSingle("Offset", offset).AttrSingle("Stride", stride).Finalize());
}
static OpDef split_piece(const Sym &a, int parts, int index) {
  return OpDefBuilder("Slice").Input(a.output(0)).Dtype(a.type()).Device(dev_of(a)).AttrSingle("Split", parts)
      .AttrSingle("Index", index).AttrSingle("Axis", 0).Finalize();
}
std::tuple<Sym, Sym> Sym::Split2(const Sym &a) {
  Sym s0(split_piece(a, 2, 0)), s1(split_piece(a, 2, 1));
  return std::make_tuple(s0, s1);
}
std::tuple<Sym, Sym, Sym> Sym::Split3(const Sym &a) {
  Sym s0(split_piece(a, 3, 0)), s1(split_piece(a, 3, 1)), s2(split_piece(a, 3, 2));
  return std::make_tuple(s0, s1, s2);
}
std::tuple<Sym, Sym, Sym, Sym> Sym::Split4(const Sym &a) {
  Sym s0(split_piece(a, 4, 0)), s1(split_piece(a, 4, 1)), s2(split_piece(a, 4, 2)), s3(split_piece(a, 4, 3));
  return std::make_tuple(s0, s1, s2, s3);
}

Sym Sym::Add(const Sym &a, const Sym &b, string device) { return Sym(binary("Add", a, b, device)); }
Sym Sym::Sub(const Sym &a, const Sym &b, string device) { return Sym(binary("Sub", a, b, device)); }
Sym Sym::Mul(const Sym &a, const Sym &b, string device) { return Sym(binary("Mul", a, b, device)); }
Sym Sym::MatMul(const Sym &a, const Sym &b, string device) { return Sym(binary("MatMul", a, b, device)); }
Sym Sym::SoftmaxEntropyLoss(const Sym &a, const Sym &b, string device) { return Sym(binary("SoftmaxEntropyLoss", a, b, device)); }
Sym Sym::Equal(const Sym &a, const Sym &b, string device) { return Sym(binary("Equal", a, b, device)); }
Sym Sym::EmbeddingLookup(const Sym &a, const Sym &b, string device) { return Sym(binary("EmbeddingLookup", a, b, device)); }
Sym Sym::ControlDependency(const Sym &a, const Sym &b) {
  return Sym(OpDefBuilder("ControlDependency").Input(a.output(0)).Input(b.output(0)).Finalize());
}
Sym Sym::FullyConnected(const Sym &x, const Sym &w, const Sym &b, string device) {
  return Sym(OpDefBuilder("FullyConnected").Input(x.output(0)).Input(w.output(0)).Input(b.output(0)).Dtype(x.type())
                 .Device(device).Finalize());
}
Sym Sym::Concat(const vector<Sym> &syms, string device) {
  vector<string> inputs;
  for (auto &s : syms) {
    CHECK(s.output_size() == 1);
    CHECK(s.type() == syms[0].type());
    inputs.push_back(s.output(0));
  }
  return Sym(OpDefBuilder("Concat").Input(inputs).Dtype(syms[0].type()).Device(dev_of(syms[0])).AttrSingle("Axis", 0).Finalize());
}

static Sym::ATTRIBUTE filler(const char *label, std::initializer_list<std::pair<const char *, float>> kv) {
  vector<OpDef::AttrDef> v;
  for (auto &p : kv) {
    OpDef::AttrDef a;
    a.set_name(p.first);
    a.mutable_value()->set_f(p.second);
    v.push_back(a);
  }
  return std::make_pair(string(label), v);
}
Sym::ATTRIBUTE Sym::Ones() { return filler("ConstantFiller", {{"const_value", 1.f}}); }
Sym::ATTRIBUTE Sym::Zeros() { return filler("ConstantFiller", {{"const_value", 0.f}}); }
Sym::ATTRIBUTE Sym::Const(float c) { return filler("ConstantFiller", {{"const_value", c}}); }
Sym::ATTRIBUTE Sym::Uniform(float lo, float hi) { return filler("Uniform", {{"minval", lo}, {"maxval", hi}}); }
Sym::ATTRIBUTE Sym::Xavier() { return filler("Xavier", {}); }
Sym::ATTRIBUTE Sym::NormalRandom() { return filler("Normal", {}); }

void Sym::print() {
  CHECK_NOTNULL(data());
  long n = 1;
  for (int d : shape(0)) n *= d;
  for (long i = 0; i < std::min<long>(n, 10); i++)
    LOG(INFO) << "[" << i << "]:\t" << std::fixed << std::setprecision(15) << static_cast<const float *>(data())[i];
}
