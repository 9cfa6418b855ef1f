// OpDef / FunctionDef as plain structs with the accessor names the reference's
// protobuf messages generate (cavs/proto/op_def.proto:7-36, func_def.proto:5-8), plus a
// small length-prefixed serialisation so that definitions can cross the C API as bytes
// like the reference's serialized protobufs do (cavs/frontend/c_api.cc:90-147).
#ifndef CAVS_PROTO_OP_DEF_H_
#define CAVS_PROTO_OP_DEF_H_

#include <cstdint>
#include <string>
#include <vector>

#include "cavs/proto/types.h"

struct TensorShapeDef {
  std::vector<int> dims;
  const std::vector<int> &dim() const { return dims; }
  int dim(int i) const { return dims[i]; }
  int dim_size() const { return (int)dims.size(); }
  void add_dim(int d) { dims.push_back(d); }
  void set_dim(int i, int d) { dims[i] = d; }
  void clear() { dims.clear(); }
};

struct OpDef {
  struct AttrType {
    enum Kind { NONE, S, I, F, B, LIST_S, LIST_I, LIST_F } kind = NONE;
    std::string s;
    int64_t i = 0;
    float f = 0.f;
    bool b = false;
    std::vector<std::string> list_s;
    std::vector<int64_t> list_i;
    std::vector<float> list_f;
    void set_s(const std::string &v) { kind = S; s = v; }
    void set_i(int64_t v) { kind = I; i = v; }
    void set_f(float v) { kind = F; f = v; }
    void set_b(bool v) { kind = B; b = v; }
  };
  struct AttrDef {
    std::string name_;
    AttrType value_;
    void set_name(const std::string &n) { name_ = n; }
    const std::string &name() const { return name_; }
    AttrType *mutable_value() { return &value_; }
    const AttrType &value() const { return value_; }
  };

  std::string name_;
  std::vector<std::string> input_, output_;
  std::vector<TensorShapeDef> shape_;
  DeviceType device_ = GPU;
  DataType dtype_ = DT_FLOAT;
  std::string label_;
  std::vector<AttrDef> attr_;

  const std::string &name() const { return name_; }
  void set_name(const std::string &n) { name_ = n; }
  const std::vector<std::string> &input() const { return input_; }
  const std::string &input(int i) const { return input_[i]; }
  int input_size() const { return (int)input_.size(); }
  void add_input(const std::string &s) { input_.push_back(s); }
  const std::vector<std::string> &output() const { return output_; }
  const std::string &output(int i) const { return output_[i]; }
  int output_size() const { return (int)output_.size(); }
  void add_output(const std::string &s) { output_.push_back(s); }
  const std::vector<TensorShapeDef> &shape() const { return shape_; }
  const TensorShapeDef &shape(int i) const { return shape_[i]; }
  int shape_size() const { return (int)shape_.size(); }
  TensorShapeDef *add_shape() { shape_.emplace_back(); return &shape_.back(); }
  void clear_shape() { shape_.clear(); }
  DeviceType device() const { return device_; }
  DataType dtype() const { return dtype_; }
  const std::string &label() const { return label_; }
  const std::vector<AttrDef> &attr() const { return attr_; }
  const AttrDef *find_attr(const std::string &key) const {
    for (auto &a : attr_) if (a.name_ == key) return &a;
    return nullptr;
  }

  std::string DebugString() const;
  bool SerializeToString(std::string *out) const;
  bool ParseFromArray(const void *data, size_t len);
};

struct FunctionDef {
  std::string name_;
  std::vector<OpDef> ops_;
  const std::string &name() const { return name_; }
  void set_name(const std::string &n) { name_ = n; }
  OpDef *add_ops() { ops_.emplace_back(); return &ops_.back(); }
  const std::vector<OpDef> &ops() const { return ops_; }
  void Clear() { name_.clear(); ops_.clear(); }
  std::string DebugString() const;
  bool SerializeToString(std::string *out) const;
  bool ParseFromArray(const void *data, size_t len);
};

// cavs/util/op_util.h: attribute getters and gradient-name helpers
template <typename T> T GetSingleArg(const OpDef &def, const std::string &key, T dflt);
template <typename T> T GetSingleArg(const OpDef &def, const std::string &key);
std::vector<std::string> GetListArgS(const OpDef &def, const std::string &key);
std::string GetGradientName(const std::string &name);   // X -> X_grad
std::string GetOriginName(const std::string &name);     // X_grad -> X
bool IsGradientName(const std::string &name);

#endif
