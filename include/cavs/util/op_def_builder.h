// cavs/util/op_def_builder.h:12-55 restated over the plain OpDef struct.
#ifndef CAVS_UTIL_OP_DEF_BUILDER_H_
#define CAVS_UTIL_OP_DEF_BUILDER_H_

#include <string>
#include <vector>

#include "cavs/proto/op_def.h"

class OpDefBuilder {
 public:
  explicit OpDefBuilder(const std::string &op_name) { op_def_.set_name(op_name); }
  OpDefBuilder &Input(const std::string &input) { op_def_.add_input(input); return *this; }
  OpDefBuilder &Input(const std::vector<std::string> &inputs) { for (auto &s : inputs) op_def_.add_input(s); return *this; }
  OpDefBuilder &Output(const std::string &output) { op_def_.add_output(output); return *this; }
  OpDefBuilder &Output(const std::vector<std::string> &outputs) { for (auto &s : outputs) op_def_.add_output(s); return *this; }
  OpDefBuilder &Device(const std::string &dev) { op_def_.device_ = (dev == "CPU") ? CPU : GPU; return *this; }
  OpDefBuilder &Device(DeviceType t) { op_def_.device_ = t; return *this; }
  OpDefBuilder &Device(const OpDef &def) { op_def_.device_ = def.device_; return *this; }
  OpDefBuilder &Shape(const std::vector<int> &shape) { op_def_.clear_shape(); op_def_.add_shape()->dims = shape; return *this; }
  OpDefBuilder &Shape(const OpDef &def) { op_def_.shape_ = def.shape_; return *this; }
  OpDefBuilder &Dtype(DataType t) { op_def_.dtype_ = t; return *this; }
  OpDefBuilder &Label(const std::string &l) { op_def_.label_ = l; return *this; }
  OpDefBuilder &Attr(const OpDef &def) { for (auto &a : def.attr_) op_def_.attr_.push_back(a); return *this; }
  OpDefBuilder &Attr(const OpDef::AttrDef &a) { op_def_.attr_.push_back(a); return *this; }
  OpDefBuilder &Attr(const std::vector<OpDef::AttrDef> &v) { for (auto &a : v) op_def_.attr_.push_back(a); return *this; }
  OpDefBuilder &AttrSingle(const std::string &key, int v) { return add(key, [&](OpDef::AttrType *t) { t->set_i(v); }); }
  OpDefBuilder &AttrSingle(const std::string &key, float v) { return add(key, [&](OpDef::AttrType *t) { t->set_f(v); }); }
  OpDefBuilder &AttrSingle(const std::string &key, double v) { return add(key, [&](OpDef::AttrType *t) { t->set_f((float)v); }); }
  OpDefBuilder &AttrSingle(const std::string &key, bool v) { return add(key, [&](OpDef::AttrType *t) { t->set_b(v); }); }
  OpDefBuilder &AttrSingle(const std::string &key, const std::string &v) { return add(key, [&](OpDef::AttrType *t) { t->set_s(v); }); }
  OpDefBuilder &AttrSingle(const std::string &key, const char *v) { return AttrSingle(key, std::string(v)); }
  OpDefBuilder &AttrList(const std::string &key, const std::vector<std::string> &v) {
    return add(key, [&](OpDef::AttrType *t) { t->kind = OpDef::AttrType::LIST_S; t->list_s = v; });
  }
  OpDefBuilder &AttrList(const std::string &key, const std::vector<int> &v) {
    return add(key, [&](OpDef::AttrType *t) { t->kind = OpDef::AttrType::LIST_I; t->list_i.assign(v.begin(), v.end()); });
  }
  const OpDef &Finalize() const { return op_def_; }
  void Finalize(OpDef *out) const { *out = op_def_; }

 private:
  template <typename F>
  OpDefBuilder &add(const std::string &key, F &&set) {
    for (auto &a : op_def_.attr_)
      if (a.name_ == key) { set(&a.value_); return *this; }
    OpDef::AttrDef a;
    a.set_name(key);
    set(a.mutable_value());
    op_def_.attr_.push_back(a);
    return *this;
  }
  OpDef op_def_;
};

#endif
