// OpDef / FunctionDef helpers: debug text, byte serialisation, attribute getters,
// gradient-name helpers (cavs/util/op_util.cc:9-47), and the tiny logger.
#include <cstring>
#include <stdexcept>

#include "cavs/proto/op_def.h"
#include "cavs/util/logging.h"

namespace cavs_log {
int verbosity() {
  static int v = [] {
    const char *e = std::getenv("CAVS_V");
    return e ? std::atoi(e) : 0;
  }();
  return v;
}
Message::~Message() noexcept(false) {
  if (!on_) return;
  os_ << "\n";
  std::cerr << os_.str() << std::flush;
  if (sev_ == FATAL) throw std::runtime_error(os_.str());
}
}  // namespace cavs_log

namespace {
struct Writer {
  std::string *o;
  void u32(uint32_t v) { o->append(reinterpret_cast<const char *>(&v), 4); }
  void i64(int64_t v) { o->append(reinterpret_cast<const char *>(&v), 8); }
  void f32(float v) { o->append(reinterpret_cast<const char *>(&v), 4); }
  void str(const std::string &s) { u32((uint32_t)s.size()); o->append(s); }
};
struct Reader {
  const char *p, *end;
  bool ok = true;
  bool need(size_t n) { if ((size_t)(end - p) < n) ok = false; return ok; }
  uint32_t u32() { uint32_t v = 0; if (need(4)) { std::memcpy(&v, p, 4); p += 4; } return v; }
  int64_t i64() { int64_t v = 0; if (need(8)) { std::memcpy(&v, p, 8); p += 8; } return v; }
  float f32() { float v = 0; if (need(4)) { std::memcpy(&v, p, 4); p += 4; } return v; }
  std::string str() { uint32_t n = u32(); std::string s; if (need(n)) { s.assign(p, n); p += n; } return s; }
};

void write_op(Writer &w, const OpDef &d) {
  w.str(d.name_);
  w.u32((uint32_t)d.input_.size());
  for (auto &s : d.input_) w.str(s);
  w.u32((uint32_t)d.output_.size());
  for (auto &s : d.output_) w.str(s);
  w.u32((uint32_t)d.shape_.size());
  for (auto &s : d.shape_) {
    w.u32((uint32_t)s.dims.size());
    for (int x : s.dims) w.i64(x);
  }
  w.u32(d.device_);
  w.u32(d.dtype_);
  w.str(d.label_);
  w.u32((uint32_t)d.attr_.size());
  for (auto &a : d.attr_) {
    w.str(a.name_);
    const auto &v = a.value_;
    w.u32(v.kind);
    w.str(v.s);
    w.i64(v.i);
    w.f32(v.f);
    w.u32(v.b);
    w.u32((uint32_t)v.list_s.size());
    for (auto &s : v.list_s) w.str(s);
    w.u32((uint32_t)v.list_i.size());
    for (auto x : v.list_i) w.i64(x);
    w.u32((uint32_t)v.list_f.size());
    for (auto x : v.list_f) w.f32(x);
  }
}

bool read_op(Reader &r, OpDef *d) {
  *d = OpDef();
  d->name_ = r.str();
  for (uint32_t n = r.u32(), i = 0; i < n && r.ok; i++) d->input_.push_back(r.str());
  for (uint32_t n = r.u32(), i = 0; i < n && r.ok; i++) d->output_.push_back(r.str());
  for (uint32_t n = r.u32(), i = 0; i < n && r.ok; i++) {
    TensorShapeDef s;
    for (uint32_t m = r.u32(), j = 0; j < m && r.ok; j++) s.dims.push_back((int)r.i64());
    d->shape_.push_back(s);
  }
  d->device_ = (DeviceType)r.u32();
  d->dtype_ = (DataType)r.u32();
  d->label_ = r.str();
  for (uint32_t n = r.u32(), i = 0; i < n && r.ok; i++) {
    OpDef::AttrDef a;
    a.name_ = r.str();
    auto &v = a.value_;
    v.kind = (OpDef::AttrType::Kind)r.u32();
    v.s = r.str();
    v.i = r.i64();
    v.f = r.f32();
    v.b = r.u32() != 0;
    for (uint32_t m = r.u32(), j = 0; j < m && r.ok; j++) v.list_s.push_back(r.str());
    for (uint32_t m = r.u32(), j = 0; j < m && r.ok; j++) v.list_i.push_back(r.i64());
    for (uint32_t m = r.u32(), j = 0; j < m && r.ok; j++) v.list_f.push_back(r.f32());
    d->attr_.push_back(a);
  }
  return r.ok;
}
}  // namespace

std::string OpDef::DebugString() const {
  std::ostringstream o;
  o << name_ << "(";
  for (size_t i = 0; i < input_.size(); i++) o << (i ? ", " : "") << input_[i];
  o << ") -> (";
  for (size_t i = 0; i < output_.size(); i++) o << (i ? ", " : "") << output_[i];
  o << ")";
  for (auto &s : shape_) {
    o << " [";
    for (size_t i = 0; i < s.dims.size(); i++) o << (i ? "," : "") << s.dims[i];
    o << "]";
  }
  for (auto &a : attr_) {
    o << " " << a.name_ << "=";
    switch (a.value_.kind) {
      case AttrType::S: o << a.value_.s; break;
      case AttrType::I: o << a.value_.i; break;
      case AttrType::F: o << a.value_.f; break;
      case AttrType::B: o << (a.value_.b ? "true" : "false"); break;
      default: o << "<list>";
    }
  }
  return o.str();
}

bool OpDef::SerializeToString(std::string *out) const {
  out->clear();
  Writer w{out};
  write_op(w, *this);
  return true;
}

bool OpDef::ParseFromArray(const void *data, size_t len) {
  Reader r{static_cast<const char *>(data), static_cast<const char *>(data) + len};
  return read_op(r, this) && r.p == r.end;
}

std::string FunctionDef::DebugString() const {
  std::string s = "function " + name_ + " {\n";
  for (auto &o : ops_) s += "  " + o.DebugString() + "\n";
  return s + "}";
}

bool FunctionDef::SerializeToString(std::string *out) const {
  out->clear();
  Writer w{out};
  w.str(name_);
  w.u32((uint32_t)ops_.size());
  for (auto &o : ops_) write_op(w, o);
  return true;
}

bool FunctionDef::ParseFromArray(const void *data, size_t len) {
  Reader r{static_cast<const char *>(data), static_cast<const char *>(data) + len};
  Clear();
  name_ = r.str();
  for (uint32_t n = r.u32(), i = 0; i < n && r.ok; i++) {
    OpDef d;
    if (!read_op(r, &d)) return false;
    ops_.push_back(d);
  }
  return r.ok && r.p == r.end;
}

template <> int GetSingleArg<int>(const OpDef &def, const std::string &key, int dflt) {
  auto *a = def.find_attr(key);
  return a ? (int)a->value_.i : dflt;
}
template <> float GetSingleArg<float>(const OpDef &def, const std::string &key, float dflt) {
  auto *a = def.find_attr(key);
  if (!a) return dflt;
  return a->value_.kind == OpDef::AttrType::I ? (float)a->value_.i : a->value_.f;
}
template <> bool GetSingleArg<bool>(const OpDef &def, const std::string &key, bool dflt) {
  auto *a = def.find_attr(key);
  return a ? a->value_.b : dflt;
}
template <> std::string GetSingleArg<std::string>(const OpDef &def, const std::string &key, std::string dflt) {
  auto *a = def.find_attr(key);
  return a ? a->value_.s : dflt;
}
template <> int GetSingleArg<int>(const OpDef &def, const std::string &key) {
  CHECK(def.find_attr(key)) << "missing attribute " << key << " in " << def.DebugString();
  return GetSingleArg<int>(def, key, 0);
}
template <> float GetSingleArg<float>(const OpDef &def, const std::string &key) {
  CHECK(def.find_attr(key)) << "missing attribute " << key << " in " << def.DebugString();
  return GetSingleArg<float>(def, key, 0.f);
}
std::vector<std::string> GetListArgS(const OpDef &def, const std::string &key) {
  auto *a = def.find_attr(key);
  return a ? a->value_.list_s : std::vector<std::string>();
}

std::string GetGradientName(const std::string &name) { return name + "_grad"; }
bool IsGradientName(const std::string &name) {
  return name.size() > 5 && name.compare(name.size() - 5, 5, "_grad") == 0;
}
std::string GetOriginName(const std::string &name) {
  CHECK(IsGradientName(name)) << name;
  return name.substr(0, name.size() - 5);
}
