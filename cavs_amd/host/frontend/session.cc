// Session::Run: copies each feed into a cached host tensor, runs, and points every
// requested Sym at the host copy of its value (cavs/frontend/cxx/session.cc:9-49).
#include "cavs/frontend/cxx/session.h"

#include <cstdlib>
#include <cstring>
#include <stdexcept>

Session::~Session() {
  for (auto *t : last_outputs_) C_DeleteTensor(t);
  for (auto &kv : feed_map_) C_DeleteTensor(kv.second);
  C_DeleteSession(s_);
}

void Session::Run(std::vector<Sym> outputs, const std::vector<std::pair<Sym, void *>> &feed) {
  std::vector<C_Tensor *> in_t;
  std::vector<const char *> in_n;
  for (auto &f : feed) {
    const Sym &sym = f.first;
    const string &name = sym.output(0);
    if (!feed_map_.count(name)) {
      std::vector<int> shp = sym.shape(0);
      feed_map_[name] = C_NewTensor(name.c_str(), name.length(), shp.data(), (int)shp.size(), (C_Dtype)sym.type());
    }
    C_Tensor *t = feed_map_[name];
    std::memcpy(C_TensorData(t), f.second, C_TensorSize(t));
    in_t.push_back(t);
    in_n.push_back(name.c_str());
  }
  std::vector<const char *> out_n;
  for (auto &o : outputs) out_n.push_back(o.output(0).c_str());
  std::vector<C_Tensor *> out_t(out_n.size(), nullptr);
  // a failed run throws here; the plain C_Run entry point aborts like the reference's CHECKs
  if (C_TryRun(s_, out_n.data(), out_t.data(), (int)out_n.size(), in_n.data(), in_t.data(), (int)in_n.size()) != 0)
    throw std::runtime_error(C_LastError());
  for (auto *t : last_outputs_) C_DeleteTensor(t);
  last_outputs_ = out_t;
  for (size_t i = 0; i < outputs.size(); i++) *outputs[i].mutable_data() = out_t[i] ? C_TensorData(out_t[i]) : nullptr;
}

void Session::Run(std::vector<Sym> outputs, const std::initializer_list<std::pair<Sym &, void *>> &feed) {
  std::vector<std::pair<Sym, void *>> v;
  for (auto &f : feed) v.emplace_back(f.first, f.second);
  Run(outputs, v);
}

void Session::SetVariable(const Sym &var, const float *data, size_t n) {
  CHECK(C_SetVariable(s_, var.output(0).c_str(), data, n) == 0) << C_LastError();
}

std::vector<float> Session::Read(const std::string &edge_name) {
  long n = C_ReadTensor(s_, edge_name.c_str(), nullptr, 0);
  CHECK(n != 0) << "no tensor named " << edge_name;
  std::vector<float> out((size_t)(n < 0 ? -n : n));
  long got = C_ReadTensor(s_, edge_name.c_str(), out.data(), out.size());
  CHECK(got == (long)out.size()) << C_LastError();
  return out;
}
