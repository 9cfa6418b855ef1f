// Session(opt): opt is the OptLevel bitmask (OPT_FUSION | OPT_BATCHING | OPT_STREAMMING),
// cavs/frontend/cxx/session.h:13-36.  Run() feeds host arrays, executes the requested
// symbols and exposes their values through Sym::eval().
#ifndef CAVS_FRONTEND_CXX_SESSION_H_
#define CAVS_FRONTEND_CXX_SESSION_H_

#include <initializer_list>
#include <string>
#include <unordered_map>
#include <vector>

#include "cavs/frontend/c_api.h"
#include "cavs/frontend/cxx/sym.h"
#include "cavs/proto/opt.pb.h"

class Session {
 public:
  Session(int opt = 0, std::string name = "SimpleSession") { s_ = C_NewSession(name.c_str(), name.length(), opt); }
  ~Session();
  Session(const Session &) = delete;
  Session &operator=(const Session &) = delete;

  void Run(std::vector<Sym> outputs, const std::initializer_list<std::pair<Sym &, void *>> &feed = {});
  void Run(Sym &output, const std::initializer_list<std::pair<Sym &, void *>> &feed = {}) {
    std::vector<Sym> out = {output};
    Run(out, feed);
  }
  // same, with the feeds in a container (extension: initializer lists cannot be built at run time)
  void Run(std::vector<Sym> outputs, const std::vector<std::pair<Sym, void *>> &feed);

  // ---- extensions (no counterpart in the reference) ----
  void SetVariable(const Sym &var, const float *data, size_t n);
  std::vector<float> Read(const std::string &edge_name);
  bool UsesFusedPath() const { return C_SessionUsesFusedPath(s_) != 0; }
  int GeneratedKernels() const { return C_SessionGeneratedKernels(s_); }
  int FusedPathKind() const { return C_SessionUsesFusedPath(s_); }  // 0 none, 1 hand-written, 2 generated
  void AllowFusedPath(bool allow) { C_SessionAllowFusedPath(s_, allow ? 1 : 0); }
  void SetLoweringMode(int mode) { C_SessionAllowFusedPath(s_, mode); }  // 0 none, 1 any, 2 generated kernels only, 3 the same with split backward rounds
  void SetPairing(int pairing) { C_SessionSetPairing(s_, pairing); }
  C_Session *handle() const { return s_; }

 private:
  C_Session *s_;
  std::unordered_map<string, C_Tensor *> feed_map_;
  std::vector<C_Tensor *> last_outputs_;
};

#endif
