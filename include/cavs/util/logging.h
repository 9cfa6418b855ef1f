// Minimal stand-in for the glog macros the reference's applications use
// (cavs/util/logging.h): LOG(INFO|WARNING|FATAL), CHECK*, VLOG.
#ifndef CAVS_UTIL_LOGGING_H_
#define CAVS_UTIL_LOGGING_H_

#include <cstdlib>
#include <iostream>
#include <sstream>

namespace cavs_log {
enum Severity { INFO = 0, WARNING = 1, ERROR = 2, FATAL = 3 };
int verbosity();  // CAVS_V environment variable, default 0
class Message {
 public:
  Message(const char *file, int line, Severity sev, bool enabled) : sev_(sev), on_(enabled) {
    if (on_) os_ << "[" << "IWEF"[sev] << " " << file << ":" << line << "] ";
  }
  ~Message() noexcept(false);
  std::ostream &stream() { return os_; }
 private:
  std::ostringstream os_;
  Severity sev_;
  bool on_;
};
struct Voidify { void operator&(std::ostream &) {} };
}  // namespace cavs_log

#define V_TIMING 1
#define V_DEBUG 2
#define V_EXHAUSTIVE_DEBUG 3
#define LOG(sev) ::cavs_log::Message(__FILE__, __LINE__, ::cavs_log::sev, true).stream()
#define VLOG(n) \
  if ((n) <= ::cavs_log::verbosity()) ::cavs_log::Message(__FILE__, __LINE__, ::cavs_log::INFO, true).stream()
#define VLOG_IS_ON(n) ((n) <= ::cavs_log::verbosity())
#define CHECK(cond) \
  (cond) ? (void)0 : ::cavs_log::Voidify() & ::cavs_log::Message(__FILE__, __LINE__, ::cavs_log::FATAL, true).stream() << "Check failed: " #cond " "
#define CHECK_NOTNULL(p) CHECK((p) != nullptr)
#define CHECK_EQ(a, b) CHECK((a) == (b))

#endif
