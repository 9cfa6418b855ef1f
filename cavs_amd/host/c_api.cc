// extern "C" surface of the host runtime (cavs_session.h): exceptions end here.
#include <algorithm>
#include <vector>
#include <cstdio>
#include <cstring>
#include <string>

#include "cavs_session.h"
#include "engine.h"

struct cavs_session {
  cavs::Engine engine;
  explicit cavs_session(const cavs_session_config &c) : engine(c) {}
};

namespace {
thread_local std::string g_error;

template <typename F>
int guarded(F &&f) {
  try {
    f();
    return CAVS_OK;
  } catch (const cavs::Error &e) {
    g_error = e.what();
    return e.code;
  } catch (const std::bad_alloc &) {
    g_error = "host allocation failed";
    return CAVS_ENOMEM;
  } catch (const std::exception &e) {
    g_error = e.what();
    return CAVS_EINVAL;
  }
}

int need(const void *p, const char *what) {
  if (p) return CAVS_OK;
  g_error = std::string("null ") + what;
  return CAVS_EINVAL;
}

int emit(const std::vector<int> &t, int *out, int cap) {
  if ((int)t.size() > cap || !out) return -(int)t.size();
  std::memcpy(out, t.data(), sizeof(int) * t.size());
  return (int)t.size();
}
}  // namespace

extern "C" {

const char *cavs_session_error(void) { return g_error.c_str(); }

int cavs_session_create(const cavs_session_config *cfg, cavs_session **out) {
  if (int rc = need(cfg, "config")) return rc;
  if (int rc = need(out, "out pointer")) return rc;
  *out = nullptr;
  return guarded([&] { *out = new cavs_session(*cfg); });
}

int cavs_session_destroy(cavs_session *s) {
  return guarded([&] { delete s; });
}

int cavs_session_set_param(cavs_session *s, const char *name, const float *host, size_t n) {
  if (int rc = need(s, "session")) return rc;
  if (int rc = need(name, "parameter name")) return rc;
  return guarded([&] { s->engine.set_param(name, host, n); });
}

int cavs_session_get_param(cavs_session *s, const char *name, float *host, size_t n) {
  if (int rc = need(s, "session")) return rc;
  if (int rc = need(name, "parameter name")) return rc;
  return guarded([&] { s->engine.get_param(name, host, n, false); });
}

int cavs_session_get_grad(cavs_session *s, const char *name, float *host, size_t n) {
  if (int rc = need(s, "session")) return rc;
  if (int rc = need(name, "parameter name")) return rc;
  return guarded([&] { s->engine.get_param(name, host, n, true); });
}

int cavs_session_step(cavs_session *s, const int *graph, int B, int maxlen, const void *x,
                      const void *labels, int inputs_on_device, int backward, float lr) {
  if (int rc = need(s, "session")) return rc;
  return guarded([&] { s->engine.step(graph, B, maxlen, x, labels, inputs_on_device != 0, backward != 0, lr); });
}

int cavs_session_sync(cavs_session *s) {
  if (int rc = need(s, "session")) return rc;
  return guarded([&] { s->engine.sync(); });
}

int cavs_session_fetch(cavs_session *s, const char *what, float *host, size_t n) {
  if (int rc = need(s, "session")) return rc;
  if (int rc = need(what, "result name")) return rc;
  return guarded([&] { s->engine.fetch(what, host, n); });
}

int cavs_session_total_length(cavs_session *s) { return s ? s->engine.total_length() : CAVS_EINVAL; }

int cavs_session_schedule_trace(cavs_session *s, int *out, int cap) {
  if (!s) return 0;
  std::vector<int> t;
  if (guarded([&] { t = s->engine.schedule().trace(true); }) != CAVS_OK) return 0;
  return emit(t, out, cap);
}

int cavs_schedule_trace(const int *graph, int B, int maxlen, int batching, int with_backward, int *out,
                        int cap) {
  cavs::Schedule sch;
  std::string err = cavs::build_schedule(graph, B, maxlen, batching != 0, &sch);
  if (!err.empty()) {
    g_error = err;
    return 0;
  }
  return emit(sch.trace(with_backward != 0), out, cap);
}

int cavs_schedule_index_lists(const int *graph, int B, int maxlen, int nchild, int pairing, int fused_limit, int *t2j,
                              int *pair, int *child, int *roots, int *kid_rows, int *orphans, int *n_orphans) {
  cavs::Schedule sch;
  std::string err = cavs::build_schedule(graph, B, maxlen, true, &sch);
  if (err.empty() && sch.executed != sch.N) err = "the batch holds a single-vertex sample";
  if (err.empty() && (nchild < 1 || nchild > 2 || pairing < 0 || pairing > 1)) err = "bad nchild or pairing";
  if (err.empty() && !(t2j && pair && child && roots)) err = "null output";
  if (err.empty()) err = cavs::build_index_lists(sch, nchild, pairing, t2j, pair, child, roots);
  if (!err.empty()) {
    g_error = err;
    return 0;
  }
  if (n_orphans) {
    int n = 0;
    const bool ok = kid_rows && orphans && cavs::build_forest_lists(sch, nchild, fused_limit, pair, child, kid_rows, orphans, &n);
    *n_orphans = ok ? n : -1;
  }
  return sch.N;
}

int cavs_schedule_tail_lists(const int *graph, int B, int maxlen, int pairing, int fused_limit, int rows_limit, int groups,
                             int max_lists, int *meta, int *nrounds, int *start, int *count, int *flags, int *bstart, int *bcount,
                             int *bflags, int *rows_out) {
  if (!graph || B <= 0 || maxlen <= 0 || pairing < 0 || pairing > 1 || groups < 1 || groups > 8 || max_lists < 1 || rows_limit < 1 ||
      !meta || !nrounds || !start || !count || !flags || !bstart || !bcount || !bflags || !rows_out) {
    g_error = "bad arguments";
    return -1;
  }
  cavs::Schedule sch;
  std::string err = cavs::build_schedule(graph, B, maxlen, true, &sch);
  if (err.empty() && sch.executed != sch.N) err = "the batch holds a single-vertex sample";
  const size_t N = err.empty() ? (size_t)sch.N : 0;
  std::vector<int> t2j(N), pair(N), child(2 * N), roots((size_t)B), kid(2 * N), orphans(N);
  if (err.empty()) err = cavs::build_index_lists(sch, 2, pairing, t2j.data(), pair.data(), child.data(), roots.data());
  if (!err.empty()) {
    g_error = err;
    return -1;
  }
  meta[0] = -1;
  meta[1] = meta[2] = meta[3] = 0;
  int n_orphans = 0;
  if (!cavs::build_forest_lists(sch, 2, fused_limit, pair.data(), child.data(), kid.data(), orphans.data(), &n_orphans)) return 0;
  cavs::TailLists t;
  cavs::build_tail_lists(sch, kid.data(), rows_limit, groups, max_lists, 32, &t, rows_out);
  if (t.first < 0) return 0;
  meta[0] = t.first;
  meta[1] = t.max_rounds;
  meta[2] = t.lists_max;
  meta[3] = t.tiles_max;
  std::copy(t.nrounds.begin(), t.nrounds.end(), nrounds);
  const size_t n = (size_t)groups * t.max_rounds;
  std::copy(t.start.begin(), t.start.begin() + n, start);
  std::copy(t.count.begin(), t.count.begin() + n, count);
  std::copy(t.flags.begin(), t.flags.begin() + n, flags);
  std::copy(t.bstart.begin(), t.bstart.begin() + n, bstart);
  std::copy(t.bcount.begin(), t.bcount.begin() + n, bcount);
  std::copy(t.bflags.begin(), t.bflags.begin() + n, bflags);
  return (int)t.rows;
}

int cavs_schedule_trace_from_lists(int B, int maxlen, int N, int nchild, const int *round2offset, int R, const int *t2j,
                                   const int *pair, const int *child, const int *roots, int with_backward, int *out, int cap) {
  if (B <= 0 || N <= 0 || R < 0 || !round2offset || !t2j || !pair || !child || !roots) {
    g_error = "bad arguments";
    return 0;
  }
  // the lists index each other: nothing out of range may reach the rebuilding code
  if (nchild < 1 || nchild > 2 || maxlen <= 0) {
    g_error = "bad arguments: 1 or 2 children per vertex, positive maxlen";
    return 0;
  }
  if (round2offset[0] != 0 || round2offset[R] != N) {
    g_error = "round offsets must start at 0 and end at N";
    return 0;
  }
  for (int r = 0; r < R; r++)
    if (round2offset[r + 1] < round2offset[r]) {
      g_error = "round offsets must not decrease";
      return 0;
    }
  {
    std::vector<char> seen((size_t)N, 0);
    for (int t = 0; t < N; t++) {
      if (t2j[t] < 0 || t2j[t] >= N || seen[t2j[t]]) {
        g_error = "t2j is not a permutation of the vertex ids";
        return 0;
      }
      seen[t2j[t]] = 1;
    }
  }
  for (int i = 0; i < B; i++)
    if (roots[i] < 0 || roots[i] >= N || (i > 0 && roots[i] <= roots[i - 1])) {
      g_error = "roots must be increasing vertex ids below N";
      return 0;
    }
  for (size_t i = 0; i < (size_t)nchild * N; i++)
    if (child[i] >= N) {
      g_error = "a child list names a row beyond N";
      return 0;
    }
  for (int t = 0; t < N; t++)
    if (pair[t] >= N) {
      g_error = "the scatter list names a row beyond N";
      return 0;
    }
  cavs::Schedule sch;
  cavs::schedule_from_lists(B, maxlen, N, nchild, round2offset, R, t2j, pair, child, roots, &sch);
  return emit(sch.trace(with_backward != 0), out, cap);
}

int cavs_session_timing(cavs_session *s, const char *name, float *ms) {
  if (int rc = need(s, "session")) return rc;
  if (int rc = need(ms, "output")) return rc;
  return guarded([&] { *ms = s->engine.timing(name ? name : ""); });
}

int cavs_session_profile(cavs_session *s, int enable) {
  if (int rc = need(s, "session")) return rc;
  return guarded([&] { s->engine.profile_enable(enable != 0); });
}

int cavs_session_profile_read(cavs_session *s, const char *kernel_class, double *total_ms, double *launches) {
  if (int rc = need(s, "session")) return rc;
  if (int rc = need(total_ms, "output")) return rc;
  if (int rc = need(launches, "output")) return rc;
  static const char *names[] = {"gemm", "gather", "scatter", "gates", "other", "round"};
  int cls = -1;
  for (int i = 0; i < 6; i++)
    if (kernel_class && !std::strcmp(kernel_class, names[i])) cls = i;
  if (cls < 0) {
    g_error = "unknown kernel class";
    return CAVS_EINVAL;
  }
  return guarded([&] { s->engine.profile_read(cls, total_ms, launches); });
}

void *cavs_session_stream(cavs_session *s) { return s ? s->engine.stream() : nullptr; }

int cavs_session_counter(cavs_session *s, const char *key, double *value) {
  if (int rc = need(s, "session")) return rc;
  if (int rc = need(value, "output")) return rc;
  return guarded([&] { *value = s->engine.counter(key ? key : ""); });
}

}  // extern "C"
