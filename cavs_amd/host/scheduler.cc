#include "scheduler.h"

#include <algorithm>

namespace cavs {

// LoadGraph, cavs/midend/graph_scheduler.cc:12-71.
static std::string load_graph(const int32_t *g, int B, int maxlen, Schedule *s) {
  s->B = B;
  s->maxlen = maxlen;
  s->sample_offset.assign(B, 0);
  s->parent.clear();
  int off = 0;
  for (int i = 0; i < B; i++) {
    const int32_t *row = g + (size_t)i * maxlen;
    int k = 0;
    while (k < maxlen && row[k] != -1) k++;
    if (k == maxlen) return "sample " + std::to_string(i) + " has no -1 terminator within maxlen";
    int len = k + 1;
    s->sample_offset[i] = off;
    for (int j = 0; j < len - 1; j++) {
      if (row[j] < 0 || row[j] >= len)
        return "sample " + std::to_string(i) + ": parent id out of range at vertex " + std::to_string(j);
      s->parent.push_back(off + row[j]);
    }
    s->parent.push_back(-1);
    off += len;
  }
  const int N = s->N = off;
  // children in ascending vertex id (graph_scheduler.cc:52-58 appends in vertex order)
  s->child_begin.assign(N + 1, 0);
  for (int v = 0; v < N; v++)
    if (s->parent[v] >= 0) s->child_begin[s->parent[v] + 1]++;
  for (int v = 0; v < N; v++) s->child_begin[v + 1] += s->child_begin[v];
  s->child.assign(s->child_begin[N], 0);
  std::vector<int> fill(s->child_begin.begin(), s->child_begin.end() - 1);
  for (int v = 0; v < N; v++)
    if (s->parent[v] >= 0) s->child[fill[s->parent[v]]++] = v;
  return "";
}

static inline int nchild(const Schedule &s, int v) { return s.child_begin[v + 1] - s.child_begin[v]; }

// BatchGraphScheduler::Initialize / ActivateNext, forward branch
// (cavs/midend/graph_scheduler.cc:169-193, 202-245).
static void batch_rounds(Schedule *s) {
  const int N = s->N;
  s->tids_to_jobids.assign(N, 0);
  s->jobids_to_tids.assign(N, 0);
  s->round2offset.assign(1, 0);
  std::vector<int> activated(N, 0);
  int begin = 0, end = 0;  // current round = tids [begin, end)
  for (int v = 0; v < N; v++)
    if (nchild(*s, v) == 0 && s->parent[v] >= 0) {
      s->tids_to_jobids[end] = v;
      s->jobids_to_tids[v] = end;
      end++;
    }
  s->leaf_prefix = end;
  while (end > begin) {
    Round r;
    r.offset = begin;
    r.n = end - begin;
    // lists this round exposes: gather lists were appended while the round was being
    // formed (below); the scatter list holds the non-root jobs in job order
    for (int c = 0; c < 2; c++) r.gather_end[c] = (int)s->gather_ids[c].size();
    r.scatter_begin = (int)s->scatter_ids.size();
    for (int t = begin; t < end; t++)
      if (s->parent[s->tids_to_jobids[t]] >= 0) s->scatter_ids.push_back(t);
    r.scatter_end = (int)s->scatter_ids.size();
    for (int c = 0; c < 2; c++)
      r.gather_begin[c] = s->rounds.empty() ? r.gather_end[c] : s->rounds.back().gather_end[c];
    s->rounds.push_back(r);
    s->max_round = std::max(s->max_round, r.n);
    s->round2offset.push_back(end);
    int next = end;
    for (int t = begin; t < end; t++) {
      int p = s->parent[s->tids_to_jobids[t]];
      if (p < 0) continue;
      if (++activated[p] == nchild(*s, p)) {
        s->tids_to_jobids[next] = p;
        s->jobids_to_tids[p] = next;
        for (int i = 0; i < nchild(*s, p) && i < 2; i++)
          s->gather_ids[i].push_back(s->jobids_to_tids[s->child[s->child_begin[p] + i]]);
        if (s->parent[p] < 0) s->root_tids.push_back(next);
        next++;
      }
    }
    begin = end;
    end = next;
  }
  s->executed = end;
  for (int k = (int)s->rounds.size() - 1; k >= 0; k--) s->bwd_rounds.push_back(k);
}

// SerialGraphScheduler (cavs/midend/graph_scheduler.cc:83-167): one vertex per round,
// tensor id == vertex id, samples one after the other, FIFO activation order.
static void serial_rounds(Schedule *s) {
  const int N = s->N;
  s->tids_to_jobids.assign(N, 0);
  s->jobids_to_tids.assign(N, 0);
  for (int v = 0; v < N; v++) s->tids_to_jobids[v] = s->jobids_to_tids[v] = v;
  std::vector<int> activated(N, 0), fifo;
  fifo.reserve(N);
  for (int i = 0; i < s->B; i++) {
    int lo = s->sample_offset[i], hi = i + 1 < s->B ? s->sample_offset[i + 1] : N;
    size_t head = fifo.size();
    for (int v = lo; v < hi; v++)
      if (nchild(*s, v) == 0 && s->parent[v] >= 0) fifo.push_back(v);
    for (; head < fifo.size(); head++) {
      int v = fifo[head], p = s->parent[v];
      if (p >= 0 && ++activated[p] == nchild(*s, p)) fifo.push_back(p);
    }
  }
  for (int v : fifo) {
    Round r;
    r.offset = v;
    r.n = 1;
    for (int c = 0; c < 2; c++) {
      r.gather_begin[c] = (int)s->gather_ids[c].size();
      if (nchild(*s, v) > c) s->gather_ids[c].push_back(s->child[s->child_begin[v] + c]);
      r.gather_end[c] = (int)s->gather_ids[c].size();
    }
    r.scatter_begin = (int)s->scatter_ids.size();
    if (s->parent[v] >= 0) s->scatter_ids.push_back(v); else s->root_tids.push_back(v);
    r.scatter_end = (int)s->scatter_ids.size();
    s->rounds.push_back(r);
  }
  s->executed = (int)fifo.size();
  s->max_round = fifo.empty() ? 0 : 1;
  s->leaf_prefix = 0;
  // Backward order (ReverseGraph + the same FIFO, graph_scheduler.cc:73-81,110-140): roots
  // first, children after their parent.  The reference starts the next sample whenever
  // the vertex it pops has no forward children, i.e. at every leaf, not only at the end
  // of a sample; the order below reproduces that.
  std::vector<int> round_of(N, -1);
  for (size_t k = 0; k < s->rounds.size(); k++) round_of[s->rounds[k].offset] = (int)k;
  std::vector<int> bf;
  bf.reserve(N);
  auto init_sample = [&](int i) {
    int lo = s->sample_offset[i], hi = i + 1 < s->B ? s->sample_offset[i + 1] : N;
    for (int v = lo; v < hi; v++)
      if (s->parent[v] < 0 && nchild(*s, v) > 0) bf.push_back(v);
  };
  int sample_id = 0;
  init_sample(0);
  for (size_t head = 0; head < bf.size(); head++) {
    int v = bf[head];
    if (nchild(*s, v) > 0) {
      for (int k = s->child_begin[v]; k < s->child_begin[v + 1]; k++) bf.push_back(s->child[k]);
    } else if (++sample_id < s->B) {
      init_sample(sample_id);
    }
  }
  for (int v : bf) s->bwd_rounds.push_back(round_of[v]);
}

std::string build_schedule(const int32_t *graph, int B, int maxlen, bool batching, Schedule *out) {
  *out = Schedule();
  out->batching = batching;
  if (!graph || B <= 0 || maxlen <= 0) return "empty graph feed";
  std::string err = load_graph(graph, B, maxlen, out);
  if (!err.empty()) return err;
  for (int v = 0; v < out->N; v++)
    if (nchild(*out, v) > 2)
      return "vertex " + std::to_string(v) + " has " + std::to_string(nchild(*out, v)) +
             " children; the scheduler's gather lists hold two (graph_scheduler.h:16-18)";
  if (batching) batch_rounds(out); else serial_rounds(out);
  if (out->executed != out->N) {
    // A sample of a single vertex is never executed (graph_scheduler.cc:180); the schedule of the
    // rest stands, and it is the caller's business whether it accepts such a batch.  Any other
    // vertex that did not run sits on a parent cycle.
    int singles = 0;
    for (int i = 0; i < B; i++) {
      const int hi = i + 1 < B ? out->sample_offset[i + 1] : out->N;
      if (hi - out->sample_offset[i] == 1) singles++;
    }
    if (out->executed + singles != out->N)
      return std::to_string(out->N - out->executed - singles) + " vertices never become ready: the parent array holds a cycle "
             "(a vertex that is its own ancestor)";
  }
  return "";
}

std::string build_index_lists(const Schedule &s, int nch, int pairing, int *t2j, int *pair, int *child, int *roots) {
  const int N = s.N;
  std::copy(s.tids_to_jobids.begin(), s.tids_to_jobids.end(), t2j);
  std::fill(pair, pair + N, -1);
  std::fill(child, child + (size_t)nch * N, -1);
  for (const Round &r : s.rounds) {
    const int m = r.scatter_end - r.scatter_begin;
    if (pairing == 0) {
      for (int b = 0; b < m; b++) pair[r.offset + b] = s.scatter_ids[r.scatter_begin + b];
    } else {
      for (int b = 0; b < m; b++) pair[s.scatter_ids[r.scatter_begin + b]] = s.scatter_ids[r.scatter_begin + b];
    }
    if (r.gather_begin[0] == r.gather_end[0] && r.gather_begin[1] == r.gather_end[1]) continue;  // a round of leaves
    for (int c = 0; c < nch; c++) {
      const int len = r.gather_end[c] - r.gather_begin[c];
      if (len != r.n)
        return "round at tensor id " + std::to_string(r.offset) + " mixes vertices with and without child " + std::to_string(c) +
               " (the reference's gather lists misalign there too)";
      for (int b = 0; b < len; b++) child[(size_t)nch * (r.offset + b) + c] = s.gather_ids[c][r.gather_begin[c] + b];
    }
    if (nch == 1 && r.gather_end[1] != r.gather_begin[1]) return "a chain vertex function got a vertex with two children";
  }
  int nr = 0;
  for (int v = 0; v < N; v++)
    if (s.parent[v] < 0) roots[nr++] = v;
  return "";
}

bool build_forest_lists(const Schedule &s, int nch, int fused_limit, const int *pair, const int *child, int *kid_rows,
                        int *orphans, int *n_orphans) {
  const int N = s.N;
  *n_orphans = 0;
  auto leaf_round = [](const Round &r) { return r.gather_begin[0] == r.gather_end[0] && r.gather_begin[1] == r.gather_end[1]; };
  if (!s.batching || s.rounds.empty() || !leaf_round(s.rounds[0]) || s.rounds[0].n != s.leaf_prefix) return false;
  std::vector<int> inv_pair(N, -1), round_of_row(N);
  for (size_t k = 0; k < s.rounds.size(); k++) {
    const Round &r = s.rounds[k];
    if (k > 0 && (leaf_round(r) || r.n > fused_limit)) return false;  // every round with children runs as a fused launch
    for (int b = 0; b < r.n; b++) round_of_row[r.offset + b] = (int)k;
  }
  for (int v = 0; v < N; v++) {
    const int p = pair[v];
    if (p < 0) continue;
    if (p >= N || inv_pair[p] >= 0) return false;  // two writers of one pool row
    inv_pair[p] = v;
  }
  std::vector<char> read(N, 0);
  for (size_t i = 0; i < (size_t)nch * N; i++) {
    kid_rows[i] = -1;
    const int p = child[i];
    if (p < 0) continue;
    const int b = (int)(i / nch);
    if (p >= N || inv_pair[p] < 0 || read[p]) return false;  // reads a row nobody wrote, or a second reader
    const int v = inv_pair[p];
    if (round_of_row[v] >= round_of_row[b]) return false;
    read[p] = 1;
    kid_rows[i] = v;
  }
  for (int v = 0; v < N; v++) {
    if (pair[v] >= 0 && !read[pair[v]]) return false;  // a message nobody reads: its gradient is whatever the pool holds
    if (pair[v] < 0) orphans[(*n_orphans)++] = v;
  }
  return true;
}

// Which rounds run inside the tail launches, and who runs which row.  The rounds are a suffix of the
// forward order (a prefix of the backward order).  Inside it the message flow is a forest over slab
// rows (kid_rows: the rows whose messages a row consumes); a tree of that forest goes to one group
// as a whole, so nothing a group reads is written by another during the launch.  Trees are dealt
// heaviest first to the group with the fewest rows so far; the suffix starts at the earliest round
// from which no group gets more rows of a round than `lim`, nor more lists than `max_lists`.
void build_tail_lists(const Schedule &s, const int *kid_rows, int lim, int groups, int max_lists, int slice, TailLists *out,
                      int *rows_out) {
  *out = TailLists();
  const int R = (int)s.rounds.size(), N = s.N, G = groups, cap = max_lists;
  auto leaf_round = [](const Round &r) { return r.gather_begin[0] == r.gather_end[0] && r.gather_begin[1] == r.gather_end[1]; };
  if (lim <= 0 || G < 1 || G > 16 || slice < 1 || !s.batching || R < 3) return;
  int k0 = 1;
  while (k0 < R && (s.rounds[k0].n > G * lim || leaf_round(s.rounds[k0]))) k0++;
  std::vector<int> comp, weight, group, order, per;
  for (; R - k0 >= 2; k0++) {
    bool ok = true;
    for (int k = k0; k < R && ok; k++) ok = !leaf_round(s.rounds[k]);
    if (!ok) continue;
    const int lo = s.rounds[k0].offset;
    comp.assign(N - lo, -1);
    weight.clear();
    for (int v = N - 1; v >= lo; v--) {  // a row's consumer sits in a later round: parents come first
      if (comp[v - lo] < 0) {
        comp[v - lo] = (int)weight.size();
        weight.push_back(0);
      }
      weight[comp[v - lo]]++;
      for (int i = 0; i < 2; i++) {
        const int c = kid_rows[2 * (size_t)v + i];
        if (c >= lo) comp[c - lo] = comp[v - lo];
      }
    }
    order.resize(weight.size());
    for (size_t i = 0; i < order.size(); i++) order[i] = (int)i;
    std::stable_sort(order.begin(), order.end(), [&](int a, int b) { return weight[a] > weight[b]; });
    group.assign(weight.size(), 0);
    int load[16] = {0};
    for (int c : order) {
      int best = 0;
      for (int g = 1; g < G; g++)
        if (load[g] < load[best]) best = g;
      group[c] = best;
      load[best] += weight[c];
    }
    // rows of round k that group g runs, and the lists that makes
    const int nr = R - k0;
    per.assign((size_t)G * nr, 0);
    for (int k = k0; k < R; k++)
      for (int b = s.rounds[k].offset; b < s.rounds[k].offset + s.rounds[k].n; b++) per[(size_t)group[comp[b - lo]] * nr + (k - k0)]++;
    int lists = 0;
    for (int g = 0; g < G && ok; g++) {
      int mine = 0;
      for (int k = 0; k < nr; k++) {
        if (per[(size_t)g * nr + k] > lim) ok = false;
        mine += (per[(size_t)g * nr + k] + slice - 1) / slice;
      }
      if (mine > cap) ok = false;
      lists = std::max(lists, mine);
    }
    if (!ok) continue;
    TailLists &t = *out;
    t.first = k0;
    t.max_rounds = std::max(lists, 1);
    const size_t M = t.max_rounds;
    t.nrounds.assign(G, 0);
    for (auto *v : {&t.start, &t.count, &t.flags, &t.bstart, &t.bcount, &t.bflags}) v->assign((size_t)G * M, 0);
    // the device list: group by group, round by round
    std::vector<int> at((size_t)G * nr, -1);
    size_t fill = 0;
    for (int g = 0; g < G; g++)
      for (int k = 0; k < nr; k++) {
        at[(size_t)g * nr + k] = (int)fill;
        fill += per[(size_t)g * nr + k];
      }
    {
      std::vector<int> cur(at);
      for (int k = k0; k < R; k++)
        for (int b = s.rounds[k].offset; b < s.rounds[k].offset + s.rounds[k].n; b++) rows_out[cur[(size_t)group[comp[b - lo]] * nr + (k - k0)]++] = b;
    }
    // A group's share of a round as lists of at most `slice` rows: the first waits for the rounds the
    // group has done so far, the last is an arrival.  Forward: rounds in order; backward: reversed.
    for (int g = 0; g < G; g++) {
      int tiles = 0;
      for (int dir = 0; dir < 2; dir++) {
        std::vector<int> &st = dir ? t.bstart : t.start, &ct = dir ? t.bcount : t.count, &fl = dir ? t.bflags : t.flags;
        int i = 0, done = 0;
        for (int kk = 0; kk < nr; kk++) {
          const int k = dir ? nr - 1 - kk : kk, c = per[(size_t)g * nr + k];
          for (int c0 = 0; c0 < c; c0 += slice, i++) {
            st[g * M + i] = at[(size_t)g * nr + k] + c0;
            ct[g * M + i] = std::min(slice, c - c0);
            fl[g * M + i] = ((c0 == 0 ? done : 0) << 1) | (c0 + slice >= c ? 1 : 0);
            if (!dir) tiles += (ct[g * M + i] + 3) / 4;
          }
          done += c > 0;
        }
        t.nrounds[g] = i;
      }
      t.tiles_max = std::max(t.tiles_max, tiles);
      t.lists_max = std::max(t.lists_max, t.nrounds[g]);
    }
    t.rows = fill;
    return;
  }
}

void schedule_from_lists(int B, int maxlen, int N, int nch, const int *round2offset, int R, const int *t2j,
                         const int *pair, const int *child, const int *roots, Schedule *out) {
  *out = Schedule();
  Schedule &s = *out;
  s.B = B;
  s.maxlen = maxlen;
  s.N = N;
  s.batching = true;
  s.tids_to_jobids.assign(t2j, t2j + N);
  s.jobids_to_tids.assign(N, 0);
  for (int t = 0; t < N; t++) s.jobids_to_tids[t2j[t]] = t;
  s.round2offset.assign(round2offset, round2offset + R + 1);
  std::vector<char> is_root(N, 0);
  for (int i = 0; i < B; i++) is_root[roots[i]] = 1;
  // sample offsets and parents follow from the roots (each sample ends at its root) and the child lists
  s.sample_offset.assign(B, 0);
  for (int i = 1; i < B; i++) s.sample_offset[i] = roots[i - 1] + 1;
  s.parent.assign(N, -1);
  for (int r = 0; r < R; r++) {
    Round rd;
    rd.offset = round2offset[r];
    rd.n = round2offset[r + 1] - round2offset[r];
    for (int c = 0; c < 2; c++) rd.gather_begin[c] = (int)s.gather_ids[c].size();
    rd.scatter_begin = (int)s.scatter_ids.size();
    for (int b = 0; b < rd.n; b++) {
      const int t = rd.offset + b;
      for (int c = 0; c < nch; c++) {
        const int p = child[(size_t)nch * t + c];
        if (p < 0) continue;
        s.gather_ids[c].push_back(p);
        s.parent[t2j[p]] = t2j[t];
      }
      // the scatter list is the round's non-root jobs in job order under either pairing
      if (!is_root[t2j[t]]) s.scatter_ids.push_back(t); else s.root_tids.push_back(t);
    }
    for (int c = 0; c < 2; c++) rd.gather_end[c] = (int)s.gather_ids[c].size();
    rd.scatter_end = (int)s.scatter_ids.size();
    s.rounds.push_back(rd);
    s.max_round = std::max(s.max_round, rd.n);
  }
  (void)pair;
  s.executed = N;
  s.leaf_prefix = R > 0 ? round2offset[1] : 0;
  for (int k = R - 1; k >= 0; k--) s.bwd_rounds.push_back(k);
  // children in ascending vertex id, as LoadGraph builds them
  s.child_begin.assign(N + 1, 0);
  for (int v = 0; v < N; v++)
    if (s.parent[v] >= 0) s.child_begin[s.parent[v] + 1]++;
  for (int v = 0; v < N; v++) s.child_begin[v + 1] += s.child_begin[v];
  s.child.assign(s.child_begin[N], 0);
  std::vector<int> fill(s.child_begin.begin(), s.child_begin.end() - 1);
  for (int v = 0; v < N; v++)
    if (s.parent[v] >= 0) s.child[fill[s.parent[v]]++] = v;
}

// trace_format: [N, R_fwd, R_bwd, then per round: offset, n_exec, exec..., n_g0, g0...,
// n_g1, g1..., n_s0, s0..., n_s1, s1..., n_init, init..., then tids_to_jobids (N),
// n_r2o, round2offset...].  Backward rounds are the forward rounds last to first with
// gather := recorded scatter lists and scatter := recorded gather lists
// (cavs/midend/graph_scheduler.cc:194-199, 246-257).
std::vector<int> Schedule::trace(bool with_backward) const {
  std::vector<int> o;
  auto put_list = [&](const int *p, int n) {
    o.push_back(n);
    o.insert(o.end(), p, p + n);
  };
  const int R = (int)rounds.size();
  o.push_back(N);
  o.push_back(R);
  o.push_back(with_backward ? (int)bwd_rounds.size() : 0);
  // forward gather_init list: the leaves of round 0 (batch) / the current leaf (serial)
  std::vector<int> init_fwd;
  if (batching && R) init_fwd.assign(tids_to_jobids.begin(), tids_to_jobids.begin() + rounds[0].n);
  for (int k = 0; k < R; k++) {
    const Round &r = rounds[k];
    o.push_back(r.offset);
    if (batching) put_list(&tids_to_jobids[r.offset], r.n); else put_list(&r.offset, 1);
    for (int c = 0; c < 2; c++) put_list(gather_ids[c].data() + r.gather_begin[c], r.gather_end[c] - r.gather_begin[c]);
    put_list(scatter_ids.data() + r.scatter_begin, r.scatter_end - r.scatter_begin);
    o.push_back(0);
    if (!batching && r.gather_end[0] == r.gather_begin[0]) init_fwd.assign(1, r.offset);
    put_list(init_fwd.data(), (int)init_fwd.size());
  }
  if (with_backward) {
    std::vector<int> init_bwd = batching ? root_tids : std::vector<int>();
    bool first = true;
    for (int k : bwd_rounds) {
      const Round &r = rounds[k];
      o.push_back(r.offset);
      if (batching) put_list(&tids_to_jobids[r.offset], r.n); else put_list(&r.offset, 1);
      if (batching) {
        put_list(scatter_ids.data() + r.scatter_begin, r.scatter_end - r.scatter_begin);
        o.push_back(0);
      } else {
        // serial backward: the gather list is one copy of the vertex per forward parent
        // (graph_scheduler.cc:158-161); the first round is set up by Initialize, which
        // fills no gather list (:100-107)
        int v = r.offset;
        int has_parent = parent[v] >= 0;
        if (first) o.push_back(0); else put_list(&v, has_parent);
        o.push_back(0);
        if (!has_parent) init_bwd.assign(1, v);
      }
      for (int c = 0; c < 2; c++) put_list(gather_ids[c].data() + r.gather_begin[c], r.gather_end[c] - r.gather_begin[c]);
      put_list(init_bwd.data(), (int)init_bwd.size());
      first = false;
    }
  }
  o.insert(o.end(), tids_to_jobids.begin(), tids_to_jobids.end());
  put_list(round2offset.data(), (int)round2offset.size());
  return o;
}

}  // namespace cavs
