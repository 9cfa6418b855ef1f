// Level-wise ready frontier on the GPU: reproduces the round structure and the
// within-round order of the host batch scheduler from the global parent array.
//
// One workgroup walks the rounds.  A vertex joins round r+1 when its last child
// (in the order the current round executes) fires; "last" is decided per job
// without counters: job v activates its parent p iff every sibling of v has
// already run, and no sibling runs later than v in the same round.  The jobs that
// activate a parent are compacted in order with a block-wide prefix sum, which
// gives exactly the sequential append order of the host loop.  Every wave reaches
// the loop exit because the round counter is uniform across the workgroup.
#include "common.h"

namespace cavs {

constexpr int kSchedThreads = 1024;

__global__ void sched_init_kernel(int N, int *__restrict__ nchild, int *__restrict__ cmin,
                                  int *__restrict__ cmax, int *__restrict__ level, int *__restrict__ t2j,
                                  int *__restrict__ j2t) {
  int v = blockIdx.x * blockDim.x + threadIdx.x;
  if (v >= N) return;
  nchild[v] = 0;
  cmin[v] = 0x7fffffff;
  cmax[v] = -1;
  level[v] = -1;
  t2j[v] = 0;  // slots of vertices that never run read 0, as in the host scheduler
  j2t[v] = 0;
}

__global__ void sched_children_kernel(const int *__restrict__ parent, int N, int *__restrict__ nchild,
                                      int *__restrict__ cmin, int *__restrict__ cmax) {
  int v = blockIdx.x * blockDim.x + threadIdx.x;
  if (v >= N) return;
  int p = parent[v];
  if (p >= 0) {
    atomicAdd(nchild + p, 1);
    atomicMin(cmin + p, v);
    atomicMax(cmax + p, v);
  }
}

// inclusive scan of one int per thread over the workgroup; returns the exclusive
// prefix and (through total) the workgroup sum
__device__ inline int block_excl_scan(int x, int *lds, int *total) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
  int incl = x;
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) {
    int y = __shfl_up(incl, o, 64);
    if (lane >= o) incl += y;
  }
  if (lane == 63) lds[wave] = incl;
  __syncthreads();
  if (wave == 0) {
    int w = lane < nw ? lds[lane] : 0;
    int wi = w;
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
      int y = __shfl_up(wi, o, 64);
      if (lane >= o) wi += y;
    }
    if (lane < nw) lds[64 + lane] = wi - w;  // exclusive wave prefix
    if (lane == 63) lds[128] = wi;
  }
  __syncthreads();
  int res = lds[64 + wave] + incl - x;
  *total = lds[128];
  __syncthreads();
  return res;
}

__global__ __launch_bounds__(kSchedThreads) void sched_frontier_kernel(
    const int *__restrict__ parent, int N, const int *__restrict__ nchild,
    const int *__restrict__ cmin, const int *__restrict__ cmax, int *__restrict__ t2j,
    int *__restrict__ j2t, int *__restrict__ level /* round of vertex, -1 = not run */,
    int *__restrict__ round_of_tid, int *__restrict__ round2offset, int *__restrict__ n_rounds) {
  __shared__ int lds[129];
  const int tid = threadIdx.x;
  // the two gather lists hold two children (cavs/midend/graph_scheduler.h:16-18): a vertex with
  // more is refused (n_rounds = -1) instead of being scheduled twice
  int many = 0;
  for (int v = tid; v < N; v += kSchedThreads) many |= nchild[v] > 2;
  if (__syncthreads_or(many)) {
    if (tid == 0) *n_rounds = -1;
    return;
  }
  // round 0: leaves that have a parent, ascending vertex id
  int count = 0;
  for (int base = 0; base < N; base += kSchedThreads) {
    int v = base + tid;
    int flag = (v < N && nchild[v] == 0 && parent[v] >= 0) ? 1 : 0;
    int tot;
    int pos = block_excl_scan(flag, lds, &tot);
    if (flag) {
      int t = count + pos;
      t2j[t] = v;
      j2t[v] = t;
      level[v] = 0;
      round_of_tid[t] = 0;
    }
    count += tot;
  }
  if (tid == 0) round2offset[0] = 0;
  int off = 0, ncur = count, r = 0;
  __threadfence_block();
  __syncthreads();
  while (ncur > 0) {  // ncur is uniform over the workgroup
    int next = 0;
    const int noff = off + ncur;
    for (int base = 0; base < ncur; base += kSchedThreads) {
      int b = base + tid;
      int flag = 0, p = -1;
      if (b < ncur) {
        int v = t2j[off + b];
        p = parent[v];
        if (p >= 0) {
          if (nchild[p] == 1) {
            flag = 1;
          } else {
            int s = cmin[p] == v ? cmax[p] : cmin[p];
            int ls = level[s];
            flag = (ls >= 0 && (ls < r || j2t[s] < off + b)) ? 1 : 0;
          }
        }
      }
      int tot;
      int pos = block_excl_scan(flag, lds, &tot);
      if (flag && noff + next + pos < N) {  // (a vertex with >2 children could be flagged twice)
        int t = noff + next + pos;
        t2j[t] = p;
        j2t[p] = t;
        round_of_tid[t] = r + 1;
      }
      next += tot;
    }
    __syncthreads();
    // publish the levels of the new round only after every job of this round was tested
    if (noff + next > N) next = N - noff;
    for (int b = tid; b < next; b += kSchedThreads) level[t2j[noff + b]] = r + 1;
    r++;
    if (tid == 0) round2offset[r] = noff;
    off = noff;
    ncur = next;
    __threadfence_block();
    __syncthreads();
  }
  if (tid == 0) *n_rounds = r;
}

// ------------------------------------------------------------------ the whole index arena
// The schedule of a batch is the schedules of its samples merged: round 0 lists the leaves in
// ascending vertex id, i.e. sample by sample, and a vertex joins the next round at the moment its
// last child fires, so by induction every round lists its vertices sample by sample, each
// sample's in the order its own frontier produces them.  Hence
//   tensor id(v) = round2offset[r] + (vertices of earlier samples in round r) + (position of v
//                  among its sample's vertices of round r),
// and the work splits into three launches that never need a grid-wide barrier:
//   1. one wavefront per sample walks that sample's ready frontier in LDS (arena_sample_kernel);
//   2. per round, a prefix sum over the samples' counts (arena_round_kernel), then one over the
//      rounds (arena_offsets_kernel);
//   3. one wavefront per sample writes its vertices' entries of every list (arena_lists_kernel).
// Lists (each `cap` ints apart unless noted; cap >= B * maxlen):
//   t2j   [N]       tensor id -> global vertex id
//   pair  [N]       per slab row: the pool row its message is scattered to / gathered back from, or -1
//                   (reference pairing: b-th entry of the round's compacted list of non-roots with
//                   the b-th slab row; row-id pairing: the row itself)
//   child [nch*N]   per slab row and child slot: pool row of that child (-1 for leaves)
//   kid   [nch*N]   per slab row and child slot: slab row whose message that child's pool row holds
//   roots [B]       vertex ids of the roots;  orph [B]: the slab rows with pair < 0, ascending
// meta (maxlen + 9 ints): [0] N, [1] R, [2] error bits, [3] largest round, [8 + r] round2offset[r], r <= R.
enum { kErrNoEnd = 1, kErrRange = 2, kErrArity = 4, kErrSingle = 8, kErrCycle = 16 };

struct ArenaArgs {
  const int *graph;  // [B, maxlen] local parent ids, first -1 ends the sample
  int B, maxlen, nch, pairing;
  long cap;
  // per-sample scratch, [B, maxlen] each
  int *ord, *rnd, *c0, *c1, *cnt, *rst, *bs, *rb;
  int *len, *depth, *soff;       // [B]
  int *total, *nroots, *rsb;     // [maxlen] vertices / roots of round r, roots of earlier rounds
  int *meta;
  int *t2j, *pair, *child, *kid, *roots, *orph;
};

__device__ inline int lanes_before(unsigned long long mask, int lane) {
  return __popcll(mask & ((1ull << lane) - 1ull));
}

__global__ __launch_bounds__(256) void arena_clear_kernel(ArenaArgs a) {
  const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < a.cap) {
    a.t2j[i] = 0;
    a.pair[i] = -1;
  }
  if (i < a.cap * a.nch) {
    a.child[i] = -1;
    a.kid[i] = -1;
  }
  if (i < a.maxlen) a.total[i] = 0;
  if (i < 8) a.meta[i] = 0;
}

// One wavefront per sample: LoadGraph for the sample (length, children in ascending id) and its
// ready frontier, round by round.  LDS: par, nchild, c0, c1, pos, ord -- six ints per vertex.
__global__ __launch_bounds__(64) void arena_sample_kernel(ArenaArgs a) {
  extern __shared__ int lds[];
  const int s = blockIdx.x, lane = threadIdx.x, ML = a.maxlen;
  int *par = lds, *nchild = lds + ML, *c0 = lds + 2 * ML, *c1 = lds + 3 * ML, *pos = lds + 4 * ML, *ord = lds + 5 * ML;
  const int *row = a.graph + (long)s * ML;
  int err = 0;
  // the sample ends at its first -1 (cavs/midend/graph_scheduler.cc:39)
  int first = ML;
  for (int j = lane; j < ML; j += 64) {
    const int p = row[j];
    par[j] = p;
    if (p == -1 && j < first) first = j;
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) first = min(first, __shfl_xor(first, o, 64));
  int L = first + 1;
  if (first == ML) {
    err |= kErrNoEnd;
    L = 0;
  }
  for (int v = lane; v < ML; v += 64) {
    nchild[v] = 0;
    c0[v] = 0x7fffffff;
    c1[v] = -1;
    pos[v] = -1;
  }
  __syncthreads();
  for (int v = lane; v < L - 1; v += 64) {
    const int p = par[v];
    if (p < 0 || p >= L) {
      err |= kErrRange;
      par[v] = -1;  // (keeps the walk inside the sample; the batch is rejected anyway)
      continue;
    }
    atomicAdd(&nchild[p], 1);
    atomicMin(&c0[p], v);
    atomicMax(&c1[p], v);
  }
  __syncthreads();
  for (int v = lane; v < L; v += 64)
    if (nchild[v] != 0 && nchild[v] != a.nch) err |= kErrArity;
  if (L == 1) err |= kErrSingle;
  // round 0: the childless vertices that have a parent, ascending
  // (BatchGraphScheduler::Initialize, cavs/midend/graph_scheduler.cc:176-186)
  int *g_ord = a.ord + (long)s * ML, *g_rnd = a.rnd + (long)s * ML, *g_cnt = a.cnt + (long)s * ML, *g_rst = a.rst + (long)s * ML;
  int count = 0;
  for (int base = 0; base < L; base += 64) {
    const int v = base + lane;
    const bool f = v < L && nchild[v] == 0 && par[v] >= 0;
    const unsigned long long m = __ballot(f);
    if (f) {
      const int k = count + lanes_before(m, lane);
      ord[k] = v;
      pos[v] = k;
      g_ord[k] = v;
      g_rnd[k] = 0;
    }
    count += __popcll(m);
  }
  __syncthreads();
  // ActivateNext (cavs/midend/graph_scheduler.cc:202-236): job b of the round activates its parent
  // iff every sibling ran before it -- in an earlier round or earlier in this one, i.e. at a smaller
  // position of the execution order; the activating jobs, compacted in order, are the next round
  int off = 0, ncur = count, r = 0;
  while (ncur > 0) {  // uniform over the wavefront
    if (lane == 0) {
      g_cnt[r] = ncur;
      g_rst[r] = off;
    }
    const int noff = off + ncur;
    int next = 0;
    for (int base = 0; base < ncur; base += 64) {
      const int b = base + lane;
      bool f = false;
      int p = -1;
      if (b < ncur) {
        const int v = ord[off + b];
        p = par[v];
        if (p >= 0) {
          if (nchild[p] <= 1) {
            f = true;
          } else {
            const int sib = c0[p] == v ? c1[p] : c0[p];
            const int ps = pos[sib];
            f = ps >= 0 && ps < off + b;
          }
        }
      }
      const unsigned long long m = __ballot(f);
      const int k = noff + next + lanes_before(m, lane);
      if (f && k < L) {  // (k >= L only on a malformed sample, which is rejected)
        ord[k] = p;
        pos[p] = k;
        g_ord[k] = p;
        g_rnd[k] = r + 1;
      }
      next += __popcll(m);
    }
    __syncthreads();
    off = noff;
    ncur = min(next, L - noff);
    r++;
  }
  if (off != L && L > 1) err |= kErrCycle;  // vertices on a parent cycle never become ready
  for (int q = r + lane; q < ML; q += 64) {
    g_cnt[q] = 0;
    g_rst[q] = off;
  }
  for (int v = lane; v < ML; v += 64) {
    a.c0[(long)s * ML + v] = c0[v];
    a.c1[(long)s * ML + v] = c1[v];
  }
  if (lane == 0) {
    a.len[s] = L;
    a.depth[s] = r;
  }
  if (err) atomicOr(a.meta + 2, err);
}

// One workgroup per round r: over the samples in order, the vertices (bs) and the roots (rb) that
// precede each sample's block of the round.  A sample's root is the only vertex of its last round.
__global__ __launch_bounds__(256) void arena_round_kernel(ArenaArgs a) {
  __shared__ int lds[129];
  const int r = blockIdx.x, tid = threadIdx.x, ML = a.maxlen;
  int run = 0, runr = 0;
  for (int base = 0; base < a.B; base += 256) {
    const int s = base + tid;
    const int c = s < a.B ? a.cnt[(long)s * ML + r] : 0;
    const int isroot = (s < a.B && a.depth[s] - 1 == r) ? 1 : 0;
    int tot, totr;
    const int e = block_excl_scan(c, lds, &tot);
    const int er = block_excl_scan(isroot, lds, &totr);
    if (s < a.B) {
      a.bs[(long)s * ML + r] = run + e;
      a.rb[(long)s * ML + r] = runr + er;
    }
    run += tot;
    runr += totr;
  }
  if (tid == 0) {
    a.total[r] = run;
    a.nroots[r] = runr;
  }
}

// One workgroup: round2offset, N, R; the samples' vertex offsets; roots of earlier rounds.
__global__ __launch_bounds__(1024) void arena_offsets_kernel(ArenaArgs a) {
  __shared__ int lds[129];
  const int tid = threadIdx.x;
  int run = 0, runr = 0, R = 0;
  for (int base = 0; base < a.maxlen; base += 1024) {
    const int r = base + tid;
    const int c = r < a.maxlen ? a.total[r] : 0, nr = r < a.maxlen ? a.nroots[r] : 0;
    int tot, totr, cntr;
    const int e = block_excl_scan(c, lds, &tot);
    const int er = block_excl_scan(nr, lds, &totr);
    block_excl_scan(c > 0 ? 1 : 0, lds, &cntr);
    if (r < a.maxlen) {
      a.meta[8 + r] = run + e;
      a.rsb[r] = runr + er;
    }
    int m = c;
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) m = max(m, __shfl_xor(m, o, 64));
    if ((tid & 63) == 0 && m > 0) atomicMax(a.meta + 3, m);
    run += tot;
    runr += totr;
    R += cntr;
  }
  __syncthreads();
  if (tid == 0) {
    a.meta[0] = run;
    a.meta[1] = R;
    a.meta[8 + a.maxlen] = run;
  }
  run = 0;
  for (int base = 0; base < a.B; base += 1024) {
    const int s = base + tid;
    const int c = s < a.B ? a.len[s] : 0;
    int tot;
    const int e = block_excl_scan(c, lds, &tot);
    if (s < a.B) a.soff[s] = run + e;
    run += tot;
  }
}

// One wavefront per sample: every list entry that belongs to the sample's vertices.
__global__ __launch_bounds__(64) void arena_lists_kernel(ArenaArgs a) {
  extern __shared__ int lds[];
  const int s = blockIdx.x, lane = threadIdx.x, ML = a.maxlen;
  int *tidof = lds, *rndof = lds + ML;  // by local vertex id
  if (a.meta[2]) return;                // a rejected batch: nothing below is meaningful
  const int L = a.len[s], so = a.soff[s], D = a.depth[s];
  const int *g_ord = a.ord + (long)s * ML, *g_rnd = a.rnd + (long)s * ML, *g_rst = a.rst + (long)s * ML;
  const int *g_bs = a.bs + (long)s * ML, *g_rb = a.rb + (long)s * ML;
  const int *r2o = a.meta + 8;
  for (int k = lane; k < L; k += 64) {
    const int v = g_ord[k], r = g_rnd[k];
    const int t = r2o[r] + g_bs[r] + (k - g_rst[r]);
    tidof[v] = t;
    rndof[v] = r;
    a.t2j[t] = so + v;
  }
  __syncthreads();
  const bool reference = a.pairing == 0;
  for (int v = lane; v < L; v += 64) {
    const int t = tidof[v], r = rndof[v];
    if (v != L - 1) {
      // Scatter's list holds the non-root jobs of the round, compacted
      // (cavs/midend/graph_scheduler.cc:228-235); entry b meets slab row b of the round
      // (cavs/backend/op_impl_graphop.cu:148-157) under the reference pairing
      if (reference) a.pair[t - g_rb[r]] = t; else a.pair[t] = t;
    }
    const int k0 = a.c0[(long)s * ML + v], k1 = a.c1[(long)s * ML + v];
    if (k1 >= 0) {  // has children: ascending vertex id = child slot (graph_scheduler.cc:52-58,224-227)
      const int kids[2] = {k0, k1};
      for (int i = 0; i < a.nch; i++) {
        const int c = kids[i], tc = tidof[c];
        a.child[(long)a.nch * t + i] = tc;
        a.kid[(long)a.nch * t + i] = reference ? tc - g_rb[rndof[c]] : tc;
      }
    }
  }
  if (lane == 0) {
    a.roots[s] = so + L - 1;
    // the slab rows no message leaves from, ascending: under the reference pairing the last
    // rows of each round, as many as it has roots; else the roots' own rows
    const int r = D - 1, slot = a.rsb[r] + g_rb[r];
    a.orph[slot] = reference ? r2o[r] + a.total[r] - a.nroots[r] + g_rb[r] : tidof[L - 1];
  }
}

}  // namespace cavs

using namespace cavs;

extern "C" {

size_t cavs_schedule_arena_scratch(int B, int maxlen) {
  if (B <= 0 || maxlen <= 0) return 0;
  return ((size_t)8 * B * maxlen + 3 * (size_t)B + 3 * (size_t)maxlen + 64) * sizeof(int);
}

int cavs_schedule_arena(const int *graph, int B, int maxlen, int nchild, int pairing, int *t2j, int *pair,
                        int *child, int *kid_rows, int *roots, int *orphans, long cap, int *meta, void *scratch,
                        size_t scratch_bytes, void *stream) {
  CAVS_REQUIRE(B > 0 && maxlen > 0 && (nchild == 1 || nchild == 2) && (pairing == 0 || pairing == 1),
               "cavs_schedule_arena: bad arguments B=%d maxlen=%d nchild=%d pairing=%d", B, maxlen, nchild, pairing);
  CAVS_REQUIRE(maxlen <= 2048, "cavs_schedule_arena: samples of up to %d vertices, at most 2048 supported", maxlen);
  CAVS_REQUIRE(cap >= (long)B * maxlen, "cavs_schedule_arena: lists of %ld rows for up to %ld vertices", cap, (long)B * maxlen);
  CAVS_REQUIRE(graph && t2j && pair && child && kid_rows && roots && orphans && meta && scratch,
               "cavs_schedule_arena: null pointer");
  CAVS_REQUIRE(scratch_bytes >= cavs_schedule_arena_scratch(B, maxlen), "cavs_schedule_arena: scratch of %zu bytes needed, %zu given",
               cavs_schedule_arena_scratch(B, maxlen), scratch_bytes);
  const size_t BM = (size_t)B * maxlen;
  int *w = static_cast<int *>(scratch);
  ArenaArgs a;
  a.graph = graph;
  a.B = B;
  a.maxlen = maxlen;
  a.nch = nchild;
  a.pairing = pairing;
  a.cap = cap;
  a.ord = w;
  a.rnd = w + BM;
  a.c0 = w + 2 * BM;
  a.c1 = w + 3 * BM;
  a.cnt = w + 4 * BM;
  a.rst = w + 5 * BM;
  a.bs = w + 6 * BM;
  a.rb = w + 7 * BM;
  a.len = w + 8 * BM;
  a.depth = a.len + B;
  a.soff = a.depth + B;
  a.total = a.soff + B;
  a.nroots = a.total + maxlen;
  a.rsb = a.nroots + maxlen;
  a.meta = meta;
  a.t2j = t2j;
  a.pair = pair;
  a.child = child;
  a.kid = kid_rows;
  a.roots = roots;
  a.orph = orphans;
  hipStream_t st = as_stream(stream);
  launch(arena_clear_kernel, (unsigned)((cap * nchild + 255) / 256), 256, 0, st, a);
  CAVS_LAUNCH_CHECK();
  launch(arena_sample_kernel, B, 64, (size_t)6 * maxlen * sizeof(int), st, a);
  CAVS_LAUNCH_CHECK();
  launch(arena_round_kernel, maxlen, 256, 0, st, a);
  CAVS_LAUNCH_CHECK();
  launch(arena_offsets_kernel, 1, 1024, 0, st, a);
  CAVS_LAUNCH_CHECK();
  launch(arena_lists_kernel, B, 64, (size_t)2 * maxlen * sizeof(int), st, a);
  CAVS_LAUNCH_CHECK();
  return CAVS_OK;
}

int cavs_schedule_frontier(const int *parent, int N, int *tids_to_jobids, int *jobids_to_tids,
                           int *round_of_tid, int *round2offset, int *n_rounds, int *scratch,
                           void *stream) {
  CAVS_REQUIRE(N >= 0, "cavs_schedule_frontier: negative N");
  CAVS_REQUIRE(parent && tids_to_jobids && jobids_to_tids && round_of_tid && round2offset &&
                   n_rounds && scratch,
               "cavs_schedule_frontier: null pointer");
  hipStream_t st = as_stream(stream);
  int *nchild = scratch, *cmin = scratch + N, *cmax = scratch + 2 * (size_t)N,
      *level = scratch + 3 * (size_t)N;
  if (N > 0) {
    launch(sched_init_kernel, (N + 255) / 256, 256, 0, st, N, nchild, cmin, cmax, level, tids_to_jobids, jobids_to_tids);
    CAVS_LAUNCH_CHECK();
    launch(sched_children_kernel, (N + 255) / 256, 256, 0, st, parent, N, nchild, cmin, cmax);
    CAVS_LAUNCH_CHECK();
  }
  launch(sched_frontier_kernel, 1, kSchedThreads, 0, st, parent, N, nchild, cmin, cmax, tids_to_jobids,
                                                    jobids_to_tids, level, round_of_tid,
                                                    round2offset, n_rounds);
  CAVS_LAUNCH_CHECK();
  return CAVS_OK;
}

}  // extern "C"
