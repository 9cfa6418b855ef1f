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
                                  int *__restrict__ cmax, int *__restrict__ level) {
  int v = blockIdx.x * blockDim.x + threadIdx.x;
  if (v >= N) return;
  nchild[v] = 0;
  cmin[v] = 0x7fffffff;
  cmax[v] = -1;
  level[v] = -1;
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

}  // namespace cavs

using namespace cavs;

extern "C" {

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
    launch(sched_init_kernel, (N + 255) / 256, 256, 0, st, N, nchild, cmin, cmax, level);
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
