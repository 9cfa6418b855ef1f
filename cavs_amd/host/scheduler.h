// Host-side batching policy: turns the parent-array graph feed into the level-wise
// round schedule and the gather/scatter index lists of one step.
//
// Same contract as the reference's schedulers (cavs/midend/graph_scheduler.{h,cc}):
// identical rounds, tensor ids and list contents.  Unlike the reference, which
// rebuilds vectors of vectors (and reserves four 2^20-int vectors) every round, the
// whole step is produced in one pass into flat arrays that are uploaded to the
// device once.
#ifndef CAVS_HOST_SCHEDULER_H_
#define CAVS_HOST_SCHEDULER_H_

#include <cstdint>
#include <string>
#include <vector>

namespace cavs {

struct Round {
  int offset;  // first tensor id (= slab row) of the round
  int n;       // jobs in the round
  // [begin, end) ranges into Schedule::gather_ids[c] / scatter_ids
  int gather_begin[2], gather_end[2];
  int scatter_begin, scatter_end;
};

struct Schedule {
  int B = 0, maxlen = 0, N = 0;
  bool batching = true;
  std::vector<int> sample_offset;  // [B]
  std::vector<int> parent;         // [N] global parent id or -1
  std::vector<int> child_begin;    // [N+1] CSR over children, ascending vertex id
  std::vector<int> child;          // [N - roots]
  std::vector<Round> rounds;       // forward order; backward replays them reversed
  std::vector<int> tids_to_jobids; // [N] (= concatenated job lists of the rounds)
  std::vector<int> jobids_to_tids; // [N]
  std::vector<int> round2offset;   // [R+1]; batch scheduler only
  std::vector<int> gather_ids[2];  // forward CurrentRoundTensorIdsForGather(c), concatenated
  std::vector<int> scatter_ids;    // forward CurrentRoundTensorIdsForScatter(0), concatenated
  std::vector<int> root_tids;      // tids_for_gather_init_[1] after the forward pass
  std::vector<int> bwd_rounds;     // indices into `rounds` in backward execution order
  int executed = 0;                // vertices that ran (N minus single-vertex samples)
  int max_round = 0;               // largest round size
  int leaf_prefix = 0;             // leading tensor ids that are all leaves (batch: round 0)

  // Serialises the rounds exactly as the reference's ops would see them, forward
  // then (optionally) backward: see `trace_format` in scheduler.cc.
  std::vector<int> trace(bool with_backward) const;
};

// Returns an empty string on success, else the reason the graph was rejected.
// graph: [B, maxlen] int32, entry j = local parent of vertex j, first -1 = root and
// end of sample (cavs/midend/graph_scheduler.cc:35-43).  Rejected besides malformed rows: a
// vertex with more than two children (the reference CHECK-aborts when it fills its two gather
// lists, graph_scheduler.cc:223) and parent cycles (their vertices never become ready).  A sample
// of a single vertex is scheduled around, as the reference does (graph_scheduler.cc:180):
// executed < N then tells the caller, who decides whether to accept such a batch.
std::string build_schedule(const int32_t *graph, int B, int maxlen, bool batching, Schedule *out);

// The index lists the kernels consume, one entry per slab row, from a schedule:
//   t2j   [N]      tensor id -> global vertex id (Pull, FunctionPopRet)
//   pair  [N]      per slab row: pool row the forward Scatter writes and the backward Gather
//                  reads, or -1.  pairing 0: b-th entry of the round's compacted scatter list with
//                  the b-th slab row (cavs/backend/op_impl_graphop.cu:148-157); 1: the row itself
//   child [nch*N]  per slab row and child slot: pool row the forward Gather reads (-1: none)
//   roots [B]      vertex ids of the roots
// nch: children of an internal vertex (1 chains, 2 binary trees); a round in which some but not
// all vertices have child c is an error (the reference's gather lists misalign there too).
std::string build_index_lists(const Schedule &s, int nch, int pairing, int *t2j, int *pair, int *child, int *roots);

// For the backward launches that address a child by the slab row that wrote its pool row:
// kid_rows [nch*N] (-1: none) and the slab rows nobody reads a message from (orphans, ascending;
// *n_orphans of them).  False when the message flow of the batch is not a forest (a pool row with
// two writers or two readers, a message nobody reads, a reader in a round not after its writer's)
// or a round with children is larger than `fused_limit`.
bool build_forest_lists(const Schedule &s, int nch, int fused_limit, const int *pair, const int *child, int *kid_rows,
                        int *orphans, int *n_orphans);

// What the launches over the rounds near the roots run (cavs_treelstm_tail_fwd / _bwd), for one
// batch structure: the rounds from `first` on, their rows dealt to the groups by whole trees of
// the message flow (no message crosses groups), each group's share of a round as lists of at
// most `slice` rows with the flag word the launches take (2 * arrivals to wait for + arrives).
struct TailLists {
  int first = -1;  // first round (forward order) inside the launches; -1: none
  int max_rounds = 0;                             // lists per group the arrays below are laid out for
  std::vector<int> nrounds, start, count, flags;  // per group; lists in forward order
  std::vector<int> bstart, bcount, bflags;        // the same lists in backward order
  size_t rows = 0;                                // length of the list of slab rows
  int lists_max = 0, tiles_max = 0;               // the longest group: its lists, its tiles of four rows
};
// kid_rows as build_forest_lists leaves them (binary trees); rows_out: room for N ints.
void build_tail_lists(const Schedule &s, const int *kid_rows, int lim, int groups, int max_lists, int slice, TailLists *out,
                      int *rows_out);

// The inverse of build_index_lists for a batch schedule: rounds and lists of a Schedule from the
// arrays (as a device scheduler leaves them) and the round offsets; `out` compares equal, trace
// for trace, to the schedule the lists came from.
void schedule_from_lists(int B, int maxlen, int N, int nch, const int *round2offset, int R, const int *t2j,
                         const int *pair, const int *child, const int *roots, Schedule *out);

}  // namespace cavs
#endif
