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
// end of sample (cavs/midend/graph_scheduler.cc:35-43).
std::string build_schedule(const int32_t *graph, int B, int maxlen, bool batching, Schedule *out);

}  // namespace cavs
#endif
