/*
 * cavs_session.h -- C ABI of the host runtime (libcavs_host.so): the part of the
 * reference's midend that sits on the hot path -- graph scheduler, batching memory
 * manager and the forward / backward round loops -- re-stated in C++ on top of
 * cavs_hip.h.  It plays the role of the reference's outer C API
 * (cavs/frontend/c_api.h:20-36: C_NewSession / C_Run) for the vertex functions the
 * benchmarks use; the Sym/GraphSupport front end (cavs_amd/host/frontend) lowers
 * onto it.
 *
 * Feeds follow the reference's wire format: `graph` is a host int32 [B, maxlen]
 * parent array (cavs/midend/graph_scheduler.cc:35-43; the reference requires the
 * graph placeholder on the CPU, graph_scheduler.cc:15), vertex inputs and labels are
 * fp32 packed by global vertex id (apps/paper/seq-lstm-cavs-varLength.cc:38-56).
 *
 * All functions return 0 or a negative CAVS_E* code (cavs_hip.h);
 * cavs_session_error() holds the message.
 */
#ifndef CAVS_SESSION_H_
#define CAVS_SESSION_H_

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct cavs_session cavs_session;

enum { CAVS_MODEL_TREELSTM = 0, CAVS_MODEL_LSTM = 1, CAVS_MODEL_TREEFC = 2,
       /* a vertex function lowered onto generated kernels: only the front end's sessions make
        * one (its description does not fit this struct); cavs_session_create refuses it */
       CAVS_MODEL_CELL = 3 };
enum { CAVS_LOSS_SOFTMAX = 0, CAVS_LOSS_ROOT_SQ = 1, CAVS_LOSS_SUM_ABS = 2 };
/* How the forward Scatter / backward Gather pair list entries with slab rows:
 * REFERENCE = b-th list entry with b-th slab row, exactly what the reference's
 * kernels do (cavs/backend/op_impl_graphop.cu:67-76,148-157) -- rows shift after a
 * root that is not last in its round; ROWID = the row the tensor id names. */
enum { CAVS_PAIR_REFERENCE = 0, CAVS_PAIR_ROWID = 1 };
/* cavs/proto/opt.proto:3-8 */
enum { CAVS_OPT_FUSION = 1, CAVS_OPT_BATCHING = 2, CAVS_OPT_STREAMMING = 4 };

typedef struct {
  int model, loss, pairing;
  int opt;            /* OPT_* bitmask; without OPT_BATCHING the serial scheduler runs */
  int V, E, H, C;     /* vocabulary, embedding, hidden, classes */
  int act;            /* Tree-FC activation: 0 relu, 1 tanh */
  int use_bias;       /* Tree-FC */
  int use_x;          /* Tree-FC: add the Pull'ed [H] input row */
  int device;
  /* Tree-LSTM: rounds of at most this many vertices run as one fused launch forward and
   * two backward (cavs_treelstm_round_*); larger rounds run gather / GEMM / gates / scatter
   * as separate launches.  0 = default limit, negative = never fuse. */
  int fused_round_rows;
  /* All rounds fused: 0 = when the batch's message flow is a forest, the launch that computes
   * d h of a round's children also does their gate gradients (one launch per backward round,
   * cavs_*_round_bwd_children_gates / _act); 1 = always two launches per round. */
  int split_backward_rounds;
  /* Who builds the round schedule and the index lists of a step (cavs/midend/graph_scheduler.cc:
   * 169-245): 0 = the host scheduler, lists uploaded once per step; 1 = the GPU
   * (cavs_schedule_arena: the graph feed goes up, only the round offsets come back).  Mode 1 runs
   * the serial scheduler's sessions (no OPT_BATCHING) on the host all the same, and refuses a feed
   * whose samples exceed 2048 vertices (CAVS_EUNSUPPORTED).  The counter "scheduler" says who built
   * the last step's lists. */
  int schedule_mode;
  /* Plan cache: keep the schedule and the device-resident lists of the last `plan_cache` distinct
   * graph feeds, keyed by the feed's bytes; a step on a feed seen before skips the scheduler and
   * the upload.  0 = off. */
  int plan_cache;
  /* Tree-LSTM, H = 512, batches whose message flow is a forest: the rounds from the first one on
   * whose rows can be dealt to eight groups, whole trees of the message flow per group, with at
   * most this many rows per group (the last forward rounds, the first backward rounds) run as one launch per
   * direction (cavs_treelstm_tail_fwd / _bwd) instead of one launch per round
   * (cavs/midend/statement.cc:69-76,106-111).  0 = default (64, which at 64 trees per batch takes in
   * every round above the leaves; a group's share of a round runs in slices of at most 32 rows),
   * negative = never.  The session
   * checks once, when it is created, that the device runs such a launch's workgroups all at once,
   * each group on one XCD, and keeps to one launch per round if not. */
  int tail_rows;
  /* With a plan cache: 1 = a step on a batch structure seen before, with the same input buffers
   * (inputs_on_device) and the session in the same state as the last time, enqueues its forward
   * pass, loss head and backward pass as one recorded graph of launches (cavs_graph_launch) instead
   * of re-issuing every launch from the host loop (cavs/midend/statement.cc:69-76); the launch that
   * applies the parameter updates stays a launch of its own.  The first such step records, the
   * later ones replay.  Any other call on the session, or a buffer that had to grow, makes
   * the next step an ordinary one.  Replayed steps have no "RNNForward" / "RNNBackward" timings.
   * The counter "graph_replays" counts them.  0 = off. */
  int graph_replay;
  /* Chain LSTM with a wide classifier head (head weights of at least 2^18 elements), host
   * scheduler, message flow a forest: the head runs over chunks of the rounds on a second stream
   * beside the backward rounds (cavs/midend/statement.cc:69-76,106-111 run them one
   * after the other): the chunks last first, each one's d h releasing the backward rounds of its
   * rows while the next chunk's is computed.  0 = default (two chunks), 2..4 = that many, negative =
   * off: the head in one piece between the two passes.  The counter "head_chunks" says in how many
   * chunks the last step's head ran (0: in one piece). */
  int head_chunks;
} cavs_session_config;

const char *cavs_session_error(void);
int cavs_session_create(const cavs_session_config *cfg, cavs_session **out);
int cavs_session_destroy(cavs_session *s);

/* Parameters and their gradients by name: "Emb" "W" "U" "Bv" "Wfc" "bfc"
 * (shapes: apps/paper/tree-lstm-cavs.cc:110-126, seq-lstm-cavs.cc:49-59,
 * tree-fc-cavs.cc:24). `n` is the element count and must match. */
int cavs_session_set_param(cavs_session *s, const char *name, const float *host, size_t n);
int cavs_session_get_param(cavs_session *s, const char *name, float *host, size_t n);
int cavs_session_get_grad(cavs_session *s, const char *name, float *host, size_t n);

/* One pass of F over the batch (C_Run of the train op, cavs/frontend/c_api.cc:149-172):
 * schedule, forward rounds, loss head, and if `backward` the gradient rounds and the
 * deferred weight gradients; if lr != 0 also the SGD update (cavs/backend/op_impl_sgd.cu).
 * x and labels are host pointers unless inputs_on_device is set, in which case they
 * are device pointers to buffers already resident in HBM.  The call only enqueues
 * work; cavs_session_sync() waits for it. */
int cavs_session_step(cavs_session *s, const int *graph, int B, int maxlen, const void *x,
                      const void *labels, int inputs_on_device, int backward, float lr);
int cavs_session_sync(cavs_session *s);

/* Results of the last step, copied to host (synchronises):
 *   "loss" [N] (softmax) or [1]; "graph_out" [N,H] in vertex order; "dgraph_out" [N,H];
 *   "msg_pool" [N, 2H | H] by tensor id. */
int cavs_session_fetch(cavs_session *s, const char *what, float *host, size_t n);
int cavs_session_total_length(cavs_session *s); /* N of the last step */

/* The last step's schedule in the serialisation of Schedule::trace (forward rounds,
 * backward rounds, tids_to_jobids, round2offset).  Returns the number of ints, or the
 * negative of the needed capacity. */
int cavs_session_schedule_trace(cavs_session *s, int *out, int cap);
/* Pure host call (no device): schedule of a graph feed, same serialisation. */
int cavs_schedule_trace(const int *graph, int B, int maxlen, int batching, int with_backward,
                        int *out, int cap);

/* Pure host calls (no device) around the index lists a step's kernels consume -- what the host
 * scheduler uploads and what cavs_schedule_arena (cavs_hip.h) builds on the GPU; layouts as
 * documented there.  cavs_schedule_index_lists: graph feed -> lists; arrays of N (t2j, pair),
 * nchild * N (child, kid_rows), B (roots) and N (orphans) ints; *n_orphans = -1 and kid_rows /
 * orphans undefined when the batch's message flow is not a forest or a round with children
 * exceeds fused_limit.  Returns N, or 0 with the reason in cavs_session_error().
 * cavs_schedule_trace_from_lists: the inverse -- lists and round offsets back to a complete
 * schedule, serialised like cavs_schedule_trace. */
int cavs_schedule_index_lists(const int *graph, int B, int maxlen, int nchild, int pairing, int fused_limit,
                              int *t2j, int *pair, int *child, int *roots, int *kid_rows, int *orphans,
                              int *n_orphans);
/* Pure host call: for a batch of binary trees, what the launches over the rounds near the roots
 * (cavs_treelstm_tail_fwd / _bwd, cavs_hip.h) would be given -- the deal the session makes when its
 * tail_rows allows.  rows_limit: most rows of a round a group may get; groups (1..8), max_lists: what
 * the launches take (cavs_tail_max_groups, cavs_tail_max_rounds).  Out: meta[0] = first round inside
 * the launches, meta[1] = M, the lists per group the arrays are laid out for, meta[2] / meta[3] = lists
 * and four-row tiles of the longest group; nrounds [groups]; start, count, flags (forward order) and
 * bstart, bcount, bflags (backward order), each [groups * max_lists] with list i of group g at
 * g * M + i; rows_out [B * maxlen]: the groups' slab rows.  Returns the number of slab rows (0: no
 * suffix of the rounds can be dealt that way), or -1 with the reason in cavs_session_error(). */
int cavs_schedule_tail_lists(const int *graph, int B, int maxlen, int pairing, int fused_limit, int rows_limit, int groups,
                             int max_lists, int *meta, int *nrounds, int *start, int *count, int *flags, int *bstart,
                             int *bcount, int *bflags, int *rows_out);
int cavs_schedule_trace_from_lists(int B, int maxlen, int N, int nchild, const int *round2offset, int R,
                                   const int *t2j, const int *pair, const int *child, const int *roots,
                                   int with_backward, int *out, int cap);

/* Timers of the last step in ms, by the reference's names (cavs/midend/statement.cc:
 * 53,65,68,84,102,122): "GraphParsing" (host), "RNNForward", "RNNBackward" (device); and the
 * host-side split "HostSchedule" (scheduler), "HostWait" (waiting for the device to release
 * an index staging buffer), "HostStep" (the whole enqueueing call). */
int cavs_session_timing(cavs_session *s, const char *name, float *ms);
/* Device time per kernel class.  While enabled, every entry point the session calls has its
 * kernels stamp a pair of events at their own begin and end (cavs_profile_arm); profile_read
 * waits for the stream and returns the summed kernel time and call count since profiling was
 * enabled.  Classes: "gemm" "gather" "scatter" "gates" "round" (fused rounds) "other". */
int cavs_session_profile(cavs_session *s, int enable);
int cavs_session_profile_read(cavs_session *s, const char *kernel_class, double *total_ms,
                              double *launches);
/* Raw stream the session enqueues on (for callers that want to bracket it with events). */
void *cavs_session_stream(cavs_session *s);
/* Per-step counts for roofline accounting: rows moved by indexed copies and GEMM flops
 * of the last step. keys: "gather_rows" "scatter_rows" "gemm_flops" (separate GEMM launches: 2*M*N*K
 * of the reference's products) "gemm_flops_hinted" (the part of those that multiplies blocks known
 * to be zero or unused -- the forget-gate columns of the leaves -- and is skipped tile by tile)
 * "round_flops" (products inside fused round launches) "rounds" "launches"; "tail_rounds" (rounds,
 * forward and backward, that ran inside cavs_treelstm_tail_* launches) "tail_launches"; "plan_hits" /
 * "plan_misses" of the plan cache since the session was created; "scheduler" (who produced the last
 * step's lists: 0 host scheduler, 1 device scheduler, 2 plan cache); "tail_ready" (1 when the session may
 * use the tail launches); the last step's tail plan: "tail_first_round" (-1: none), "tail_vertices",
 * and of its longest group "tail_lists_max" (rounds) and "tail_tiles_max" (tiles of four rows). */
int cavs_session_counter(cavs_session *s, const char *key, double *value);

#ifdef __cplusplus
}
#endif
#endif
