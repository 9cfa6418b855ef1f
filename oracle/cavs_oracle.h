/*
 * cavs_oracle.h -- CPU restatement of the Cavs "vertex function F over instance
 * graph G" path, forward and backward.
 *
 * THIS IS TEST INFRASTRUCTURE, NOT PRODUCT CODE.  Only the tests, the smoke
 * check and the cpu_baseline leg of the benchmark may link or load it, and only
 * as the checker.  The shipped library never calls into it.
 *
 * Every function restates one piece of the reference and cites the reference
 * file:line it follows (paths relative to the reference tree).
 *
 * What pins each function (see tests/test_oracle_*.py):
 *   scheduler (or_sched_*)      hand-derived known-answer vectors, invariants,
 *                               brute-force topological checks
 *   row copies (or_*_rows)      closed form out = in[perm], round trips
 *   or_sgemm                    numpy matmul (fp32), exact rational sums (ord_sgemm)
 *   gate math / model steps     textbook Tree-LSTM / LSTM / Tree-FC in fp64
 *                               autograd (row-preserving mode and same-shape
 *                               batches), finite differences (both modes)
 *   embedding / head            index_select / index_add_, log_softmax + NLL
 * Parity unpinned (nothing in the reference pins them and it cannot run here):
 *   the cuBLAS 8 / cuDNN 5.1 bit patterns, and the order-dependent gradient
 *   overwrite the reference exhibits when a tensor inside F is consumed twice
 *   without Mirror (the restatement accumulates, i.e. behaves as F written with
 *   Mirror on every multi-consumer tensor).
 */
#ifndef CAVS_ORACLE_H_
#define CAVS_ORACLE_H_

#ifdef __cplusplus
extern "C" {
#endif

/* The op and model restatements are compiled twice from the same source
 * (ops.c, model.c):
 *   or_*   real = float  : fp32 throughout, as the reference computes;
 *   ord_*  real = double : the same dataflow, operation for operation, with every
 *          value and every sum held in double (build with -DOR_F64).  Inputs are the
 *          same fp32 numbers widened.  This is what an fp32 implementation is held to
 *          the path's tolerance against: the checker's own fp32 rounding then takes no
 *          share of the budget.
 * The scheduler (or_sched_*) is integer work and exists once. */
#ifdef OR_F64
typedef double real;
#define ORF(name) ord_##name
#define R_EXP exp
#define R_TANH tanh
#define R_LOG log
#define R_FABS fabs
#else
typedef float real;
#define ORF(name) or_##name
#define R_EXP expf
#define R_TANH tanhf
#define R_LOG logf
#define R_FABS fabsf
#endif

/* ------------------------------------------------------------------ scheduler */
typedef struct or_sched or_sched;

/* batching != 0: BatchGraphScheduler, else SerialGraphScheduler
 * (cavs/midend/graph_scheduler.h:126-157). */
or_sched *or_sched_new(int batching);
void or_sched_free(or_sched *s);
/* cavs/midend/graph_scheduler.cc:12-71.  parent_ids is [B, maxlen] int32,
 * entry j = local parent of vertex j, first -1 = root and end of sample.
 * Returns total_length N. */
int or_sched_load_graph(or_sched *s, const int *parent_ids, int B, int maxlen);
/* cavs/midend/graph_scheduler.cc:73-81 */
int or_sched_reverse_graph(or_sched *s);
/* cavs/midend/graph_scheduler.cc:83-108 (serial), :169-200 (batch) */
void or_sched_initialize(or_sched *s);
/* cavs/midend/graph_scheduler.h:135,148 */
int or_sched_terminate(const or_sched *s);
/* cavs/midend/graph_scheduler.cc:125-167 (serial), :202-258 (batch) */
void or_sched_activate_next(or_sched *s);
/* cavs/midend/graph_scheduler.h:136,149 */
int or_sched_round_offset(const or_sched *s);
int or_sched_total_length(const or_sched *s);
int or_sched_is_forward(const or_sched *s);
/* current-round lists; each returns the length and stores the base pointer. */
int or_sched_job_ids(const or_sched *s, const int **p);                  /* GetJobId */
int or_sched_gather_ids(const or_sched *s, int child, const int **p);    /* CurrentRoundTensorIdsForGather */
int or_sched_scatter_ids(const or_sched *s, int child, const int **p);   /* CurrentRoundTensorIdsForScatter */
int or_sched_gather_init_ids(const or_sched *s, const int **p);          /* ...ForGatherInitialization */
int or_sched_tids_to_jobids(const or_sched *s, const int **p);           /* TensorIdsToJobIds */
int or_sched_round2offset(const or_sched *s, const int **p);

/* Runs LoadGraph/Initialize/loop (and, if with_backward, ReverseGraph/
 * Initialize/loop) exactly as cavs/midend/statement.cc:43-123 drives the
 * scheduler, serialising what every round exposes into `out`:
 *   [N, R_fwd, R_bwd,
 *    per round: offset, n_exec, exec..., n_g0, g0..., n_g1, g1...,
 *               n_s0, s0..., n_s1, s1..., n_init, init...,
 *    (forward rounds first, then backward rounds)
 *    N entries of tids_to_jobids, n_r2o, round2offset...]
 * Returns the number of ints written, or -needed if cap is too small. */
int or_sched_trace(const int *parent_ids, int B, int maxlen, int batching,
                   int with_backward, int *out, int cap);

/* ------------------------------------------------------------------ row copies */
/* cavs/backend/functor_batched_memcpy.cuh:33-46 : out[b,:] = inp[ids[b],:] */
void ORF(gather_rows)(real *out, int ld_out, const real *inp, int ld_inp,
                    const int *ids, int n, int w);
/* cavs/backend/functor_batched_memcpy.cuh:48-61 : out[ids[b],:] = inp[b,:] */
void ORF(scatter_rows)(real *out, int ld_out, const int *ids, const real *inp,
                     int ld_inp, int n, int w);
/* cavs/backend/functor_batched_memcpy.cuh:63-75 : out[b,:] = 0, b < n */
void ORF(zero_rows)(real *out, int ld_out, int n, int w);
/* cavs/backend/functor_batched_memcpy.cuh:18-31 : column-block copy */
void ORF(copy_rows)(real *out, int ld_out, const real *inp, int ld_inp, int n, int w);

/* ------------------------------------------------------------------ dense math */
/* Row-major C = alpha*op(A)*op(B) + beta*C, cavs/backend/cublas_wrapper.cc:12-28 */
void ORF(sgemm)(int transA, int transB, int M, int N, int K, real alpha,
              const real *A, int lda, const real *B, int ldb, real beta,
              real *C, int ldc);
/* out[j] (+)= sum_r inp[r,j]; cavs/backend/op_impl_elementwise.cuh:24-34 */
void ORF(colsum)(real *out, const real *inp, int ld, int n, int w, int accumulate);
/* cavs/backend/op_impl_embedding_lookup.cu:22-35 ; ids are floating-point values */
void ORF(embed_fwd)(real *out, int ld_out, const real *ids, const real *table, int n, int E);
/* cavs/backend/op_impl_embedding_lookup.cu:90-103 */
void ORF(embed_bwd)(real *dtable, const real *ids, const real *dy, int ld_dy, int n, int E);
/* cavs/backend/op_impl_softmax_entropy_logits_loss.cu:94-140 (loss) and
 * :150-164,212-250 (grad = (softmax - onehot)/n).  Either output may be NULL. */
void ORF(softmax_xent)(real *loss, real *dlogits, const real *logits,
                     const real *labels, int n, int C);
/* cavs/backend/op_impl_sgd.cu : w -= lr*g */
void ORF(sgd)(real *w, const real *g, real lr, long n);

/* ------------------------------------------------------------------ gate math
 * Slab-level fused restatements of the elementwise chains of the three vertex
 * functions.  Row r of every operand is vertex r of the slab.  `G` holds the
 * gathered child rows interleaved: row 2r = child 0, row 2r+1 = child 1, each
 * [h | c] of width 2H (Tree-LSTM) -- pure layout, same values as the
 * reference's two Gather outputs. */

/* Tree-LSTM forward gates, apps/paper/tree-lstm-cavs.cc:132-171.
 *  xW  [n,4H] cols [i|o|u|f]      hU [n,3H] cols [i|o|u]
 *  hUf [2n,H] rows 2r=f_l, 2r+1=f_r pre-activations from U_f
 *  G   [2n,2H]  bias [4H] blocks [i|f|u|o]
 *  gates [n,6H] = [i|o|u|f_l|f_r|tanh(c)] (saved for backward), msg [n,2H]=[h|c] */
void ORF(treelstm_gates_fwd)(const real *xW, int ld_xw, const real *hU, const real *hUf,
                           const real *G, const real *bias, real *gates,
                           real *msg, int n, int H);
/* Backward of the above.
 *  dmsg [n,2H] gathered-back [dh_m|dc_m]; dret [n,H] pulled d GraphOutput
 *  outputs: dxW [n,4H] = [d_i|d_o|d_u|d_fl+d_fr]; dF [2n,H] rows (d_fl,d_fr);
 *           dG [2n,2H]: only the c half (cols H..2H) is written here
 *           (dc_l, dc_r); the h half comes from the U GEMMs. */
void ORF(treelstm_gates_bwd)(const real *dmsg, const real *dret, const real *gates,
                           const real *G, real *dxW, int ld_dxw, real *dF, real *dG,
                           int n, int H);
/* Chain LSTM, apps/paper/seq-lstm-cavs.cc:62-86.
 *  a [n,4H] = e*U' + h_p*W' cols [i|f|u|o]; G [n,2H]=[h_p|c_p]; bias [4H] same order
 *  gates [n,5H] = [i|f|u|o|tanh(c)] */
void ORF(lstm_gates_fwd)(const real *a, int ld_a, const real *G, const real *bias,
                       real *gates, real *msg, int n, int H);
void ORF(lstm_gates_bwd)(const real *dmsg, const real *dret, const real *gates,
                       const real *G, real *da, int ld_da, real *dG, int n, int H);
/* Tree-FC, apps/paper/tree-fc-cavs.cc:28-36 : h = act(z [+ bias] [+ x]).
 *  act 0 = relu (reference app), 1 = tanh.  bias, x may be NULL. */
void ORF(treefc_fwd)(const real *z, const real *bias, const real *x, real *h,
                   int n, int H, int act);
/* dz = dh * act'(h) */
void ORF(treefc_bwd)(const real *dh_m, const real *dret, const real *h, real *dz,
                   int n, int H, int act);

/* ------------------------------------------------------------------ model steps
 * One forward+backward pass of a whole batch, driven exactly like
 * cavs/midend/statement.cc:43-123 drives F, with the head of the apps
 * (FullyConnected + SoftmaxEntropyLoss) or the alternative losses below. */
enum {
  OR_MODEL_TREELSTM = 0, /* apps/paper/tree-lstm-cavs.cc */
  OR_MODEL_LSTM = 1,     /* apps/paper/seq-lstm-cavs.cc, seq-lstm-cavs-varLength.cc */
  OR_MODEL_TREEFC = 2,   /* apps/paper/tree-fc-cavs.cc */
  /* Not one of the reference's applications: the Tree-LSTM of apps/paper/tree-lstm-cavs.cc:129-172 with
   * a forget-gate matrix per child (U = [U_iou | U_fl | U_fr], 5*H*H) and the bias blocks in the
   * order of the gate columns ([i|o|u|f]) -- a vertex function a user of the reference's API might
   * declare, run through the same ops in the same order.  Pinned by the fp64 autograd formulation
   * in tests/textbook.py. */
  OR_MODEL_TREELSTM2 = 3
};
enum {
  OR_LOSS_SOFTMAX = 0,   /* FC head + softmax cross-entropy at every vertex */
  OR_LOSS_ROOT_SQ = 1,   /* sum over root vertices of h^2 */
  OR_LOSS_SUM_ABS = 2    /* Reduce_sum = sum |h| over all vertices, gradient 1
                            (cavs/backend/op_impl_blas1_cublas.cc:62-77,
                             cavs/backend/op_decl_reduction.cc:19-28) */
};
enum {
  OR_PAIR_REFERENCE = 0, /* b-th list entry <-> b-th slab row, as the reference
                            kernels do (op_impl_graphop.cu:67-76,148-157) */
  OR_PAIR_ROWID = 1      /* row-id preserving: slab row = list[b] - round offset */
};

typedef struct {
  int model, loss, pairing, batching;
  int V, E, H, C;
  int act;        /* Tree-FC: 0 relu, 1 tanh */
  int use_bias;   /* Tree-FC */
  int use_x;      /* Tree-FC: add Pull'ed input row of width H */
  int threads;    /* OpenMP threads for the GEMMs (0/1 = serial) */
} or_config;

/* All parameter pointers are row-major arrays of `real`; unused ones may be NULL.
 *   Tree-LSTM: Emb[V,E] W[E,4H] U[4*H*H] Bv[4H]      (apps/paper/tree-lstm-cavs.cc:110-126)
 *   LSTM     : Emb[V,H] W[8*H*H] (U' then W') Bv[4H]  (apps/paper/seq-lstm-cavs.cc:49-59)
 *   Tree-FC  : W[2H,H] Bv[H]
 *   head     : Wfc[C,H] bfc[C] */
typedef struct {
  const real *Emb, *W, *U, *Bv, *Wfc, *bfc;
} ORF(params);
typedef struct {
  real *dEmb, *dW, *dU, *dBv, *dWfc, *dbfc;
} ORF(grads);

/* graph [B,maxlen] int32 parent ids; x: vertex inputs packed by global vertex id
 * (word ids as floats, or [N,H] rows for Tree-FC with use_x); labels [N] floats
 * packed by global vertex id.
 * Outputs (any may be NULL): loss_rows [N] (softmax) or [1]; graph_out [N,H] in
 * vertex-id order; dgraph_out [N,H]; msg_pool [N,2H or H] by tensor id;
 * grads are overwritten.  Returns N (>0) or a negative error. */
int ORF(model_step)(const or_config *cfg, const ORF(params) *p, const int *graph, int B,
                  int maxlen, const real *x, const real *labels, real *loss_rows,
                  real *graph_out, real *dgraph_out, real *msg_pool, ORF(grads) *g);

#ifdef __cplusplus
}
#endif
#endif
