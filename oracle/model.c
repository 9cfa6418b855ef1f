/*
 * Test infrastructure: one forward+backward pass of a whole batch through the
 * vertex function F, driven round by round exactly like the reference's
 * GraphStatement::Run / GraphGradStatement::Run (cavs/midend/statement.cc:43-123)
 * drive it, on top of the scheduler and op restatements.  Not linked into the
 * shipped library.
 *
 * Memory layout follows the reference's batching memory manager
 * (cavs/midend/graph_session.cc:45-206, cavs/midend/op_context.cc:13-91): every
 * edge of F is a [MAX_NODE, width] buffer and round r lives at rows
 * [round_offset, +n_r), i.e. row index == tensor id for every edge; gradient
 * edges are zeroed whole once per iteration (cavs/midend/tensor.cc:283-300).
 * The reference aliases all Scatter outputs, forward and backward, onto one
 * message pool; here the backward pool is a separate buffer, which is
 * observationally identical because every pool row read in backward was written
 * in backward first.
 */
#include "cavs_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

typedef struct {
  const or_config *cfg;
  const ORF(params) *p;
  ORF(grads) *g;
  or_sched *s;
  int B, N, MAXR, H, E, mw; /* mw = message width */
  const real *x;           /* packed vertex inputs */
  int xw;                   /* width of one vertex input row (Pull stride) */
  /* forward edges */
  real *pool, *G, *hlr, *xs, *e, *xW, *hU, *hUf, *gates, *msg, *ret, *z;
  /* backward edges */
  real *dpool, *dmsg, *dret, *dxW, *dF, *dG, *dhlr, *dhf, *de;
  real *GO, *dGO;
  real *bias; /* OR_MODEL_TREELSTM2: the bias in the block order the gate op reads ([i|f|u|o]) */
} ctx;

static real *zalloc(size_t n) { return (real *)calloc(n ? n : 1, sizeof(real)); }

/* Gather op, cavs/backend/op_impl_graphop.cu:32-90, into the interleaved child
 * layout (row nchild*t + child). */
static void do_gather(ctx *c, int child, int nchild, real *out, int w, const real *pool,
                      int rowid_pairing) {
  const int *ids, *init;
  int off = or_sched_round_offset(c->s);
  int n = or_sched_gather_ids(c->s, child, &ids);
  if (n > 0) {
    for (int b = 0; b < n; b++) {
      int row = rowid_pairing ? ids[b] : off + b;
      memcpy(out + ((size_t)nchild * row + child) * w, pool + (size_t)ids[b] * w,
             sizeof(real) * (size_t)w);
    }
  } else {
    int k = or_sched_gather_init_ids(c->s, &init);
    for (int b = 0; b < k; b++)
      memset(out + ((size_t)nchild * (off + b) + child) * w, 0, sizeof(real) * (size_t)w);
  }
}

/* Scatter op, cavs/backend/op_impl_graphop.cu:108-161 */
static void do_scatter(ctx *c, int child, int nchild, real *pool, int w, const real *inp,
                       int rowid_pairing) {
  const int *ids;
  int off = or_sched_round_offset(c->s);
  int n = or_sched_scatter_ids(c->s, child, &ids);
  for (int b = 0; b < n; b++) {
    int row = rowid_pairing ? ids[b] : off + b;
    memcpy(pool + (size_t)ids[b] * w, inp + ((size_t)nchild * row + child) * w,
           sizeof(real) * (size_t)w);
  }
}

/* Pull op, cavs/backend/op_impl_graphop.cu:214-254: rows of the function argument
 * selected by global job id. */
static void do_pull(ctx *c, real *out, const real *arg, int w) {
  const int *jobs;
  int off = or_sched_round_offset(c->s);
  int n = or_sched_job_ids(c->s, &jobs);
  ORF(gather_rows)(out + (size_t)off * w, w, arg, w, jobs, n, w);
}

static void fwd_round(ctx *c) {
  const or_config *cfg = c->cfg;
  const ORF(params) *p = c->p;
  const int *jobs;
  int H = c->H, E = c->E;
  int off = or_sched_round_offset(c->s);
  int n = or_sched_job_ids(c->s, &jobs);
  /* forward scatter: in row-id mode the slab row is list[b]; forward gather lists
   * are aligned with the job list in both modes. */
  int rowid = cfg->pairing == OR_PAIR_ROWID;
  if (cfg->model == OR_MODEL_TREELSTM || cfg->model == OR_MODEL_TREELSTM2) {
    do_gather(c, 0, 2, c->G, 2 * H, c->pool, 0);
    do_gather(c, 1, 2, c->G, 2 * H, c->pool, 0);
    real *G = c->G + (size_t)2 * off * 2 * H;
    real *hlr = c->hlr + (size_t)off * H;
    for (int b = 0; b < n; b++) /* h_lr = h_l + h_r, tree-lstm-cavs.cc:137 */
      for (int j = 0; j < H; j++)
        hlr[(size_t)b * H + j] = G[(size_t)(2 * b) * 2 * H + j] + G[(size_t)(2 * b + 1) * 2 * H + j];
    do_pull(c, c->xs, c->x, 1);
    real *e = c->e + (size_t)off * E;
    ORF(embed_fwd)(e, E, c->xs + off, p->Emb, n, E);
    real *xW = c->xW + (size_t)off * 4 * H, *hU = c->hU + (size_t)off * 3 * H;
    real *hUf = c->hUf + (size_t)2 * off * H;
    ORF(sgemm)(0, 0, n, 4 * H, E, 1.f, e, E, p->W, 4 * H, 0.f, xW, 4 * H);               /* :146 */
    ORF(sgemm)(0, 0, n, 3 * H, H, 1.f, hlr, H, p->U, 3 * H, 0.f, hU, 3 * H);              /* :151 */
    if (cfg->model == OR_MODEL_TREELSTM2) { /* rows 2b with U_fl, rows 2b+1 with U_fr */
      ORF(sgemm)(0, 0, n, H, H, 1.f, G, 4 * H, p->U + (size_t)3 * H * H, H, 0.f, hUf, 2 * H);
      ORF(sgemm)(0, 0, n, H, H, 1.f, G + 2 * H, 4 * H, p->U + (size_t)4 * H * H, H, 0.f, hUf + H, 2 * H);
    } else {
      ORF(sgemm)(0, 0, 2 * n, H, H, 1.f, G, 2 * H, p->U + (size_t)3 * H * H, H, 0.f, hUf, H); /* :156-157 */
    }
    ORF(treelstm_gates_fwd)(xW, 4 * H, hU, hUf, G, c->bias ? c->bias : p->Bv, c->gates + (size_t)off * 6 * H,
                          c->msg + (size_t)off * 2 * H, n, H);
    do_scatter(c, 0, 1, c->pool, 2 * H, c->msg, rowid);                                   /* :170 */
    ORF(copy_rows)(c->ret + (size_t)off * H, H, c->msg + (size_t)off * 2 * H, 2 * H, n, H); /* :171 Push */
  } else if (cfg->model == OR_MODEL_LSTM) {
    do_gather(c, 0, 1, c->G, 2 * H, c->pool, 0);
    real *G = c->G + (size_t)off * 2 * H;
    do_pull(c, c->xs, c->x, 1);
    real *e = c->e + (size_t)off * E;
    ORF(embed_fwd)(e, E, c->xs + off, p->Emb, n, E);
    real *a = c->xW + (size_t)off * 4 * H;
    /* seq-lstm-cavs.cc:69-71: x*U' + h_p*W' */
    ORF(sgemm)(0, 0, n, 4 * H, E, 1.f, e, E, p->W, 4 * H, 0.f, a, 4 * H);
    ORF(sgemm)(0, 0, n, 4 * H, H, 1.f, G, 2 * H, p->W + (size_t)4 * H * H, 4 * H, 1.f, a, 4 * H);
    ORF(lstm_gates_fwd)(a, 4 * H, G, p->Bv, c->gates + (size_t)off * 5 * H,
                      c->msg + (size_t)off * 2 * H, n, H);
    do_scatter(c, 0, 1, c->pool, 2 * H, c->msg, rowid);
    ORF(copy_rows)(c->ret + (size_t)off * H, H, c->msg + (size_t)off * 2 * H, 2 * H, n, H);
  } else {
    do_gather(c, 0, 2, c->G, H, c->pool, 0);
    do_gather(c, 1, 2, c->G, H, c->pool, 0);
    real *G = c->G + (size_t)2 * off * H; /* = [G0|G1] rows of width 2H */
    real *z = c->z + (size_t)off * H, *xin = NULL;
    if (cfg->use_x) {
      do_pull(c, c->xs, c->x, H);
      xin = c->xs + (size_t)off * H;
    }
    ORF(sgemm)(0, 0, n, H, 2 * H, 1.f, G, 2 * H, p->W, H, 0.f, z, H); /* tree-fc-cavs.cc:32 */
    ORF(treefc_fwd)(z, cfg->use_bias ? p->Bv : NULL, xin, c->msg + (size_t)off * H, n, H, cfg->act);
    do_scatter(c, 0, 1, c->pool, H, c->msg, rowid);
    ORF(copy_rows)(c->ret + (size_t)off * H, H, c->msg + (size_t)off * H, H, n, H);
  }
}

/* Weight-gradient ops over slab rows [off, off+n).  With OPT_BATCHING the
 * reference runs them once over all rows after the backward loop
 * (cavs/midend/batch_weight_updater.h:12-84, statement.cc:112-117); without it
 * they run in every round and accumulate through Mirror's Accumulate gradient
 * (cavs/backend/op_decl_slice_join.cc:173-182). */
static void weight_grads(ctx *c, int off, int n) {
  const or_config *cfg = c->cfg;
  ORF(grads) *g = c->g;
  int H = c->H, E = c->E;
  if (cfg->model == OR_MODEL_TREELSTM2) {
    const real *dxW = c->dxW + (size_t)off * 4 * H;
    const real *G = c->G + (size_t)2 * off * 2 * H, *dF = c->dF + (size_t)2 * off * H;
    ORF(sgemm)(1, 0, E, 4 * H, n, 1.f, c->e + (size_t)off * E, E, dxW, 4 * H, 1.f, g->dW, 4 * H);
    ORF(sgemm)(1, 0, H, 3 * H, n, 1.f, c->hlr + (size_t)off * H, H, dxW, 4 * H, 1.f, g->dU, 3 * H);
    ORF(sgemm)(1, 0, H, H, n, 1.f, G, 4 * H, dF, 2 * H, 1.f, g->dU + (size_t)3 * H * H, H);
    ORF(sgemm)(1, 0, H, H, n, 1.f, G + 2 * H, 4 * H, dF + H, 2 * H, 1.f, g->dU + (size_t)4 * H * H, H);
    ORF(colsum)(g->dBv, dxW, 4 * H, n, 4 * H, 1); /* bias blocks in the order of the columns */
  } else if (cfg->model == OR_MODEL_TREELSTM) {
    const real *dxW = c->dxW + (size_t)off * 4 * H;
    ORF(sgemm)(1, 0, E, 4 * H, n, 1.f, c->e + (size_t)off * E, E, dxW, 4 * H, 1.f, g->dW, 4 * H);
    ORF(sgemm)(1, 0, H, 3 * H, n, 1.f, c->hlr + (size_t)off * H, H, dxW, 4 * H, 1.f, g->dU, 3 * H);
    ORF(sgemm)(1, 0, H, H, 2 * n, 1.f, c->G + (size_t)2 * off * 2 * H, 2 * H,
             c->dF + (size_t)2 * off * H, H, 1.f, g->dU + (size_t)3 * H * H, H);
    /* bias blocks [i|f|u|o] from dxW columns [i|o|u|f] */
    ORF(colsum)(g->dBv, dxW, 4 * H, n, H, 1);
    ORF(colsum)(g->dBv + H, dxW + 3 * H, 4 * H, n, H, 1);
    ORF(colsum)(g->dBv + 2 * H, dxW + 2 * H, 4 * H, n, H, 1);
    ORF(colsum)(g->dBv + 3 * H, dxW + H, 4 * H, n, H, 1);
  } else if (cfg->model == OR_MODEL_LSTM) {
    const real *da = c->dxW + (size_t)off * 4 * H;
    ORF(sgemm)(1, 0, E, 4 * H, n, 1.f, c->e + (size_t)off * E, E, da, 4 * H, 1.f, g->dW, 4 * H);
    ORF(sgemm)(1, 0, H, 4 * H, n, 1.f, c->G + (size_t)off * 2 * H, 2 * H, da, 4 * H, 1.f,
             g->dW + (size_t)4 * H * H, 4 * H);
    ORF(colsum)(g->dBv, da, 4 * H, n, 4 * H, 1);
  } else {
    const real *dz = c->dxW + (size_t)off * H;
    ORF(sgemm)(1, 0, 2 * H, H, n, 1.f, c->G + (size_t)2 * off * H, 2 * H, dz, H, 1.f, g->dW, H);
    if (cfg->use_bias) ORF(colsum)(g->dBv, dz, H, n, H, 1);
  }
}

static void bwd_round(ctx *c) {
  const or_config *cfg = c->cfg;
  const ORF(params) *p = c->p;
  const int *jobs;
  int H = c->H, E = c->E, mw = c->mw;
  int off = or_sched_round_offset(c->s);
  int n = or_sched_job_ids(c->s, &jobs);
  int rowid = cfg->pairing == OR_PAIR_ROWID;
  /* grad of Push is Pull (op_decl_graphop.cc): rows of d GraphOutput by job id */
  ORF(gather_rows)(c->dret + (size_t)off * H, H, c->dGO, H, jobs, n, H);
  /* grad of Scatter is Gather(Child=0) on the swapped lists */
  do_gather(c, 0, 1, c->dmsg, mw, c->dpool, rowid);
  const real *dmsg = c->dmsg + (size_t)off * mw, *dret = c->dret + (size_t)off * H;
  if (cfg->model == OR_MODEL_TREELSTM || cfg->model == OR_MODEL_TREELSTM2) {
    real *dxW = c->dxW + (size_t)off * 4 * H, *dF = c->dF + (size_t)2 * off * H;
    real *dG = c->dG + (size_t)2 * off * 2 * H;
    const real *G = c->G + (size_t)2 * off * 2 * H;
    ORF(treelstm_gates_bwd)(dmsg, dret, c->gates + (size_t)off * 6 * H, G, dxW, 4 * H, dF, dG, n, H);
    real *dhlr = c->dhlr + (size_t)off * H, *dhf = c->dhf + (size_t)2 * off * H;
    ORF(sgemm)(0, 1, n, H, 3 * H, 1.f, dxW, 4 * H, p->U, 3 * H, 0.f, dhlr, H);
    if (cfg->model == OR_MODEL_TREELSTM2) {
      ORF(sgemm)(0, 1, n, H, H, 1.f, dF, 2 * H, p->U + (size_t)3 * H * H, H, 0.f, dhf, 2 * H);
      ORF(sgemm)(0, 1, n, H, H, 1.f, dF + H, 2 * H, p->U + (size_t)4 * H * H, H, 0.f, dhf + H, 2 * H);
    } else {
      ORF(sgemm)(0, 1, 2 * n, H, H, 1.f, dF, H, p->U + (size_t)3 * H * H, H, 0.f, dhf, H);
    }
    for (int b = 0; b < 2 * n; b++) /* dh_l = dh_lr + d_fl*U_f^T (Mirror accumulate) */
      for (int j = 0; j < H; j++)
        dG[(size_t)b * 2 * H + j] = dhlr[(size_t)(b / 2) * H + j] + dhf[(size_t)b * H + j];
    real *de = c->de + (size_t)off * E;
    ORF(sgemm)(0, 1, n, E, 4 * H, 1.f, dxW, 4 * H, p->W, 4 * H, 0.f, de, E);
    ORF(embed_bwd)(c->g->dEmb, c->xs + off, de, E, n, E);
    do_scatter(c, 0, 2, c->dpool, 2 * H, c->dG, 0);
    do_scatter(c, 1, 2, c->dpool, 2 * H, c->dG, 0);
  } else if (cfg->model == OR_MODEL_LSTM) {
    real *da = c->dxW + (size_t)off * 4 * H, *dG = c->dG + (size_t)off * 2 * H;
    ORF(lstm_gates_bwd)(dmsg, dret, c->gates + (size_t)off * 5 * H, c->G + (size_t)off * 2 * H, da,
                      4 * H, dG, n, H);
    ORF(sgemm)(0, 1, n, H, 4 * H, 1.f, da, 4 * H, p->W + (size_t)4 * H * H, 4 * H, 0.f, dG, 2 * H);
    real *de = c->de + (size_t)off * E;
    ORF(sgemm)(0, 1, n, E, 4 * H, 1.f, da, 4 * H, p->W, 4 * H, 0.f, de, E);
    ORF(embed_bwd)(c->g->dEmb, c->xs + off, de, E, n, E);
    do_scatter(c, 0, 1, c->dpool, 2 * H, c->dG, 0);
  } else {
    real *dz = c->dxW + (size_t)off * H, *dG = c->dG + (size_t)2 * off * H;
    ORF(treefc_bwd)(dmsg, dret, c->msg + (size_t)off * H, dz, n, H, cfg->act);
    ORF(sgemm)(0, 1, n, 2 * H, H, 1.f, dz, H, p->W, H, 0.f, dG, 2 * H);
    do_scatter(c, 0, 2, c->dpool, H, c->dG, 0);
    do_scatter(c, 1, 2, c->dpool, H, c->dG, 0);
  }
  if (!cfg->batching) weight_grads(c, off, n);
}

int ORF(model_step)(const or_config *cfg, const ORF(params) *p, const int *graph, int B, int maxlen,
                  const real *x, const real *labels, real *loss_rows, real *graph_out,
                  real *dgraph_out, real *msg_pool, ORF(grads) *g) {
#ifdef _OPENMP
  omp_set_num_threads(cfg->threads > 1 ? cfg->threads : 1);
#endif
  ctx c;
  memset(&c, 0, sizeof c);
  c.cfg = cfg;
  c.p = p;
  c.g = g;
  c.B = B;
  int H = c.H = cfg->H, E = c.E = (cfg->model == OR_MODEL_LSTM ? cfg->H : cfg->E);
  int tree = cfg->model != OR_MODEL_LSTM, fc = cfg->model == OR_MODEL_TREEFC;
  int mw = c.mw = fc ? H : 2 * H;
  c.s = or_sched_new(cfg->batching);
  int N = c.N = or_sched_load_graph(c.s, graph, B, maxlen);
  if (N <= 0) {
    or_sched_free(c.s);
    return N < 0 ? N : -3;
  }
  /* MAX_NODE rows as in the reference, plus B so the id-less zero fill
   * (functor_batched_memcpy.cuh:63-75) of a short last round stays in bounds */
  size_t R = (size_t)B * maxlen + B;
  c.MAXR = (int)R;
  c.x = x;
  int nch = tree ? 2 : 1;
  c.pool = zalloc(R * mw);
  c.dpool = zalloc(R * mw);
  c.G = zalloc(R * nch * mw);
  c.dG = zalloc(R * nch * mw);
  c.msg = zalloc(R * mw);
  c.dmsg = zalloc(R * mw); /* zeroed once per iteration */
  c.ret = zalloc(R * H);
  c.dret = zalloc(R * H);
  c.GO = zalloc((size_t)N * H);
  c.dGO = zalloc((size_t)N * H);
  if (!fc) {
    c.xs = zalloc(R);
    c.e = zalloc(R * E);
    c.de = zalloc(R * E);
    c.xW = zalloc(R * 4 * H);
    c.dxW = zalloc(R * 4 * H);
    c.gates = zalloc(R * 6 * H);
  } else {
    c.xs = zalloc(R * H);
    c.z = zalloc(R * H);
    c.dxW = zalloc(R * H);
  }
  if (cfg->model == OR_MODEL_TREELSTM2) {
    static const int from[4] = {0, 3, 2, 1}; /* block k of [i|f|u|o] is block from[k] of [i|o|u|f] */
    c.bias = zalloc((size_t)4 * H);
    for (int k = 0; k < 4; k++) memcpy(c.bias + (size_t)k * H, p->Bv + (size_t)from[k] * H, sizeof(real) * (size_t)H);
  }
  if (cfg->model == OR_MODEL_TREELSTM || cfg->model == OR_MODEL_TREELSTM2) {
    c.hlr = zalloc(R * H);
    c.dhlr = zalloc(R * H);
    c.hU = zalloc(R * 3 * H);
    c.hUf = zalloc(R * 2 * H);
    c.dF = zalloc(R * 2 * H);
    c.dhf = zalloc(R * 2 * H);
  }

  /* ---- forward: statement.cc:43-85 ---- */
  or_sched_initialize(c.s);
  while (!or_sched_terminate(c.s)) {
    fwd_round(&c);
    or_sched_activate_next(c.s);
  }
  /* FunctionPopRet, op_impl_graphop.cu:304-318: GraphOutput[tids_to_jobids[t]] = ret[t] */
  const int *t2j;
  or_sched_tids_to_jobids(c.s, &t2j);
  ORF(scatter_rows)(c.GO, H, t2j, c.ret, H, N, H);
  if (graph_out) memcpy(graph_out, c.GO, sizeof(real) * (size_t)N * H);
  if (msg_pool) memcpy(msg_pool, c.pool, sizeof(real) * (size_t)N * mw);

  /* ---- loss head ---- */
  if (cfg->loss == OR_LOSS_SOFTMAX) {
    int C = cfg->C;
    real *logits = zalloc((size_t)N * C), *dlogits = zalloc((size_t)N * C);
    /* FullyConnected: X*W^T then + ones*b, op_impl_fullyconnected_cublas.cc:71-79 */
    ORF(sgemm)(0, 1, N, C, H, 1.f, c.GO, H, p->Wfc, H, 0.f, logits, C);
    for (int r = 0; r < N; r++)
      for (int j = 0; j < C; j++) logits[(size_t)r * C + j] += p->bfc[j];
    ORF(softmax_xent)(loss_rows, dlogits, logits, labels, N, C);
    if (g) {
      /* FullyConnected_grad, op_impl_fullyconnected_cublas.cc:150-163 */
      ORF(sgemm)(1, 0, C, H, N, 1.f, dlogits, C, c.GO, H, 0.f, g->dWfc, H);
      ORF(colsum)(g->dbfc, dlogits, C, N, C, 0);
      ORF(sgemm)(0, 0, N, H, C, 1.f, dlogits, C, p->Wfc, H, 0.f, c.dGO, H);
    }
    free(logits);
    free(dlogits);
  } else if (cfg->loss == OR_LOSS_ROOT_SQ) {
    real acc = 0.f;
    for (int i = 0; i < B; i++) {
      const int *row = graph + (size_t)i * maxlen;
      int k = 0;
      while (row[k] != -1) k++;
      /* the root is the vertex whose parent entry is -1: the sample's last one */
      int gid = 0;
      for (int q = 0; q < i; q++) {
        const int *rq = graph + (size_t)q * maxlen;
        int kk = 0;
        while (rq[kk] != -1) kk++;
        gid += kk + 1;
      }
      gid += k;
      for (int j = 0; j < H; j++) {
        real h = c.GO[(size_t)gid * H + j];
        acc += h * h;
        c.dGO[(size_t)gid * H + j] = 2.f * h;
      }
    }
    if (loss_rows) loss_rows[0] = acc;
  } else {
    real acc = 0.f;
    for (size_t k = 0; k < (size_t)N * H; k++) {
      acc += R_FABS(c.GO[k]);
      c.dGO[k] = 1.f;
    }
    if (loss_rows) loss_rows[0] = acc;
  }
  if (dgraph_out) memcpy(dgraph_out, c.dGO, sizeof(real) * (size_t)N * H);

  /* ---- backward: statement.cc:87-123 ---- */
  if (g) {
    if (!fc) {
      memset(g->dEmb, 0, sizeof(real) * (size_t)cfg->V * E);
      memset(g->dBv, 0, sizeof(real) * (size_t)4 * H);
    } else if (cfg->use_bias) {
      memset(g->dBv, 0, sizeof(real) * (size_t)H);
    }
    if (cfg->model == OR_MODEL_TREELSTM || cfg->model == OR_MODEL_TREELSTM2) {
      memset(g->dW, 0, sizeof(real) * (size_t)E * 4 * H);
      memset(g->dU, 0, sizeof(real) * (size_t)(cfg->model == OR_MODEL_TREELSTM2 ? 5 : 4) * H * H);
    } else if (cfg->model == OR_MODEL_LSTM) {
      memset(g->dW, 0, sizeof(real) * (size_t)8 * H * H);
    } else {
      memset(g->dW, 0, sizeof(real) * (size_t)2 * H * H);
    }
    or_sched_reverse_graph(c.s);
    or_sched_initialize(c.s);
    while (!or_sched_terminate(c.s)) {
      bwd_round(&c);
      or_sched_activate_next(c.s);
    }
    if (cfg->batching) weight_grads(&c, 0, N);
  }

  real *all[] = {c.pool, c.dpool, c.G, c.dG, c.msg, c.dmsg, c.ret, c.dret, c.GO, c.dGO, c.xs,
                  c.e, c.de, c.xW, c.dxW, c.gates, c.z, c.hlr, c.dhlr, c.hU, c.hUf, c.dF, c.dhf, c.bias};
  for (size_t i = 0; i < sizeof all / sizeof all[0]; i++) free(all[i]);
  or_sched_free(c.s);
  return N;
}
