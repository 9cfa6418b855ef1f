/*
 * Test infrastructure: CPU restatement of the reference's graph schedulers
 * (cavs/midend/graph_scheduler.{h,cc}).  Deliberately mirrors the reference's
 * state machine step by step, including which lists are moved, cleared or left
 * over between rounds, so the lists it exposes are the ones the reference's
 * Gather/Scatter/Pull ops would read.  Not linked into the shipped library.
 */
#include "cavs_oracle.h"

#include <stdlib.h>
#include <string.h>

typedef struct {
  int *v;
  int n, cap;
} ivec;

static void iv_push(ivec *a, int x) {
  if (a->n == a->cap) {
    a->cap = a->cap ? a->cap * 2 : 8;
    a->v = (int *)realloc(a->v, sizeof(int) * (size_t)a->cap);
  }
  a->v[a->n++] = x;
}
static void iv_clear(ivec *a) { a->n = 0; }
static void iv_free(ivec *a) {
  free(a->v);
  a->v = NULL;
  a->n = a->cap = 0;
}
static void iv_copy(ivec *dst, const ivec *src) {
  iv_clear(dst);
  for (int i = 0; i < src->n; i++) iv_push(dst, src->v[i]);
}
/* std::move of a vector: dst takes src's storage, src is left empty. */
static void iv_move(ivec *dst, ivec *src) {
  free(dst->v);
  *dst = *src;
  src->v = NULL;
  src->n = src->cap = 0;
}

/* a vector<vector<int>> with a run-time outer size (the reference builds the
 * next-round scatter lists with outer size 1 and the gather lists with 2). */
typedef struct {
  ivec l[2];
  int outer;
} ivec2;

static void iv2_move(ivec2 *dst, ivec2 *src) {
  for (int i = 0; i < 2; i++) iv_move(&dst->l[i], &src->l[i]);
  dst->outer = src->outer;
  src->outer = 0;
}
static void iv2_free(ivec2 *a) {
  iv_free(&a->l[0]);
  iv_free(&a->l[1]);
}

struct or_sched {
  int batching;
  int B, maxlen, N;
  int *sample_off;
  ivec *fwd_parents;  /* __forward_parents_ids_  */
  ivec *fwd_children; /* __forward_children_ids_ */
  ivec *parents, *children;
  int nslots; /* B*maxlen */
  int rc, forward;
  ivec ready;
  int *activated;
  ivec2 gather_init; /* tids_for_gather_init_ [0]=fwd [1]=bwd */
  ivec2 gather, scatter;
  int *j2t, *t2j;
  ivec round2offset;
  /* batch only */
  ivec *exec_tr;
  ivec2 *gather_tr, *scatter_tr;
  int ntr, captr;
  /* serial only */
  ivec pending; /* FIFO: [phead, n) */
  int phead, sample_id;
};

or_sched *or_sched_new(int batching) {
  or_sched *s = (or_sched *)calloc(1, sizeof(or_sched));
  s->batching = batching;
  s->rc = -1;
  s->forward = 1;
  s->gather_init.outer = s->gather.outer = s->scatter.outer = 2; /* graph_scheduler.h:16-18 */
  if (!batching) iv_push(&s->ready, 0); /* graph_scheduler.h:129: resize(1) */
  return s;
}

static void clear_tracers(or_sched *s) {
  for (int i = 0; i < s->ntr; i++) {
    iv_free(&s->exec_tr[i]);
    iv2_free(&s->gather_tr[i]);
    iv2_free(&s->scatter_tr[i]);
  }
  s->ntr = 0;
}

void or_sched_free(or_sched *s) {
  if (!s) return;
  for (int i = 0; i < s->nslots; i++) {
    iv_free(&s->fwd_parents[i]);
    iv_free(&s->fwd_children[i]);
  }
  free(s->fwd_parents);
  free(s->fwd_children);
  free(s->sample_off);
  free(s->activated);
  free(s->j2t);
  free(s->t2j);
  iv_free(&s->ready);
  iv2_free(&s->gather_init);
  iv2_free(&s->gather);
  iv2_free(&s->scatter);
  iv_free(&s->round2offset);
  clear_tracers(s);
  free(s->exec_tr);
  free(s->gather_tr);
  free(s->scatter_tr);
  iv_free(&s->pending);
  free(s);
}

/* cavs/midend/graph_scheduler.cc:12-71 */
int or_sched_load_graph(or_sched *s, const int *g, int B, int maxlen) {
  if (s->B == 0 && s->maxlen == 0) {
    s->B = B;
    s->maxlen = maxlen;
    s->nslots = B * maxlen;
    s->fwd_parents = (ivec *)calloc((size_t)s->nslots, sizeof(ivec));
    s->fwd_children = (ivec *)calloc((size_t)s->nslots, sizeof(ivec));
    s->sample_off = (int *)calloc((size_t)B, sizeof(int));
    /* vectors only ever grow to total_length <= B*maxlen; allocate the bound */
    s->activated = (int *)calloc((size_t)s->nslots, sizeof(int));
    s->j2t = (int *)calloc((size_t)s->nslots, sizeof(int));
    s->t2j = (int *)calloc((size_t)s->nslots, sizeof(int));
  } else {
    if (B != s->B || maxlen != s->maxlen) return -1; /* :25-26 CHECK */
    for (int i = 0; i < s->nslots; i++) {
      iv_clear(&s->fwd_parents[i]);
      iv_clear(&s->fwd_children[i]);
    }
  }
  s->N = 0;
  int prev = 0;
  for (int i = 0; i < B; i++) {
    const int *start = g + (size_t)i * maxlen;
    int k = 0;
    while (k < maxlen && start[k] != -1) k++;
    int len = k + 1; /* :39 find(-1)+1-start */
    s->sample_off[i] = prev + (i > 0 ? s->sample_off[i - 1] : 0);
    if (len > maxlen) return -2; /* :41 CHECK */
    s->N += len;
    int off = s->sample_off[i];
    for (int j = 0; j < len - 1; j++) iv_push(&s->fwd_parents[off + j], off + start[j]);
    for (int j = 0; j < len; j++)
      if (s->fwd_parents[off + j].n) iv_push(&s->fwd_children[s->fwd_parents[off + j].v[0]], off + j);
    prev = len;
  }
  s->parents = s->fwd_parents;
  s->children = s->fwd_children;
  iv_clear(&s->round2offset);
  s->rc = -1;
  s->forward = 1;
  return s->N;
}

/* cavs/midend/graph_scheduler.cc:73-81 */
int or_sched_reverse_graph(or_sched *s) {
  s->children = s->fwd_parents;
  s->parents = s->fwd_children;
  s->forward = 0;
  return s->N;
}

static void rc_inc(or_sched *s) { s->rc += s->forward ? 1 : -1; }

int or_sched_terminate(const or_sched *s) {
  if (s->batching) return s->ready.n == 0;
  return s->phead == s->pending.n;
}

int or_sched_round_offset(const or_sched *s) {
  if (s->batching) return s->round2offset.v[s->rc];
  return s->ready.v[0];
}

/* cavs/midend/graph_scheduler.cc:110-123 */
static void serial_init_sample(or_sched *s, int sid) {
  int end = (sid < s->B - 1) ? s->sample_off[sid + 1] : s->N;
  int len = end - s->sample_off[sid];
  for (int i = 0; i < len; i++) {
    int gid = s->sample_off[sid] + i;
    if (s->children[gid].n == 0 && s->parents[gid].n != 0) iv_push(&s->pending, gid);
  }
  s->sample_id = sid;
}

static void serial_lists(or_sched *s, int gid) {
  /* cavs/midend/graph_scheduler.cc:93-107 and :144-166 */
  iv_clear(&s->gather.l[0]);
  iv_clear(&s->gather.l[1]);
  iv_clear(&s->scatter.l[0]);
  iv_clear(&s->scatter.l[1]);
  if (s->forward) {
    for (int i = 0; i < s->parents[gid].n; i++) iv_push(&s->scatter.l[0], gid);
    if (s->children[gid].n == 0) {
      iv_clear(&s->gather_init.l[0]);
      iv_push(&s->gather_init.l[0], gid);
    }
  } else {
    for (int i = 0; i < s->parents[gid].n; i++) iv_push(&s->scatter.l[i], s->parents[gid].v[i]);
    if (s->children[gid].n == 0) {
      iv_clear(&s->gather_init.l[1]);
      iv_push(&s->gather_init.l[1], gid);
    }
  }
}

static void grow_tracers(or_sched *s) {
  if (s->ntr == s->captr) {
    int nc = s->captr ? s->captr * 2 : 16;
    s->exec_tr = (ivec *)realloc(s->exec_tr, sizeof(ivec) * (size_t)nc);
    s->gather_tr = (ivec2 *)realloc(s->gather_tr, sizeof(ivec2) * (size_t)nc);
    s->scatter_tr = (ivec2 *)realloc(s->scatter_tr, sizeof(ivec2) * (size_t)nc);
    memset(s->exec_tr + s->captr, 0, sizeof(ivec) * (size_t)(nc - s->captr));
    memset(s->gather_tr + s->captr, 0, sizeof(ivec2) * (size_t)(nc - s->captr));
    memset(s->scatter_tr + s->captr, 0, sizeof(ivec2) * (size_t)(nc - s->captr));
    s->captr = nc;
  }
}

void or_sched_initialize(or_sched *s) {
  rc_inc(s);
  memset(s->activated, 0, sizeof(int) * (size_t)s->N);
  if (!s->batching) {
    /* cavs/midend/graph_scheduler.cc:83-108 */
    iv_clear(&s->pending);
    s->phead = 0;
    serial_init_sample(s, 0);
    int gid = s->pending.v[s->phead];
    s->ready.v[0] = gid;
    s->t2j[gid] = gid;
    /* Initialize (unlike ActivateNext) fills no gather list for the first
     * vertex: in forward it is a leaf, in backward gather lists are counts. */
    serial_lists(s, gid);
    return;
  }
  /* cavs/midend/graph_scheduler.cc:169-200 */
  if (s->round2offset.n == 0) iv_push(&s->round2offset, 0);
  if (s->forward) {
    for (int gid = 0; gid < s->N; gid++) {
      if (s->children[gid].n == 0 && s->parents[gid].n != 0) {
        int tid = or_sched_round_offset(s) + s->ready.n;
        s->t2j[tid] = gid;
        s->j2t[gid] = tid;
        iv_push(&s->scatter.l[0], tid); /* appended without clearing, :184 */
        iv_push(&s->ready, gid);
      }
    }
    iv_copy(&s->gather_init.l[0], &s->ready);
    iv_clear(&s->gather_init.l[1]);
    clear_tracers(s);
  } else {
    iv_move(&s->ready, &s->exec_tr[s->rc]);
    iv2_move(&s->gather, &s->scatter_tr[s->rc]);
    iv2_move(&s->scatter, &s->gather_tr[s->rc]);
  }
}

void or_sched_activate_next(or_sched *s) {
  if (!s->batching) {
    /* cavs/midend/graph_scheduler.cc:125-167 */
    rc_inc(s);
    int gid = s->pending.v[s->phead];
    if (s->parents[gid].n) {
      for (int k = 0; k < s->parents[gid].n; k++) {
        int pid = s->parents[gid].v[k];
        if (++s->activated[pid] == s->children[pid].n) iv_push(&s->pending, pid);
      }
    } else if (++s->sample_id < s->B) {
      serial_init_sample(s, s->sample_id);
    }
    s->t2j[gid] = gid;
    s->phead++;
    if (or_sched_terminate(s)) return;
    int next = s->pending.v[s->phead];
    s->ready.v[0] = next;
    serial_lists(s, next);
    if (s->forward) {
      for (int i = 0; i < s->children[next].n; i++) iv_push(&s->gather.l[i], s->children[next].v[i]);
    } else {
      for (int i = 0; i < s->children[next].n; i++) iv_push(&s->gather.l[0], next);
    }
    return;
  }
  /* cavs/midend/graph_scheduler.cc:202-258 */
  rc_inc(s);
  if (s->rc >= 0 && s->round2offset.n <= s->rc)
    iv_push(&s->round2offset, s->round2offset.v[s->round2offset.n - 1] + s->ready.n);
  if (s->forward) {
    ivec jobs = {0, 0, 0};
    ivec2 gnext, snext;
    memset(&gnext, 0, sizeof gnext);
    memset(&snext, 0, sizeof snext);
    gnext.outer = 2;
    snext.outer = 1;
    for (int a = 0; a < s->ready.n; a++) {
      int gid = s->ready.v[a];
      for (int k = 0; k < s->parents[gid].n; k++) {
        int pid = s->parents[gid].v[k];
        if (++s->activated[pid] == s->children[pid].n) {
          int tid = or_sched_round_offset(s) + jobs.n;
          s->t2j[tid] = pid;
          s->j2t[pid] = tid;
          iv_push(&jobs, pid);
          for (int i = 0; i < s->children[pid].n && i < 2; i++)
            iv_push(&gnext.l[i], s->j2t[s->children[pid].v[i]]);
          if (s->parents[pid].n == 0)
            iv_push(&s->gather_init.l[1], tid);
          else
            for (int i = 0; i < s->parents[pid].n; i++) iv_push(&snext.l[0], tid);
        }
      }
    }
    grow_tracers(s);
    iv_move(&s->exec_tr[s->ntr], &s->ready);
    iv2_move(&s->gather_tr[s->ntr], &s->gather);
    iv2_move(&s->scatter_tr[s->ntr], &s->scatter);
    s->ntr++;
    iv_move(&s->ready, &jobs);
    iv2_move(&s->gather, &gnext);
    iv2_move(&s->scatter, &snext);
  } else {
    if (s->rc >= 0) {
      iv_move(&s->ready, &s->exec_tr[s->rc]);
      iv2_move(&s->gather, &s->scatter_tr[s->rc]);
      iv2_move(&s->scatter, &s->gather_tr[s->rc]);
    } else {
      iv_clear(&s->ready);
      iv_clear(&s->gather.l[0]);
      iv_clear(&s->gather.l[1]);
      iv_clear(&s->scatter.l[0]);
      iv_clear(&s->scatter.l[1]);
    }
  }
}

int or_sched_total_length(const or_sched *s) { return s->N; }
int or_sched_is_forward(const or_sched *s) { return s->forward; }
int or_sched_job_ids(const or_sched *s, const int **p) {
  *p = s->ready.v;
  return s->ready.n;
}
int or_sched_gather_ids(const or_sched *s, int c, const int **p) {
  *p = s->gather.l[c].v;
  return s->gather.l[c].n;
}
int or_sched_scatter_ids(const or_sched *s, int c, const int **p) {
  *p = s->scatter.l[c].v;
  return s->scatter.l[c].n;
}
int or_sched_gather_init_ids(const or_sched *s, const int **p) {
  const ivec *v = &s->gather_init.l[s->forward ? 0 : 1];
  *p = v->v;
  return v->n;
}
int or_sched_tids_to_jobids(const or_sched *s, const int **p) {
  *p = s->t2j;
  return s->N;
}
int or_sched_round2offset(const or_sched *s, const int **p) {
  *p = s->round2offset.v;
  return s->round2offset.n;
}

/* ---- trace serialisation for the tests ---- */
typedef struct {
  int *out;
  int cap, n;
} sink;
static void put(sink *k, int x) {
  if (k->n < k->cap) k->out[k->n] = x;
  k->n++;
}
static void put_list(sink *k, const int *p, int n) {
  put(k, n);
  for (int i = 0; i < n; i++) put(k, p[i]);
}
static int dump_rounds(or_sched *s, sink *k) {
  int rounds = 0;
  const int *p;
  while (!or_sched_terminate(s)) {
    put(k, or_sched_round_offset(s));
    int n = or_sched_job_ids(s, &p);
    put_list(k, p, n);
    for (int c = 0; c < 2; c++) {
      n = or_sched_gather_ids(s, c, &p);
      put_list(k, p, n);
    }
    for (int c = 0; c < 2; c++) {
      n = or_sched_scatter_ids(s, c, &p);
      put_list(k, p, n);
    }
    n = or_sched_gather_init_ids(s, &p);
    put_list(k, p, n);
    or_sched_activate_next(s);
    rounds++;
  }
  return rounds;
}

int or_sched_trace(const int *g, int B, int maxlen, int batching, int with_backward,
                   int *out, int cap) {
  or_sched *s = or_sched_new(batching);
  sink k = {out, cap, 0};
  int N = or_sched_load_graph(s, g, B, maxlen);
  if (N < 0) {
    or_sched_free(s);
    return 0;
  }
  put(&k, N);
  put(&k, 0);
  put(&k, 0);
  or_sched_initialize(s);
  int rf = dump_rounds(s, &k), rb = 0;
  if (with_backward) {
    or_sched_reverse_graph(s);
    or_sched_initialize(s);
    rb = dump_rounds(s, &k);
  }
  if (cap > 2) {
    out[1] = rf;
    out[2] = rb;
  }
  const int *p;
  int n = or_sched_tids_to_jobids(s, &p);
  for (int i = 0; i < n; i++) put(&k, p[i]);
  n = or_sched_round2offset(s, &p);
  put_list(&k, p, n);
  or_sched_free(s);
  return k.n <= cap ? k.n : -k.n;
}
