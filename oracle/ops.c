/*
 * Test infrastructure: CPU restatement of the op kernels on the F-over-G path.
 * Plain loops in `real`: fp32 throughout as the reference computes (or_*), or the
 * same operations in double (ord_*, -DOR_F64).  Not linked into the shipped library.
 */
#include "cavs_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>

/* cavs/backend/functor_batched_memcpy.cuh:33-46 */
void ORF(gather_rows)(real *out, int ld_out, const real *inp, int ld_inp, const int *ids,
                    int n, int w) {
  for (int b = 0; b < n; b++)
    memcpy(out + (size_t)b * ld_out, inp + (size_t)ids[b] * ld_inp, sizeof(real) * (size_t)w);
}

/* cavs/backend/functor_batched_memcpy.cuh:48-61 */
void ORF(scatter_rows)(real *out, int ld_out, const int *ids, const real *inp, int ld_inp,
                     int n, int w) {
  for (int b = 0; b < n; b++)
    memcpy(out + (size_t)ids[b] * ld_out, inp + (size_t)b * ld_inp, sizeof(real) * (size_t)w);
}

/* cavs/backend/functor_batched_memcpy.cuh:63-75 (the id list is not read) */
void ORF(zero_rows)(real *out, int ld_out, int n, int w) {
  for (int b = 0; b < n; b++) memset(out + (size_t)b * ld_out, 0, sizeof(real) * (size_t)w);
}

/* cavs/backend/functor_batched_memcpy.cuh:18-31 */
void ORF(copy_rows)(real *out, int ld_out, const real *inp, int ld_inp, int n, int w) {
  for (int b = 0; b < n; b++)
    memcpy(out + (size_t)b * ld_out, inp + (size_t)b * ld_inp, sizeof(real) * (size_t)w);
}

/* Row-major C[M,N] = alpha*op(A)*op(B) + beta*C.  The reference obtains this from
 * column-major cublasSgemm by swapping the operands (cublas_wrapper.cc:12-28);
 * the result is the plain row-major product restated here. */
void ORF(sgemm)(int tA, int tB, int M, int N, int K, real alpha, const real *A, int lda,
              const real *B, int ldb, real beta, real *C, int ldc) {
#pragma omp parallel for schedule(static)
  for (int i = 0; i < M; i++) {
    real *c = C + (size_t)i * ldc;
    if (beta == 0.f)
      for (int j = 0; j < N; j++) c[j] = 0.f;
    else if (beta != 1.f)
      for (int j = 0; j < N; j++) c[j] *= beta;
    if (!tB) {
      for (int k = 0; k < K; k++) {
        real a = alpha * (tA ? A[(size_t)k * lda + i] : A[(size_t)i * lda + k]);
        const real *b = B + (size_t)k * ldb;
        for (int j = 0; j < N; j++) c[j] += a * b[j];
      }
    } else {
      for (int j = 0; j < N; j++) {
        const real *b = B + (size_t)j * ldb;
        real acc = 0.f;
        if (!tA) {
          const real *a = A + (size_t)i * lda;
          for (int k = 0; k < K; k++) acc += a[k] * b[k];
        } else {
          for (int k = 0; k < K; k++) acc += A[(size_t)k * lda + i] * b[k];
        }
        c[j] += alpha * acc;
      }
    }
  }
}

/* cavs/backend/op_impl_elementwise.cuh:24-34: out[i] = sum_j inp[i + j*n_out],
 * rows added in ascending order. */
void ORF(colsum)(real *out, const real *inp, int ld, int n, int w, int accumulate) {
  for (int j = 0; j < w; j++) {
    real acc = 0.f;
    for (int r = 0; r < n; r++) acc += inp[(size_t)r * ld + j];
    out[j] = accumulate ? out[j] + acc : acc;
  }
}

/* cavs/backend/op_impl_embedding_lookup.cu:22-35: the element offset is the
 * floating-point product id*E truncated to int (exact in either precision for every
 * id and width the configurations use). */
void ORF(embed_fwd)(real *out, int ld_out, const real *ids, const real *table, int n, int E) {
  for (int b = 0; b < n; b++) {
    int off = (int)(ids[b] * (real)E);
    memcpy(out + (size_t)b * ld_out, table + off, sizeof(real) * (size_t)E);
  }
}

/* cavs/backend/op_impl_embedding_lookup.cu:90-103 (atomicAdd; order-free up to rounding) */
void ORF(embed_bwd)(real *dtable, const real *ids, const real *dy, int ld_dy, int n, int E) {
  for (int b = 0; b < n; b++) {
    int off = (int)(ids[b] * (real)E);
    for (int j = 0; j < E; j++) dtable[off + j] += dy[(size_t)b * ld_dy + j];
  }
}

/* cavs/backend/op_impl_softmax_entropy_logits_loss.cu:94-140,212-250.  cuDNN's
 * SOFTMAX_ACCURATE subtracts the row maximum before exponentiating. */
void ORF(softmax_xent)(real *loss, real *dlogits, const real *logits, const real *labels,
                     int n, int C) {
  real *p = (real *)malloc(sizeof(real) * (size_t)C);
  for (int r = 0; r < n; r++) {
    const real *x = logits + (size_t)r * C;
    real mx = x[0];
    for (int j = 1; j < C; j++) mx = x[j] > mx ? x[j] : mx;
    real sum = 0.f;
    for (int j = 0; j < C; j++) {
      p[j] = R_EXP(x[j] - mx);
      sum += p[j];
    }
    for (int j = 0; j < C; j++) p[j] /= sum;
    int lab = (int)labels[r];
    if (loss) loss[r] = -R_LOG(p[lab]);
    if (dlogits)
      for (int j = 0; j < C; j++)
        dlogits[(size_t)r * C + j] = ((j == lab) ? p[j] - 1.f : p[j]) * (1.f / (real)n);
  }
  free(p);
}

void ORF(sgd)(real *w, const real *g, real lr, long n) {
  for (long i = 0; i < n; i++) w[i] -= lr * g[i];
}

/* cuDNN activation forward formulas, cavs/backend/op_impl_activation_cudnn.cu:57-87;
 * same formulas as the fusion generator, runtime_compiler/expression.h:40-71. */
static inline real sigm(real x) { return 1.f / (1.f + R_EXP(-x)); }

void ORF(treelstm_gates_fwd)(const real *xW, int ld_xw, const real *hU, const real *hUf,
                           const real *G, const real *bias, real *gates, real *msg,
                           int n, int H) {
  const real *b_i = bias, *b_f = bias + H, *b_u = bias + 2 * H, *b_o = bias + 3 * H;
  for (int r = 0; r < n; r++) {
    const real *xw = xW + (size_t)r * ld_xw, *hu = hU + (size_t)r * 3 * H;
    const real *fl = hUf + (size_t)(2 * r) * H, *fr = hUf + (size_t)(2 * r + 1) * H;
    const real *cl = G + (size_t)(2 * r) * 2 * H + H, *cr = G + (size_t)(2 * r + 1) * 2 * H + H;
    real *g = gates + (size_t)r * 6 * H, *m = msg + (size_t)r * 2 * H;
    for (int j = 0; j < H; j++) {
      /* tree-lstm-cavs.cc:160-165; Add is left-associative: (xW + hU) + b */
      real i = sigm((xw[j] + hu[j]) + b_i[j]);
      real o = sigm((xw[H + j] + hu[H + j]) + b_o[j]);
      real u = R_TANH((xw[2 * H + j] + hu[2 * H + j]) + b_u[j]);
      real f_l = sigm((xw[3 * H + j] + fl[j]) + b_f[j]);
      real f_r = sigm((xw[3 * H + j] + fr[j]) + b_f[j]);
      /* :167-168 : (i*u + f_l*c_l) + f_r*c_r */
      real c = (i * u + f_l * cl[j]) + f_r * cr[j];
      real tc = R_TANH(c);
      g[j] = i;
      g[H + j] = o;
      g[2 * H + j] = u;
      g[3 * H + j] = f_l;
      g[4 * H + j] = f_r;
      g[5 * H + j] = tc;
      m[j] = o * tc;
      m[H + j] = c;
    }
  }
}

void ORF(treelstm_gates_bwd)(const real *dmsg, const real *dret, const real *gates,
                           const real *G, real *dxW, int ld_dxw, real *dF, real *dG,
                           int n, int H) {
  for (int r = 0; r < n; r++) {
    const real *g = gates + (size_t)r * 6 * H;
    const real *dm = dmsg + (size_t)r * 2 * H, *dr = dret + (size_t)r * H;
    const real *cl = G + (size_t)(2 * r) * 2 * H + H, *cr = G + (size_t)(2 * r + 1) * 2 * H + H;
    real *dx = dxW + (size_t)r * ld_dxw;
    real *dfl = dF + (size_t)(2 * r) * H, *dfr = dF + (size_t)(2 * r + 1) * H;
    real *dcl = dG + (size_t)(2 * r) * 2 * H + H, *dcr = dG + (size_t)(2 * r + 1) * 2 * H + H;
    for (int j = 0; j < H; j++) {
      real i = g[j], o = g[H + j], u = g[2 * H + j], f_l = g[3 * H + j], f_r = g[4 * H + j],
            tc = g[5 * H + j];
      real dh = dm[j] + dr[j];                     /* Mirror of h: Accumulate */
      real d_o = dh * tc;                          /* Mul grad */
      real dc = dm[H + j] + (dh * o) * (1.f - tc * tc); /* Mirror of c + tanh' */
      real d_i = dc * u, d_u = dc * i;
      real d_fl = dc * cl[j], d_fr = dc * cr[j];
      dcl[j] = dc * f_l;
      dcr[j] = dc * f_r;
      /* cudnn activation backward, op_impl_activation_cudnn.cu:101-139 */
      real del_i = d_i * (i * (1.f - i));
      real del_o = d_o * (o * (1.f - o));
      real del_u = d_u * (1.f - u * u);
      real del_fl = d_fl * (f_l * (1.f - f_l));
      real del_fr = d_fr * (f_r * (1.f - f_r));
      dx[j] = del_i;
      dx[H + j] = del_o;
      dx[2 * H + j] = del_u;
      dx[3 * H + j] = del_fl + del_fr;
      dfl[j] = del_fl;
      dfr[j] = del_fr;
    }
  }
}

void ORF(lstm_gates_fwd)(const real *a, int ld_a, const real *G, const real *bias,
                       real *gates, real *msg, int n, int H) {
  for (int r = 0; r < n; r++) {
    const real *x = a + (size_t)r * ld_a, *cp = G + (size_t)r * 2 * H + H;
    real *g = gates + (size_t)r * 5 * H, *m = msg + (size_t)r * 2 * H;
    for (int j = 0; j < H; j++) {
      /* seq-lstm-cavs.cc:76-79 */
      real i = sigm(x[j] + bias[j]);
      real f = sigm(x[H + j] + bias[H + j]);
      real u = R_TANH(x[2 * H + j] + bias[2 * H + j]);
      real o = sigm(x[3 * H + j] + bias[3 * H + j]);
      real c = i * u + f * cp[j]; /* :81 */
      real tc = R_TANH(c);
      g[j] = i;
      g[H + j] = f;
      g[2 * H + j] = u;
      g[3 * H + j] = o;
      g[4 * H + j] = tc;
      m[j] = o * tc;
      m[H + j] = c;
    }
  }
}

void ORF(lstm_gates_bwd)(const real *dmsg, const real *dret, const real *gates,
                       const real *G, real *da, int ld_da, real *dG, int n, int H) {
  for (int r = 0; r < n; r++) {
    const real *g = gates + (size_t)r * 5 * H;
    const real *dm = dmsg + (size_t)r * 2 * H, *dr = dret + (size_t)r * H;
    const real *cp = G + (size_t)r * 2 * H + H;
    real *d = da + (size_t)r * ld_da, *dcp = dG + (size_t)r * 2 * H + H;
    for (int j = 0; j < H; j++) {
      real i = g[j], f = g[H + j], u = g[2 * H + j], o = g[3 * H + j], tc = g[4 * H + j];
      real dh = dm[j] + dr[j];
      real d_o = dh * tc;
      real dc = dm[H + j] + (dh * o) * (1.f - tc * tc);
      d[j] = (dc * u) * (i * (1.f - i));
      d[H + j] = (dc * cp[j]) * (f * (1.f - f));
      d[2 * H + j] = (dc * i) * (1.f - u * u);
      d[3 * H + j] = d_o * (o * (1.f - o));
      dcp[j] = dc * f;
    }
  }
}

void ORF(treefc_fwd)(const real *z, const real *bias, const real *x, real *h, int n, int H,
                   int act) {
  for (int r = 0; r < n; r++)
    for (int j = 0; j < H; j++) {
      real v = z[(size_t)r * H + j];
      if (bias) v += bias[j];
      if (x) v += x[(size_t)r * H + j];
      h[(size_t)r * H + j] = act ? R_TANH(v) : (v > 0.f ? v : 0.f);
    }
}

void ORF(treefc_bwd)(const real *dh_m, const real *dret, const real *h, real *dz, int n,
                   int H, int act) {
  for (size_t k = 0; k < (size_t)n * H; k++) {
    real dh = dh_m[k] + dret[k];
    real y = h[k];
    dz[k] = act ? dh * (1.f - y * y) : (y > 0.f ? dh : 0.f);
  }
}
