/*
 * Test infrastructure: CPU restatement of the op kernels on the F-over-G path.
 * Plain loops, fp32 throughout (as the reference computes).  Not linked into
 * the shipped library.
 */
#include "cavs_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>

/* cavs/backend/functor_batched_memcpy.cuh:33-46 */
void or_gather_rows(float *out, int ld_out, const float *inp, int ld_inp, const int *ids,
                    int n, int w) {
  for (int b = 0; b < n; b++)
    memcpy(out + (size_t)b * ld_out, inp + (size_t)ids[b] * ld_inp, sizeof(float) * (size_t)w);
}

/* cavs/backend/functor_batched_memcpy.cuh:48-61 */
void or_scatter_rows(float *out, int ld_out, const int *ids, const float *inp, int ld_inp,
                     int n, int w) {
  for (int b = 0; b < n; b++)
    memcpy(out + (size_t)ids[b] * ld_out, inp + (size_t)b * ld_inp, sizeof(float) * (size_t)w);
}

/* cavs/backend/functor_batched_memcpy.cuh:63-75 (the id list is not read) */
void or_zero_rows(float *out, int ld_out, int n, int w) {
  for (int b = 0; b < n; b++) memset(out + (size_t)b * ld_out, 0, sizeof(float) * (size_t)w);
}

/* cavs/backend/functor_batched_memcpy.cuh:18-31 */
void or_copy_rows(float *out, int ld_out, const float *inp, int ld_inp, int n, int w) {
  for (int b = 0; b < n; b++)
    memcpy(out + (size_t)b * ld_out, inp + (size_t)b * ld_inp, sizeof(float) * (size_t)w);
}

/* Row-major C[M,N] = alpha*op(A)*op(B) + beta*C.  The reference obtains this from
 * column-major cublasSgemm by swapping the operands (cublas_wrapper.cc:12-28);
 * the result is the plain row-major product restated here. */
void or_sgemm(int tA, int tB, int M, int N, int K, float alpha, const float *A, int lda,
              const float *B, int ldb, float beta, float *C, int ldc) {
#pragma omp parallel for schedule(static)
  for (int i = 0; i < M; i++) {
    float *c = C + (size_t)i * ldc;
    if (beta == 0.f)
      for (int j = 0; j < N; j++) c[j] = 0.f;
    else if (beta != 1.f)
      for (int j = 0; j < N; j++) c[j] *= beta;
    if (!tB) {
      for (int k = 0; k < K; k++) {
        float a = alpha * (tA ? A[(size_t)k * lda + i] : A[(size_t)i * lda + k]);
        const float *b = B + (size_t)k * ldb;
        for (int j = 0; j < N; j++) c[j] += a * b[j];
      }
    } else {
      for (int j = 0; j < N; j++) {
        const float *b = B + (size_t)j * ldb;
        float acc = 0.f;
        if (!tA) {
          const float *a = A + (size_t)i * lda;
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
void or_colsum(float *out, const float *inp, int ld, int n, int w, int accumulate) {
  for (int j = 0; j < w; j++) {
    float acc = 0.f;
    for (int r = 0; r < n; r++) acc += inp[(size_t)r * ld + j];
    out[j] = accumulate ? out[j] + acc : acc;
  }
}

/* cavs/backend/op_impl_embedding_lookup.cu:22-35: the element offset is the float
 * product id*E truncated to int. */
void or_embed_fwd(float *out, int ld_out, const float *ids, const float *table, int n, int E) {
  for (int b = 0; b < n; b++) {
    int off = (int)(ids[b] * (float)E);
    memcpy(out + (size_t)b * ld_out, table + off, sizeof(float) * (size_t)E);
  }
}

/* cavs/backend/op_impl_embedding_lookup.cu:90-103 (atomicAdd; order-free up to rounding) */
void or_embed_bwd(float *dtable, const float *ids, const float *dy, int ld_dy, int n, int E) {
  for (int b = 0; b < n; b++) {
    int off = (int)(ids[b] * (float)E);
    for (int j = 0; j < E; j++) dtable[off + j] += dy[(size_t)b * ld_dy + j];
  }
}

/* cavs/backend/op_impl_softmax_entropy_logits_loss.cu:94-140,212-250.  cuDNN's
 * SOFTMAX_ACCURATE subtracts the row maximum before exponentiating. */
void or_softmax_xent(float *loss, float *dlogits, const float *logits, const float *labels,
                     int n, int C) {
  float *p = (float *)malloc(sizeof(float) * (size_t)C);
  for (int r = 0; r < n; r++) {
    const float *x = logits + (size_t)r * C;
    float mx = x[0];
    for (int j = 1; j < C; j++) mx = x[j] > mx ? x[j] : mx;
    float sum = 0.f;
    for (int j = 0; j < C; j++) {
      p[j] = expf(x[j] - mx);
      sum += p[j];
    }
    for (int j = 0; j < C; j++) p[j] /= sum;
    int lab = (int)labels[r];
    if (loss) loss[r] = -logf(p[lab]);
    if (dlogits)
      for (int j = 0; j < C; j++)
        dlogits[(size_t)r * C + j] = ((j == lab) ? p[j] - 1.f : p[j]) * (1.f / (float)n);
  }
  free(p);
}

void or_sgd(float *w, const float *g, float lr, long n) {
  for (long i = 0; i < n; i++) w[i] -= lr * g[i];
}

/* cuDNN activation forward formulas, cavs/backend/op_impl_activation_cudnn.cu:57-87;
 * same formulas as the fusion generator, runtime_compiler/expression.h:40-71. */
static inline float sigm(float x) { return 1.f / (1.f + expf(-x)); }

void or_treelstm_gates_fwd(const float *xW, int ld_xw, const float *hU, const float *hUf,
                           const float *G, const float *bias, float *gates, float *msg,
                           int n, int H) {
  const float *b_i = bias, *b_f = bias + H, *b_u = bias + 2 * H, *b_o = bias + 3 * H;
  for (int r = 0; r < n; r++) {
    const float *xw = xW + (size_t)r * ld_xw, *hu = hU + (size_t)r * 3 * H;
    const float *fl = hUf + (size_t)(2 * r) * H, *fr = hUf + (size_t)(2 * r + 1) * H;
    const float *cl = G + (size_t)(2 * r) * 2 * H + H, *cr = G + (size_t)(2 * r + 1) * 2 * H + H;
    float *g = gates + (size_t)r * 6 * H, *m = msg + (size_t)r * 2 * H;
    for (int j = 0; j < H; j++) {
      /* tree-lstm-cavs.cc:160-165; Add is left-associative: (xW + hU) + b */
      float i = sigm((xw[j] + hu[j]) + b_i[j]);
      float o = sigm((xw[H + j] + hu[H + j]) + b_o[j]);
      float u = tanhf((xw[2 * H + j] + hu[2 * H + j]) + b_u[j]);
      float f_l = sigm((xw[3 * H + j] + fl[j]) + b_f[j]);
      float f_r = sigm((xw[3 * H + j] + fr[j]) + b_f[j]);
      /* :167-168 : (i*u + f_l*c_l) + f_r*c_r */
      float c = (i * u + f_l * cl[j]) + f_r * cr[j];
      float tc = tanhf(c);
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

void or_treelstm_gates_bwd(const float *dmsg, const float *dret, const float *gates,
                           const float *G, float *dxW, int ld_dxw, float *dF, float *dG,
                           int n, int H) {
  for (int r = 0; r < n; r++) {
    const float *g = gates + (size_t)r * 6 * H;
    const float *dm = dmsg + (size_t)r * 2 * H, *dr = dret + (size_t)r * H;
    const float *cl = G + (size_t)(2 * r) * 2 * H + H, *cr = G + (size_t)(2 * r + 1) * 2 * H + H;
    float *dx = dxW + (size_t)r * ld_dxw;
    float *dfl = dF + (size_t)(2 * r) * H, *dfr = dF + (size_t)(2 * r + 1) * H;
    float *dcl = dG + (size_t)(2 * r) * 2 * H + H, *dcr = dG + (size_t)(2 * r + 1) * 2 * H + H;
    for (int j = 0; j < H; j++) {
      float i = g[j], o = g[H + j], u = g[2 * H + j], f_l = g[3 * H + j], f_r = g[4 * H + j],
            tc = g[5 * H + j];
      float dh = dm[j] + dr[j];                     /* Mirror of h: Accumulate */
      float d_o = dh * tc;                          /* Mul grad */
      float dc = dm[H + j] + (dh * o) * (1.f - tc * tc); /* Mirror of c + tanh' */
      float d_i = dc * u, d_u = dc * i;
      float d_fl = dc * cl[j], d_fr = dc * cr[j];
      dcl[j] = dc * f_l;
      dcr[j] = dc * f_r;
      /* cudnn activation backward, op_impl_activation_cudnn.cu:101-139 */
      float del_i = d_i * (i * (1.f - i));
      float del_o = d_o * (o * (1.f - o));
      float del_u = d_u * (1.f - u * u);
      float del_fl = d_fl * (f_l * (1.f - f_l));
      float del_fr = d_fr * (f_r * (1.f - f_r));
      dx[j] = del_i;
      dx[H + j] = del_o;
      dx[2 * H + j] = del_u;
      dx[3 * H + j] = del_fl + del_fr;
      dfl[j] = del_fl;
      dfr[j] = del_fr;
    }
  }
}

void or_lstm_gates_fwd(const float *a, int ld_a, const float *G, const float *bias,
                       float *gates, float *msg, int n, int H) {
  for (int r = 0; r < n; r++) {
    const float *x = a + (size_t)r * ld_a, *cp = G + (size_t)r * 2 * H + H;
    float *g = gates + (size_t)r * 5 * H, *m = msg + (size_t)r * 2 * H;
    for (int j = 0; j < H; j++) {
      /* seq-lstm-cavs.cc:76-79 */
      float i = sigm(x[j] + bias[j]);
      float f = sigm(x[H + j] + bias[H + j]);
      float u = tanhf(x[2 * H + j] + bias[2 * H + j]);
      float o = sigm(x[3 * H + j] + bias[3 * H + j]);
      float c = i * u + f * cp[j]; /* :81 */
      float tc = tanhf(c);
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

void or_lstm_gates_bwd(const float *dmsg, const float *dret, const float *gates,
                       const float *G, float *da, int ld_da, float *dG, int n, int H) {
  for (int r = 0; r < n; r++) {
    const float *g = gates + (size_t)r * 5 * H;
    const float *dm = dmsg + (size_t)r * 2 * H, *dr = dret + (size_t)r * H;
    const float *cp = G + (size_t)r * 2 * H + H;
    float *d = da + (size_t)r * ld_da, *dcp = dG + (size_t)r * 2 * H + H;
    for (int j = 0; j < H; j++) {
      float i = g[j], f = g[H + j], u = g[2 * H + j], o = g[3 * H + j], tc = g[4 * H + j];
      float dh = dm[j] + dr[j];
      float d_o = dh * tc;
      float dc = dm[H + j] + (dh * o) * (1.f - tc * tc);
      d[j] = (dc * u) * (i * (1.f - i));
      d[H + j] = (dc * cp[j]) * (f * (1.f - f));
      d[2 * H + j] = (dc * i) * (1.f - u * u);
      d[3 * H + j] = d_o * (o * (1.f - o));
      dcp[j] = dc * f;
    }
  }
}

void or_treefc_fwd(const float *z, const float *bias, const float *x, float *h, int n, int H,
                   int act) {
  for (int r = 0; r < n; r++)
    for (int j = 0; j < H; j++) {
      float v = z[(size_t)r * H + j];
      if (bias) v += bias[j];
      if (x) v += x[(size_t)r * H + j];
      h[(size_t)r * H + j] = act ? tanhf(v) : (v > 0.f ? v : 0.f);
    }
}

void or_treefc_bwd(const float *dh_m, const float *dret, const float *h, float *dz, int n,
                   int H, int act) {
  for (size_t k = 0; k < (size_t)n * H; k++) {
    float dh = dh_m[k] + dret[k];
    float y = h[k];
    dz[k] = act ? dh * (1.f - y * y) : (y > 0.f ? dh : 0.f);
  }
}
